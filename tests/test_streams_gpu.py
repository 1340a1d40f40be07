"""The operators run on torch's current stream, and warm operators can be captured into a HIP graph.

Every C entry point takes a stream; the Python layer hands it the current torch stream.  On a side stream an
operator must therefore see the result of the work queued there just before it (a launch on another stream would
race with it), and under graph capture its launches must land in the graph: replays with new input values give
the eager results.
"""

import pytest
import torch

import blksprs_amd as bs
from tests.helpers import rand_layout

pytestmark = pytest.mark.gpu


def _problem(device, dtype=torch.bfloat16, sbs=64):
    lx = rand_layout((2, 4, 5), 0.6, seed=1, ensure_rows=True).to(device)
    ly = rand_layout((2, 5, 3), 0.6, seed=2, ensure_rows=True).to(device)
    lo = bs.layouting.build_sparsity_layout_matmul(lx, ly)
    g = torch.Generator(device=device).manual_seed(3)
    x = (torch.randn((int(lx.sum()), sbs, sbs), device=device, generator=g) / 8).to(dtype)
    y = torch.randn((int(ly.sum()), sbs, sbs), device=device, generator=g).to(dtype)
    return lx, ly, lo, x, y


def test_operators_follow_the_current_stream(device):
    sbs = 64
    lx, ly, lo, x, y = _problem(device)
    la = rand_layout((2, 4, 4), 0.7, seed=4, ensure_rows=True).to(device)
    full = torch.ones((2, 4, 1), dtype=torch.bool, device=device)
    q = torch.randn((8, sbs, sbs), device=device).to(torch.bfloat16)
    caches = [{}, {}, {}, {}]

    def work(xin, qin):
        out = bs.ops.matmul(xin, lx, y, ly, lo, sbs, layout_cache=caches[0])
        soft = bs.ops.softmax(xin.float(), lx, sbs, layout_cache=caches[1])
        dense = bs.ops.to_dense(xin, lx, sbs, layout_cache=caches[2])
        qq = qin.clone().requires_grad_(True)
        att = bs.ops.flash_attention(qq, full, qin, full, qin, full, la, sbs, layout_cache=caches[3])
        att.float().square().sum().backward()
        return out, soft, dense, att.detach(), qq.grad

    expected = work(x, q)  # also warms the caches
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=device)
    big = torch.randn((4096, 4096), device=device)
    with torch.cuda.stream(side):
        # inputs that exist only once a long chain of work on this stream has finished
        acc = big
        for _ in range(8):
            acc = (acc @ big).clamp_(-1, 1)
        x_late = x + (acc[0, 0] * 0).to(x.dtype)
        q_late = q + (acc[0, 1] * 0).to(q.dtype)
        got = work(x_late, q_late)
    side.synchronize()
    for a, b in zip(got, expected):
        assert torch.equal(a, b)


def test_warm_operators_replay_from_a_graph(device):
    sbs = 64
    lx, ly, lo, x, y = _problem(device)
    caches = [{}, {}]
    x_static = x.clone()

    def work():
        out = bs.ops.matmul(x_static, lx, y, ly, lo, sbs, layout_cache=caches[0])
        return out, bs.ops.softmax(out.float(), lo, sbs, layout_cache=caches[1])

    bs.utils.disable_validation()  # value checks of layouts read the device; the layouts were checked above
    try:
        side = torch.cuda.Stream(device=device)
        with torch.cuda.stream(side):
            for _ in range(3):
                work()
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = work()
        for scale in (1.0, -0.5, 2.0):
            x_static.copy_(x * scale)
            graph.replay()
            torch.cuda.synchronize()
            replayed = [t.clone() for t in captured]
            eager = work()
            torch.cuda.synchronize()
            for a, b in zip(replayed, eager):
                assert torch.equal(a, b)
    finally:
        bs.utils.enable_validation()
