"""bsa_lut_packed_static (the layout scan with its scratch in a static device array) against bsa_lut_packed.

Called through the C ABI: two calls in a row on one device, the second with a smaller layout, so that what
the first call left in the shared array must not leak into the second; every output is compared bit for bit
with the workspace-taking entry point and with the numpy oracle.
"""

import numpy as np
import pytest
import torch

from blksprs_amd import _capi
from oracle import blksprs_oracle as orc

pytestmark = pytest.mark.gpu


def _scan(name, lay, row_len, dev):
    n = lay.numel()
    packed = torch.full((n,), -7, dtype=torch.int64, device=dev)
    n_rows = n // row_len if row_len else 0
    row_offsets = torch.full((n_rows + 1,), -7, dtype=torch.int32, device=dev)
    stats = torch.full((2,), -7, dtype=torch.int64, device=dev)
    stream = _capi.stream(dev)
    lib = _capi.load()
    if name == "bsa_lut_packed":
        ws_bytes = lib.bsa_lut_workspace_bytes(n)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        _capi.call(name, _capi.ptr(lay), n, row_len, _capi.ptr(packed), row_offsets.data_ptr() if row_len else 0,
                   stats.data_ptr(), 0, _capi.ptr(ws), ws_bytes, stream)
    else:
        _capi.call(name, _capi.ptr(lay), n, row_len, _capi.ptr(packed), row_offsets.data_ptr() if row_len else 0,
                   stats.data_ptr(), stream)
    torch.cuda.synchronize(dev)
    return packed, row_offsets, stats


def _layout(shape, density, seed, dev):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(shape, generator=g) < density).to(torch.uint8).to(dev)


def test_static_scratch_scan_equals_the_workspace_scan_on_two_calls_in_a_row(device):
    # first a layout of many tiles (C5's operand layout: 64 x 128 x 128 = 512 tiles of 2048), then a small ragged
    # one (3 tiles, the last partial), then an empty one
    cases = [((64, 128, 128), 0.05, 128), ((3, 37, 41), 0.4, 41), ((5, 11, 7), 0.0, 7)]
    for seed, (shape, density, row_len) in enumerate(cases):
        lay = _layout(shape, density, seed, device)
        got = _scan("bsa_lut_packed_static", lay, row_len, device)
        want = _scan("bsa_lut_packed", lay, row_len, device)
        for g, w in zip(got, want):
            assert torch.equal(g, w)
        ref = orc.packed_indices(lay.cpu().numpy())
        assert np.array_equal(got[0].cpu().numpy(), np.asarray(ref).reshape(-1))
        assert int(got[2][0]) == int(lay.sum())
        counts = lay.reshape(-1, row_len).sum(dim=1, dtype=torch.int64)
        assert int(got[2][1]) == int(counts.max())
        assert torch.equal(got[1][1:].long(), counts.cumsum(0))


def test_static_scratch_scan_without_row_offsets_and_size_limit(device):
    lay = _layout((2, 50, 60), 0.5, 11, device)
    got = _scan("bsa_lut_packed_static", lay, 0, device)
    want = _scan("bsa_lut_packed", lay, 0, device)
    assert torch.equal(got[0], want[0]) and torch.equal(got[2], want[2])
    lib = _capi.load()
    limit = lib.bsa_lut_packed_static_max_entries()
    assert limit == 1 << 24
    # one entry too many is refused on the host before anything is launched (the pointers are never read)
    rc = lib.bsa_lut_packed_static(0, limit + 1, 0, 0, 0, 0, 0)
    assert rc == -3 and b"exceed the static scratch" in lib.bsa_last_error()
