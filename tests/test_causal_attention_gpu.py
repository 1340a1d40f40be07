"""The causal builders and the native causal predicate of flash_attention describe the same attention.

Follows the reference's test of native causal lengths against the compact mask with padding
(test/cases/test_relative_flash_attention.py:292-386, plain flash attention): same outputs and same gradients,
for fp32 (generic kernels) and bf16 at sbs 64 (matrix-core kernels), and against dense torch attention."""

import pytest
import torch

import blksprs_amd as bs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,sbs,tol", [(torch.float32, 16, 1e-5), (torch.float32, 32, 1e-5),
                                           (torch.bfloat16, 64, 2e-2), (torch.float16, 64, 2e-2)])
@pytest.mark.parametrize("lengths_in_blocks", [(1.3,), (2.0, 0.4, 1.7)])
def test_native_causal_lengths_match_the_compact_mask_with_padding(device, dtype, sbs, tol, lengths_in_blocks):
    torch.manual_seed(15)
    lengths = [max(1, int(f * sbs)) for f in lengths_in_blocks]
    B = len(lengths)
    valid = torch.tensor(lengths, device=device)
    attention_layout = bs.layouting.build_causal_self_attention_layout(valid, sbs)
    n = attention_layout.size(1)
    padded = n * sbs
    mask, mask_layout = bs.layouting.build_causal_self_attention_mask(valid, attention_layout, sbs)
    feature_layout = torch.ones((B, n, 1), dtype=torch.bool, device=device)
    dense = [torch.randn((B, padded, sbs), device=device, dtype=dtype, requires_grad=True) for _ in range(3)]
    twin = [t.detach().clone().requires_grad_(True) for t in dense]

    def run(inputs, native):
        q, k, v = (bs.ops.to_sparse(t, feature_layout, sbs) for t in inputs)
        kwargs = ({"causal_lengths": valid} if native
                  else {"attention_mask": mask, "sparsity_layout_mask": mask_layout})
        out = bs.ops.flash_attention(q, feature_layout, k, feature_layout, v, feature_layout, attention_layout, sbs,
                                     sparsity_layout_o=feature_layout, **kwargs)
        return bs.ops.to_dense(out, feature_layout, sbs)

    explicit = run(dense, native=False)
    native = run(twin, native=True)
    torch.testing.assert_close(native, explicit, rtol=tol, atol=tol)

    # dense torch attention on the valid prefix of every sequence; padding rows give zeros
    for b, length in enumerate(lengths):
        q, k, v = (t[b, :length].detach().float() for t in dense)
        scores = (q @ k.T) / sbs ** 0.5
        scores = scores.masked_fill(torch.triu(torch.ones_like(scores, dtype=torch.bool), 1), float("-inf"))
        want = torch.softmax(scores, -1) @ v
        torch.testing.assert_close(explicit[b, :length].float(), want, rtol=max(tol, 2e-5), atol=max(tol, 2e-5))
        assert torch.all(explicit[b, length:] == 0) and torch.all(native[b, length:] == 0)

    gradient = torch.randn_like(explicit)
    (explicit * gradient).sum().backward()
    (native * gradient).sum().backward()
    for a, b in zip(twin, dense):
        torch.testing.assert_close(a.grad, b.grad, rtol=2 * tol, atol=2 * tol)


def test_window_layout_and_mask_give_local_attention(device):
    """fp32, sbs 16, window of 16 tokens (it ends on a block boundary, so the compact mask is exact): equal to
    dense attention with the band mask."""
    sbs, window = 16, 17
    valid = torch.tensor([48, 37], device=device)
    layout = bs.layouting.build_causal_window_self_attention_layout(valid, sbs, window)
    mask, mask_layout = bs.layouting.build_causal_window_self_attention_mask(valid, layout, sbs, window)
    n = layout.size(1)
    feature_layout = torch.ones((2, n, 1), dtype=torch.bool, device=device)
    g = torch.Generator(device=device).manual_seed(3)
    q, k, v = (torch.randn((2, n * sbs, sbs), device=device, generator=g) for _ in range(3))
    sp = lambda t: bs.ops.to_sparse(t, feature_layout, sbs)
    out = bs.ops.to_dense(bs.ops.flash_attention(sp(q), feature_layout, sp(k), feature_layout, sp(v), feature_layout,
                                                 layout, sbs, attention_mask=mask, sparsity_layout_mask=mask_layout,
                                                 sparsity_layout_o=feature_layout), feature_layout, sbs)
    for b, length in enumerate(valid.tolist()):
        pos = torch.arange(length, device=device)
        banned = (pos[None, :] > pos[:, None]) | (pos[:, None] - pos[None, :] > window - 1)
        scores = (q[b, :length] @ k[b, :length].T) / sbs ** 0.5
        want = torch.softmax(scores.masked_fill(banned, float("-inf")), -1) @ v[b, :length]
        torch.testing.assert_close(out[b, :length], want, rtol=2e-5, atol=2e-5)


def test_range_check_of_causal_lengths_follows_changes_in_place(device):
    """The range check of ``causal_lengths`` (blksprs/ops/flash_attention.py:239-241) reads the device; its verdict
    on one tensor is remembered while the tensor's version counter stands still, and a change in place is checked
    again: a tensor that was valid and is then given a length beyond the sequence is refused."""
    sbs, n = 16, 3
    layout = torch.ones((1, n, 1), dtype=torch.bool, device=device)
    attention = torch.ones((1, n, n), dtype=torch.bool, device=device)
    q = torch.randn((n, sbs, sbs), device=device)
    lengths = torch.tensor([n * sbs], device=device)
    call = lambda: bs.ops.flash_attention(q, layout, q, layout, q, layout, attention, sbs, causal_lengths=lengths)
    first = call()
    assert torch.equal(call(), first)
    lengths.add_(1)
    with pytest.raises(ValueError, match="between zero and"):
        call()
    lengths.sub_(2 * sbs)
    shorter = call()
    assert torch.all(shorter[n - 1] == 0) and not torch.equal(shorter, first)
