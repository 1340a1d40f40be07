"""Block-sparse flash attention on compressed tensors, forward and backward.

Signatures, validation order and messages, default scale, optional mask / bias /
output layout / native causal lengths and every observable cache key follow the
reference (blksprs/ops/flash_attention.py:19-242 wrapper and length normalisation,
:1736-1920 cache builder, :1923-1957 CSR metadata).  The arithmetic is done by
``bsa_attn_fwd`` / ``bsa_attn_bwd``; the learned relative-embedding branches of the
reference are not part of this package.
"""

import ctypes
import math
import threading
from numbers import Real

import torch
from torch import Tensor

from .. import _capi
from ..layouting.sparsity_layout import build_sparsity_layout_matmul
from ..utils.blksprs_tensor import BlksprsTensor
from ..utils.tools import (CacheHolder, INT32_INDEX_MAX, as_base_tensor, cast_for_autocast, csr_indices_from_packed,
                           PackedLayout, eager_only, finalize_layout_cache, layout_bytes, pack_layout,
                           pack_layouts, prepare_layout_cache)
from ..utils.validation import (ensure_contiguous, kept_ds_limit, mask_facts_enabled, validate_binary, validate_contiguous,
                                validate_device, validate_dimensions, validate_dtype_float, validate_shape,
                                validate_sparsity, validate_sparsity_block_size, validate_sparsity_layout,
                                validation_enabled)

def _select_segmented_index_dtype(n_active_blocks: int, n_blocks_col: int) -> torch.dtype:
    """int32 unless the number of active blocks or the largest column id needs more."""
    if n_active_blocks > INT32_INDEX_MAX or n_blocks_col - 1 > INT32_INDEX_MAX:
        return torch.int64
    return torch.int32


def _build_segmented_indices(attention_layout: Tensor, n_batches: int, n_blocks_row: int,
                             n_blocks_col: int, info=None) -> tuple[Tensor, Tensor, int]:
    """CSR adjacency of a ``(B, rows, cols)`` layout: ``(indices, offsets, max_blocks_per_row)``.

    ``offsets`` has ``B * rows + 1`` entries with a leading 0, ``indices`` lists the active columns of each row
    in ascending order.  Empty and all-zero layouts yield ``(empty, zeros, 1)``.  ``info``: the layout's scan with
    row offsets (``pack_layouts``), when the caller has made it together with others.
    """
    device = attention_layout.device
    n_rows = n_batches * n_blocks_row
    if attention_layout.numel() == 0:
        return (torch.empty(0, dtype=torch.int32, device=device),
                torch.zeros(n_rows + 1, dtype=torch.int32, device=device), 1)
    if info is None:
        info = pack_layout(attention_layout, row_len=n_blocks_col)
    if info.max_per_row == 0:
        return (torch.empty(0, dtype=torch.int32, device=device),
                torch.zeros(n_rows + 1, dtype=torch.int32, device=device), 1)
    dtype = _select_segmented_index_dtype(info.count, n_blocks_col)
    indices = csr_indices_from_packed(info.packed, n_blocks_col, info.count)
    offsets = info.row_offsets
    if dtype != torch.int32:
        indices, offsets = indices.to(dtype), offsets.to(dtype)
    return as_base_tensor(indices), as_base_tensor(offsets), info.max_per_row


def _build_group_lists(attention_layout: Tensor, n_batches: int, n_blocks_row: int,
                       n_blocks_col: int, info=None) -> tuple[Tensor, Tensor, int]:
    """The attention layout as lists over pairs of neighbouring query blocks: ``(offsets, entries, group_size)``.

    A group is the pair of query blocks ``(2p, 2p+1)`` and its list the union of their key lists.  ``entries``
    holds ``key_block | active_for_first << 28 | active_for_second << 29`` (int32, key blocks ascending),
    ``offsets`` has ``B * ceil(rows / 2) + 1`` int32 entries.  The forward kernel gives a pair to one workgroup,
    which fetches a K / V block both query blocks need once.  These lists have no counterpart in the reference.
    """
    union = _group_union(attention_layout, n_batches, n_blocks_row, n_blocks_col)
    if info is None:
        info = pack_layout(union, row_len=n_blocks_col)
    entries = torch.empty(info.count, dtype=torch.int32, device=union.device)
    if info.count:
        lay = layout_bytes(attention_layout)
        with _capi.on_device(union.device):
            _capi.call("bsa_lut_pair_entries", lay.data_ptr(), info.packed.data_ptr(), n_batches, n_blocks_row,
                       n_blocks_col, entries.data_ptr(), _capi.stream(union.device))
    return as_base_tensor(info.row_offsets), entries, 2


def _grouped_lists_apply(n_blocks_col, n_head_blocks, n_head_blocks_v) -> bool:
    """Whether the matrix-core forward kernel's lists over pairs of query blocks can exist for these shapes (the
    block size, which the cache builder does not know, has to be 64 as well)."""
    return (n_head_blocks is not None and n_head_blocks_v is not None and n_blocks_col < (1 << 28)
            and n_head_blocks <= 2 and n_head_blocks_v <= 2)


def _group_union(attention_layout: Tensor, n_batches: int, n_blocks_row: int, n_blocks_col: int) -> Tensor:
    """The union of rows ``2 g`` and ``2 g + 1`` of the attention layout, 0/1 bytes ``(B, ceil(rows / 2), cols)``
    (``bsa_lut_pair_union``)."""
    lay = layout_bytes(attention_layout)
    union = torch.empty((n_batches, (n_blocks_row + 1) // 2, n_blocks_col), dtype=torch.uint8, device=lay.device)
    if union.numel():
        with _capi.on_device(lay.device):
            _capi.call("bsa_lut_pair_union", lay.data_ptr(), n_batches, n_blocks_row, n_blocks_col, union.data_ptr(),
                       _capi.stream(lay.device))
    return union


def flash_attention_build_layout_cache(attention_layout: Tensor,
                                       sparsity_layout_q: Tensor | None = None,
                                       sparsity_layout_k: Tensor | None = None,
                                       sparsity_layout_v: Tensor | None = None,
                                       n_seq_blocks_q: int | None = None,
                                       n_seq_blocks_k: int | None = None,
                                       n_head_blocks: int | None = None,
                                       sparsity_layout_o: Tensor | None = None,
                                       n_head_blocks_v: int | None = None,
                                       layout_cache: dict | None = None,
                                       sparsity_layout_mask: Tensor | None = None,
                                       sparsity_layout_bias: Tensor | None = None) -> dict:
    """Builds reusable layout metadata for block-sparse flash attention.

    Args:
        attention_layout (Tensor): The block attention pattern ``(n_batches, n_seq_blocks_q, n_seq_blocks_k)``.
        sparsity_layout_q (Tensor, optional): The sparsity layout of Q (default ``None``).
        sparsity_layout_k (Tensor, optional): The sparsity layout of K (default ``None``).
        sparsity_layout_v (Tensor, optional): The sparsity layout of V (default ``None``).
        n_seq_blocks_q (int, optional): The number of Q sequence blocks (default ``None``).
        n_seq_blocks_k (int, optional): The number of K sequence blocks (default ``None``).
        n_head_blocks (int, optional): The number of Q/K head-dimension blocks (default ``None``).
        sparsity_layout_o (Tensor, optional): The output sparsity layout (default ``None``).
        n_head_blocks_v (int, optional): The number of V/output head-dimension blocks (default ``None``).
        layout_cache (dict, optional): An existing layout metadata cache to extend (default ``None``).
        sparsity_layout_mask (Tensor, optional): The attention-mask sparsity layout (default ``None``).
        sparsity_layout_bias (Tensor, optional): The attention-bias sparsity layout (default ``None``).

    Returns:
        dict: The populated layout metadata cache.

    """
    named = (("sparsity_layout_q", sparsity_layout_q), ("sparsity_layout_k", sparsity_layout_k),
             ("sparsity_layout_v", sparsity_layout_v), ("sparsity_layout_o", sparsity_layout_o),
             ("sparsity_layout_mask", sparsity_layout_mask), ("sparsity_layout_bias", sparsity_layout_bias))
    checking = validation_enabled()  # one test here instead of one in every check below
    if checking:
        validate_dimensions(attention_layout)
        validate_contiguous(attention_layout)
        validate_sparsity_layout(attention_layout)
        given = tuple(layout for _, layout in named if layout is not None)
        if given:
            validate_dimensions(*given)
            validate_contiguous(*given)
            validate_device(attention_layout, *given)
            validate_sparsity_layout(*given)
        else:
            validate_device(attention_layout)

    n_batches, rows_q, rows_k = attention_layout.shape
    if n_seq_blocks_q is None:
        n_seq_blocks_q = rows_q
    elif n_seq_blocks_q != rows_q:
        raise ValueError("n_seq_blocks_q does not match attention_layout")
    if n_seq_blocks_k is None:
        n_seq_blocks_k = rows_k
    elif n_seq_blocks_k != rows_k:
        raise ValueError("n_seq_blocks_k does not match attention_layout")

    if n_head_blocks is None:
        source = sparsity_layout_q if sparsity_layout_q is not None else sparsity_layout_k
        if source is not None:
            n_head_blocks = source.size(2)
    if n_head_blocks_v is None:
        for source in (sparsity_layout_v, sparsity_layout_o, sparsity_layout_q):
            if source is not None:
                n_head_blocks_v = source.size(2)
                break

    expected = {
        "sparsity_layout_q": (n_batches, n_seq_blocks_q, n_head_blocks),
        "sparsity_layout_k": (n_batches, n_seq_blocks_k, n_head_blocks),
        "sparsity_layout_v": (n_batches, n_seq_blocks_k, n_head_blocks_v),
        "sparsity_layout_o": (n_batches, n_seq_blocks_q, n_head_blocks_v),
        "sparsity_layout_mask": (n_batches, n_seq_blocks_q, n_seq_blocks_k),
        "sparsity_layout_bias": (n_batches, n_seq_blocks_q, n_seq_blocks_k),
    }
    if checking:
        for name, layout in named:
            if layout is not None:
                validate_shape(layout, expected[name], name)

    layout_cache = prepare_layout_cache(
        layout_cache, "flash_attention",
        attention_layout, sparsity_layout_q, sparsity_layout_k, sparsity_layout_v,
        n_seq_blocks_q, n_seq_blocks_k, n_head_blocks, sparsity_layout_o, n_head_blocks_v,
        sparsity_layout_mask, sparsity_layout_bias,
    )

    if "sparsity_layout_o" not in layout_cache:
        if sparsity_layout_o is not None:
            layout_cache["sparsity_layout_o"] = as_base_tensor(sparsity_layout_o)
        elif sparsity_layout_v is not None:
            layout_cache["sparsity_layout_o"] = build_sparsity_layout_matmul(attention_layout, sparsity_layout_v)
    resolved_o = layout_cache.get("sparsity_layout_o")

    # Every layout this cache still has to scan, in ONE batch: the scans are queued one after the other and their
    # counts come back in one read (a cold cache scans eight layouts; one by one that was eight waits).
    wanted = []  # (what for, layout, row length)
    if "key_indices" not in layout_cache and attention_layout.numel():
        wanted.append(("keys", attention_layout, n_seq_blocks_k))
    transposed = None
    if "query_indices" not in layout_cache:
        transposed = as_base_tensor(attention_layout.transpose(1, 2).contiguous())
        if transposed.numel():
            wanted.append(("queries", transposed, n_seq_blocks_q))
    for name, layout in (("q", sparsity_layout_q), ("k", sparsity_layout_k), ("v", sparsity_layout_v),
                         ("mask", sparsity_layout_mask), ("bias", sparsity_layout_bias), ("o", resolved_o)):
        if layout is not None and f"packed_indices_{name}" not in layout_cache:
            wanted.append((name, layout, 0))
    if ("key_offsets_i32" not in layout_cache and _grouped_lists_apply(n_seq_blocks_k, n_head_blocks,
                                                                       n_head_blocks_v)
            and attention_layout.numel()):
        wanted.append(("groups", _group_union(attention_layout, int(n_batches), int(n_seq_blocks_q),
                                              int(n_seq_blocks_k)), n_seq_blocks_k))
    scans = dict(zip((w[0] for w in wanted), pack_layouts(*((w[1], w[2]) for w in wanted)))) if wanted else {}

    if "key_indices" not in layout_cache:
        indices, offsets, longest = _build_segmented_indices(attention_layout, n_batches, n_seq_blocks_q,
                                                             n_seq_blocks_k, scans.get("keys"))
        layout_cache["key_indices"], layout_cache["key_offsets"] = indices, offsets
        layout_cache["max_keys_per_query"] = longest

    if "query_indices" not in layout_cache:
        indices, offsets, longest = _build_segmented_indices(transposed, n_batches, n_seq_blocks_k, n_seq_blocks_q,
                                                             scans.get("queries"))
        layout_cache["query_indices"], layout_cache["query_offsets"] = indices, offsets
        layout_cache["max_queries_per_key"] = longest

    for name in ("q", "k", "v", "mask", "bias", "o"):
        info = scans.get(name)
        if info is not None:
            layout_cache[f"packed_indices_{name}"] = info.packed
            if name in ("q", "o"):
                layout_cache[f"n_sparse_blocks_{name}"] = info.count
    if "groups" in scans:
        # the scan of the union of neighbouring query rows, from which the operator makes the lists of the
        # matrix-core forward kernel when the block size is 64
        info = scans["groups"]
        layout_cache["group_union_packed"], layout_cache["group_union_offsets"] = info.packed, info.row_offsets
        layout_cache["group_union_count"] = info.count

    tensors = [v for v in layout_cache.values() if isinstance(v, Tensor)]
    if tensors:
        validate_contiguous(*tensors)

    return finalize_layout_cache(layout_cache)


_LENGTHS_SEEN = threading.local()


def _normalise_causal_lengths(causal_lengths: Tensor | None, n_batches: int, q_length: int, k_length: int,
                              device: torch.device) -> Tensor | None:
    if causal_lengths is None:
        return None
    if not isinstance(causal_lengths, Tensor):
        raise TypeError("causal_lengths must be a tensor or None")
    if q_length != k_length:
        raise ValueError("Native causal attention requires equal query and key lengths")
    if causal_lengths.dim() != 1:
        raise ValueError("causal_lengths must be one-dimensional")
    if causal_lengths.dtype == torch.bool or torch.is_floating_point(causal_lengths):
        raise TypeError("causal_lengths must use an integral dtype")
    validate_device(causal_lengths, torch.empty(0, device=device))
    validate_shape(causal_lengths, (n_batches,), "causal_lengths")
    # The range check reads the device (two waits of the host): its verdict on one tensor is remembered, per
    # thread, for as long as the tensor's version counter says that nothing was written to it in place (the
    # reference checks on every call, blksprs/ops/flash_attention.py:239-241; a write through .data goes unseen,
    # as for the facts kept per mask).
    seen = getattr(_LENGTHS_SEEN, "last", None)
    key = (causal_lengths._version, int(q_length)) if not torch.is_inference(causal_lengths) else None
    if seen is None or seen[0] is not causal_lengths or seen[1] != key or key is None:
        if torch.any(causal_lengths < 0) or torch.any(causal_lengths > q_length):
            raise ValueError(f"causal_lengths values must be between zero and {q_length}")
        _LENGTHS_SEEN.last = (causal_lengths, key, ensure_contiguous(causal_lengths.to(dtype=torch.int64)))
    return _LENGTHS_SEEN.last[2]


def _as_index(t: Tensor | None, dtype: torch.dtype) -> Tensor | None:
    if t is None or t.dtype == dtype:
        return t
    return t.to(dtype)


def _build_forward_records(layout_cache: dict, attention_layout: Tensor, n_batches: int, nq: int, nk: int,
                           nh: int, nhv: int, own_layout: bool = False) -> tuple[Tensor, Tensor, int]:
    """``(group_offsets, group_records, group_size)``: the lists the matrix-core forward kernel walks, for an
    attention layout and a layout cache that already holds the packed indices.  ``own_layout``: the layout is
    the one the cache was built for."""
    info = None
    if own_layout and "group_union_packed" in layout_cache:  # scanned with the cache's other layouts
        info = PackedLayout(layout_cache["group_union_packed"], layout_cache["group_union_count"],
                            layout_cache["group_union_offsets"], 0)
    offsets, entries, group_size = _build_group_lists(attention_layout, n_batches, nq, nk, info)
    records = torch.zeros(entries.numel() * _capi.ATTN_RECORD_INTS, dtype=torch.int32, device=entries.device)
    a = _capi.AttnArgs()
    a.B, a.nq, a.nk, a.nh, a.nhv = n_batches, nq, nk, nh, nhv
    a.pidx_k, a.pidx_v = _capi.ptr(layout_cache["packed_indices_k"]), _capi.ptr(layout_cache["packed_indices_v"])
    if "packed_indices_mask" in layout_cache:
        a.pidx_mask = _capi.ptr(layout_cache["packed_indices_mask"])
    if "packed_indices_bias" in layout_cache:
        a.pidx_bias = _capi.ptr(layout_cache["packed_indices_bias"])
    a.group_offsets, a.group_size = offsets.data_ptr(), group_size
    with _capi.on_device(entries.device):
        _capi.check(_capi.load().bsa_attn_fwd_records(ctypes.byref(a), _capi.ptr(entries), _capi.ptr(records),
                                                      _capi.stream(entries.device)), "bsa_attn_fwd_records")
    return offsets, as_base_tensor(records), group_size


class _Tables:
    """The lookup tables of one attention layout cache as one object.  A forward pass hands this object, not the
    caller's cache dict, to its backward pass: the dict may be emptied and refilled for other layouts between the
    two (``prepare_layout_cache`` clears it in place), the object keeps what it was built with.  Nothing writes
    to its tensors after they are built."""

    _NAMES = ("n_sparse_blocks_o", "packed_indices_q", "packed_indices_k", "packed_indices_v", "packed_indices_o",
              "packed_indices_mask", "packed_indices_bias", "key_offsets_i32", "key_indices_i32",
              "query_offsets_i32", "query_indices_i32", "group_offsets", "group_records", "group_size")
    __slots__ = _NAMES

    def __init__(self, cache: dict):
        for name in self._NAMES:
            setattr(self, name, cache.get(name))


_PRUNE_AT_ONCE_BLOCKS = 32768  # active blocks of the attention layout from which dead pairs are listed at once


class _MaskFacts:
    """What one mask tensor (and one tensor of causal lengths) adds to the layout metadata.

    A pair of blocks whose mask block masks every position adds nothing to the output or to any gradient.  The
    forward lists without those pairs and the records the backward kernels walk depend on the values of the
    mask, so they are kept per mask: ``key`` names its memory, version counter, shape and dtype (an in-place
    change of the mask bumps the version), ``refs`` keeps that memory from being handed out again while the
    facts live.  A mask that changes through ``.data`` is not noticed, like a layout in the layout cache.
    No counterpart in the reference, which visits every pair (blksprs/ops/flash_attention.py:1058-1175).
    """

    __slots__ = ("key", "refs", "sightings", "group_offsets", "group_records", "bwd_scratch", "bwd_stream")

    def __init__(self, key, refs):
        self.key, self.refs, self.sightings = key, refs, 0
        self.group_offsets = self.group_records = self.bwd_scratch = self.bwd_stream = None


def _tensor_identity(t: Tensor | None):
    if t is None:
        return None
    # inference tensors have no version counter: never equal to anything seen before
    version = object() if torch.is_inference(t) else t._version
    return t.data_ptr(), version, tuple(t.shape), t.dtype


def _mask_facts(layout_cache: dict, attention_layout: Tensor, mask: Tensor | None, mask_bytes: Tensor | None,
                lengths: Tensor | None, dims: tuple[int, int, int, int, int], sbs: int) -> "_MaskFacts | None":
    """The facts for this mask in ``layout_cache``, renewed when another mask (or another version) arrives.

    The forward lists without dead pairs are built when a mask is seen for the second time in a row: a caller
    that brings a new mask with every call never pays for lists it would use once.  On a layout of
    ``_PRUNE_AT_ONCE_BLOCKS`` active blocks or more they are built at the first sighting: there the pass over the
    mask and the new lists cost about what the forward call saves by them (measured on 110 000 blocks of which 46 %
    are dead: 0.14 ms for the lists, 0.12 ms saved per call), so a mask that is used once loses nothing and a mask
    that is used again gains from its first call on.
    """
    if not mask_facts_enabled():
        return None
    holder = layout_cache.get("mask_facts")
    if holder is None:
        holder = layout_cache["mask_facts"] = CacheHolder()
        finalize_layout_cache(layout_cache)
    key = (_tensor_identity(mask), _tensor_identity(lengths))
    facts = holder.cache.get("facts")
    if facts is None or facts.key != key:
        facts = holder.cache["facts"] = _MaskFacts(key, (mask, lengths))
    facts.sightings += 1
    has_mask = mask_bytes is not None and mask_bytes.size(0) > 0
    at_once = "key_indices_i32" in layout_cache and layout_cache["key_indices_i32"].numel() >= _PRUNE_AT_ONCE_BLOCKS
    if (facts.sightings >= (1 if at_once else 2) and facts.group_offsets is None
            and (has_mask or lengths is not None)
            and "group_offsets" in layout_cache and not torch.cuda.is_current_stream_capturing()):
        B, nq, nk, nh, nhv = dims
        device = attention_layout.device
        live_layout = attention_layout.reshape(B, nq, nk) != 0
        if has_mask:
            dead = torch.empty(mask_bytes.size(0), dtype=torch.uint8, device=device)
            with _capi.on_device(device):
                _capi.call("bsa_attn_mask_dead", _capi.ptr(mask_bytes), mask_bytes.size(0), mask_bytes.size(-1),
                           _capi.ptr(dead), _capi.stream(device))
            block_of_pair = layout_cache["packed_indices_mask"].reshape(B, nq, nk)
            live_layout = live_layout & ~((block_of_pair >= 0) & (dead != 0)[block_of_pair.clamp(min=0)])
        if lengths is not None:
            # pairs the causal predicate rules out as a whole (blksprs/ops/flash_attention.py:1133-1137):
            # every key after every query, or all queries / all keys at or beyond the valid length
            query_block = torch.arange(nq, device=device).view(1, nq, 1)
            key_block = torch.arange(nk, device=device).view(1, 1, nk)
            valid = lengths.to(device).view(B, 1, 1)
            live_layout = live_layout & (key_block <= query_block) & (query_block * sbs < valid) \
                & (key_block * sbs < valid)
        facts.group_offsets, facts.group_records, _ = _build_forward_records(layout_cache, live_layout, B, nq, nk,
                                                                             nh, nhv)
    return facts


class _Meta:
    """Everything the kernels need besides the differentiable tensors."""

    __slots__ = ("tables", "dims", "sbs", "scale", "has_bias", "facts")


def _fill_args(meta: "_Meta", q, k, v, bias, mask, causal_lengths) -> _capi.AttnArgs:
    """``mask`` (one byte per element) and ``causal_lengths`` come from the caller at forward time and from
    autograd's saved tensors at backward time, so a change in place between the two is an autograd error."""
    c = meta.tables
    a = _capi.AttnArgs()
    B, nq, nk, nh, nhv = meta.dims
    a.B, a.nq, a.nk, a.nh, a.nhv = B, nq, nk, nh, nhv
    a.q, a.k, a.v = _capi.ptr(q), _capi.ptr(k), _capi.ptr(v)
    a.n_q_blocks, a.n_k_blocks, a.n_v_blocks = q.size(0), k.size(0), v.size(0)
    a.n_o_blocks = c.n_sparse_blocks_o
    a.pidx_q, a.pidx_k = _capi.ptr(c.packed_indices_q), _capi.ptr(c.packed_indices_k)
    a.pidx_v, a.pidx_o = _capi.ptr(c.packed_indices_v), _capi.ptr(c.packed_indices_o)
    # int64 CSR metadata only exists beyond 2**31 - 1 blocks; the kernels index with int32
    a.key_offsets = c.key_offsets_i32.data_ptr()
    a.key_indices = _capi.ptr(c.key_indices_i32)
    a.query_offsets = c.query_offsets_i32.data_ptr()
    a.query_indices = _capi.ptr(c.query_indices_i32)
    if c.group_offsets is not None:
        a.group_offsets = c.group_offsets.data_ptr()
        a.group_records = _capi.ptr(c.group_records)
        a.group_size = c.group_size
        if meta.facts is not None and meta.facts.group_offsets is not None:
            a.group_offsets = meta.facts.group_offsets.data_ptr()
            a.group_records = _capi.ptr(meta.facts.group_records)
    if mask is not None:
        a.mask, a.pidx_mask = _capi.ptr(mask), _capi.ptr(c.packed_indices_mask)
        a.n_mask_blocks = mask.size(0)
        a.mask_kind = 1 if mask.numel() else 0
    if meta.has_bias:
        a.bias, a.pidx_bias = _capi.ptr(bias), _capi.ptr(c.packed_indices_bias)
        a.n_bias_blocks = bias.size(0)
    if causal_lengths is not None:
        a.causal_lengths = causal_lengths.data_ptr()
    a.sbs = meta.sbs
    a.dtype = _capi.DTYPE_CODES[q.dtype]
    a.scale = meta.scale
    return a


def _forward_launch(q, k, v, bias, mask, causal_lengths, meta: "_Meta"):
    """The forward launch by itself: ``(out, lse)``."""
    B, nq, nk, nh, nhv = meta.dims
    sbs = meta.sbs
    out = torch.empty((meta.tables.n_sparse_blocks_o, sbs, sbs), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, nq, sbs), dtype=torch.float32, device=q.device)
    args = _fill_args(meta, q, k, v, bias, mask, causal_lengths)
    args.o, args.lse = _capi.ptr(out), _capi.ptr(lse)
    with _capi.on_device(q.device):
        _capi.call("bsa_attn_fwd", ctypes.byref(args), _capi.stream(q.device))
    return out, lse


def _walks_records(meta: "_Meta", dtype: torch.dtype) -> bool:
    """Whether ``bsa_attn_bwd`` runs the kernels that build and walk records in ``bwd_scratch`` (and can keep dS)
    for these operands: 16-bit, 64 x 64 blocks, one or two head slices each for q / k and for v / o."""
    _, _, _, nh, nhv = meta.dims
    return meta.sbs == 64 and dtype in (torch.bfloat16, torch.float16) and 1 <= nh <= 2 and 1 <= nhv <= 2


class _FlashAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, bias, mask, causal_lengths, meta: "_Meta"):
        out, lse = _forward_launch(q, k, v, bias, mask, causal_lengths, meta)
        # the mask and the lengths are saved like the operands (as the reference does,
        # blksprs/ops/flash_attention.py:498-501): autograd then refuses a backward pass after either was
        # changed in place
        ctx.save_for_backward(q, k, v, bias, out, lse, mask, causal_lengths)
        ctx.meta = meta
        return out

    @staticmethod
    def backward(ctx, grad_output):
        grad_output = grad_output.contiguous()
        q, k, v, bias, out, lse, mask, causal_lengths = ctx.saved_tensors
        meta = ctx.meta
        B, nq, nk, nh, nhv = meta.dims
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        delta = torch.empty((B, nq, meta.sbs), dtype=torch.float32, device=q.device)
        dbias = torch.empty(bias.shape, dtype=torch.float32, device=q.device) if meta.has_bias else None
        args = _fill_args(meta, q, k, v, bias, mask, causal_lengths)
        args.o, args.d_o, args.lse, args.delta = _capi.ptr(out), _capi.ptr(grad_output), _capi.ptr(lse), _capi.ptr(delta)
        args.dq, args.dk, args.dv, args.dbias = _capi.ptr(dq), _capi.ptr(dk), _capi.ptr(dv), _capi.ptr(dbias)
        n_layout_blocks = meta.tables.key_indices_i32.numel()
        n_mask_blocks = mask.size(0) if mask is not None else 0
        stream = _capi.stream(q.device)
        facts = meta.facts
        args.n_layout_blocks = n_layout_blocks
        # Only the 16-bit kernels for 64 x 64 blocks and at most two head slices walk records in a scratch (the
        # pairs that some score survives, built inside bsa_attn_bwd); the other kernel families never touch it.
        if _walks_records(meta, q.dtype):
            size = max(_capi.load().bsa_attn_bwd_scratch_bytes(B, nq, nk, n_layout_blocks, n_mask_blocks), 16)
            # The records depend on the layouts and on the values of the mask and of the causal lengths only: a
            # later call on the same stream with the same ones reads what this call wrote.  Remembered only here,
            # where the call that ran did write them.
            scratch = facts.bwd_scratch if facts is not None and facts.bwd_stream == stream else None
            args.bwd_scratch_ready = 1 if scratch is not None and scratch.numel() == size else 0
            if not args.bwd_scratch_ready:
                scratch = torch.empty(size, dtype=torch.uint8, device=q.device)
            args.bwd_scratch, args.bwd_scratch_bytes = scratch.data_ptr(), size
            # With room for dS of every pair (one block per active block of the attention layout) the dK / dV kernel
            # leaves it behind and dQ = dS K is a product of its own; beyond the limit (set_kept_ds_limit) dS is
            # formed a second time, as the reference does (blksprs/ops/flash_attention.py:1228-1480).  dS carries
            # nothing from one call to the next: it is taken from torch's allocator for this call alone.
            ds_bytes = _capi.load().bsa_attn_bwd_ds_bytes(n_layout_blocks, meta.sbs)
            if 0 < ds_bytes <= kept_ds_limit():
                ds = torch.empty(ds_bytes, dtype=torch.uint8, device=q.device)
                args.bwd_ds, args.bwd_ds_bytes = ds.data_ptr(), ds_bytes
            with _capi.on_device(q.device):
                _capi.call("bsa_attn_bwd", ctypes.byref(args), stream)
            if facts is not None and not args.bwd_scratch_ready and not torch.cuda.is_current_stream_capturing():
                facts.bwd_scratch, facts.bwd_stream = scratch, stream
        else:
            with _capi.on_device(q.device):
                _capi.call("bsa_attn_bwd", ctypes.byref(args), stream)
        grad_bias = dbias.to(bias.dtype) if meta.has_bias else None
        return dq, dk, dv, grad_bias, None, None, None


@eager_only
@torch.amp.custom_fwd(device_type="cuda")
def flash_attention(q: BlksprsTensor, sparsity_layout_q: Tensor,
                    k: BlksprsTensor, sparsity_layout_k: Tensor,
                    v: BlksprsTensor, sparsity_layout_v: Tensor,
                    attention_layout: Tensor,
                    sparsity_block_size: int,
                    scale: float | None = None,
                    attention_mask: BlksprsTensor | None = None, sparsity_layout_mask: Tensor | None = None,
                    attention_bias: BlksprsTensor | None = None, sparsity_layout_bias: Tensor | None = None,
                    layout_cache: dict | None = None,
                    sparsity_layout_o: Tensor | None = None,
                    causal_lengths: Tensor | None = None) -> BlksprsTensor:
    """Computes block-sparse flash attention on compressed tensors.

    All inputs use the compressed format ``(n_sparse_blocks, sbs, sbs)`` with an accompanying sparsity layout.
    In ``attention_mask`` a non-zero value marks an **ignored** position (the ``masked_fill`` convention, the
    opposite of ``scaled_dot_product_attention``'s boolean ``attn_mask``).  Supported block sizes are 16, 32
    and 64.  Mask and bias each come with their own layout.

    Args:
        q (BlksprsTensor): Queries; layout ``(n_batches, seq_q // sbs, head_dim // sbs)``.
        sparsity_layout_q (Tensor): The sparsity layout of ``q``.
        k (BlksprsTensor): Keys; layout ``(n_batches, seq_k // sbs, head_dim // sbs)``.
        sparsity_layout_k (Tensor): The sparsity layout of ``k``.
        v (BlksprsTensor): Values.
        sparsity_layout_v (Tensor): The sparsity layout of ``v``.
        attention_layout (Tensor): Which (query block, key block) pairs attend, ``(n_batches, seq_q // sbs, seq_k // sbs)``.
        sparsity_block_size (int): The size of the sparsity blocks.
        scale (float, optional): Attention scale (default ``1/sqrt(head_dim)``).
        attention_mask (BlksprsTensor, optional): Binary mask in compressed form, not differentiated.
        sparsity_layout_mask (Tensor, optional): The sparsity layout of the mask.
        attention_bias (BlksprsTensor, optional): Additive bias in compressed form, applied before softmax; differentiable.
        sparsity_layout_bias (Tensor, optional): The sparsity layout of the bias.
        layout_cache (dict, optional): Reusable layout metadata cache (default ``None``).
        sparsity_layout_o (Tensor, optional): Output layout; defaults to the structural product of
            ``attention_layout`` and ``sparsity_layout_v``.
        causal_lengths (Tensor, optional): Integral valid lengths, one per batch, for native causal
            self-attention: future keys and padded queries / keys are ignored without a mask tensor.

    Returns:
        BlksprsTensor: The attention output in compressed form.

    """
    q, k, v, attention_layout = ensure_contiguous(q, k, v, attention_layout)
    q, k, v = cast_for_autocast(q, k, v)

    checking = validation_enabled()  # one test for each group of checks instead of one inside every check
    if checking:
        validate_dimensions(q, k, v)
        validate_contiguous(q, k, v)
        validate_dtype_float(q, k, v)
        validate_device(q, k, v)
        validate_sparsity(sparsity_block_size, (q, sparsity_layout_q), (k, sparsity_layout_k), (v, sparsity_layout_v))
        validate_sparsity_block_size(sparsity_block_size, q, k, v)
    if sparsity_block_size > 64:
        raise ValueError("Flash Attention sparsity block size must be at most 64")

    if checking:
        validate_dimensions(attention_layout)
        validate_contiguous(attention_layout)
        validate_device(attention_layout, q)
        validate_sparsity_layout(attention_layout)

    n_batches = sparsity_layout_q.size(0)
    n_seq_blocks_q = sparsity_layout_q.size(1)
    n_head_blocks_qk = sparsity_layout_q.size(2)
    n_seq_blocks_k = sparsity_layout_k.size(1)
    n_head_blocks_v = sparsity_layout_v.size(2)

    if sparsity_layout_k.size(0) != n_batches or sparsity_layout_k.size(2) != n_head_blocks_qk:
        raise ValueError("K sparsity layout must be compatible with Q")
    if sparsity_layout_v.size(0) != n_batches or sparsity_layout_v.size(1) != n_seq_blocks_k:
        raise ValueError("V sparsity layout must be compatible with K")

    attention_shape = (n_batches, n_seq_blocks_q, n_seq_blocks_k)
    validate_shape(attention_layout, attention_shape, "attention_layout")
    lengths = _normalise_causal_lengths(causal_lengths, n_batches, n_seq_blocks_q * sparsity_block_size,
                                        n_seq_blocks_k * sparsity_block_size, q.device)

    if sparsity_layout_o is not None:
        sparsity_layout_o = ensure_contiguous(sparsity_layout_o)
        validate_dimensions(sparsity_layout_o)
        validate_contiguous(sparsity_layout_o)
        validate_device(sparsity_layout_o, q)
        validate_sparsity_layout(sparsity_layout_o)
        validate_shape(sparsity_layout_o, (n_batches, n_seq_blocks_q, n_head_blocks_v), "sparsity_layout_o")

    if scale is None:
        head_dimension = n_head_blocks_qk * sparsity_block_size
        scale = 1.0 if head_dimension == 0 else 1.0 / math.sqrt(head_dimension)
    elif not isinstance(scale, Real):
        raise TypeError("Attention scale must be a real number or None")
    else:
        scale = float(scale)

    if (attention_mask is None) != (sparsity_layout_mask is None):
        raise ValueError("attention_mask and sparsity_layout_mask must be provided together")
    mask_bytes = None
    if attention_mask is not None:
        attention_mask = ensure_contiguous(attention_mask)
        sparsity_layout_mask = ensure_contiguous(sparsity_layout_mask)
        validate_dimensions(attention_mask, sparsity_layout_mask)
        validate_contiguous(attention_mask, sparsity_layout_mask)
        validate_device(attention_mask, sparsity_layout_mask, q)
        if attention_mask.dtype != torch.bool:
            validate_dtype_float(attention_mask)
        validate_binary(attention_mask)
        validate_sparsity(sparsity_block_size, (attention_mask, sparsity_layout_mask))
        validate_shape(sparsity_layout_mask, attention_shape, "sparsity_layout_mask")
        base = as_base_tensor(attention_mask.detach())
        # the kernels read one byte per mask element
        mask_bytes = (base if base.dtype == torch.bool else base != 0).view(torch.uint8)

    if (attention_bias is None) != (sparsity_layout_bias is None):
        raise ValueError("attention_bias and sparsity_layout_bias must be provided together")
    has_bias = attention_bias is not None
    if has_bias:
        attention_bias = ensure_contiguous(attention_bias)
        sparsity_layout_bias = ensure_contiguous(sparsity_layout_bias)
        validate_dimensions(attention_bias, sparsity_layout_bias)
        validate_contiguous(attention_bias, sparsity_layout_bias)
        validate_device(attention_bias, sparsity_layout_bias, q)
        validate_dtype_float(attention_bias)
        validate_sparsity(sparsity_block_size, (attention_bias, sparsity_layout_bias))
        validate_shape(sparsity_layout_bias, attention_shape, "sparsity_layout_bias")
        if attention_bias.dtype != q.dtype:
            attention_bias = attention_bias.to(q.dtype)
    else:
        attention_bias = torch.empty(0, device=q.device, dtype=q.dtype)

    layout_cache = flash_attention_build_layout_cache(
        attention_layout, sparsity_layout_q, sparsity_layout_k, sparsity_layout_v,
        n_seq_blocks_q, n_seq_blocks_k, n_head_blocks_qk,
        sparsity_layout_o=sparsity_layout_o, n_head_blocks_v=n_head_blocks_v,
        sparsity_layout_mask=sparsity_layout_mask, sparsity_layout_bias=sparsity_layout_bias,
        layout_cache=layout_cache,
    )
    if "key_offsets_i32" not in layout_cache:
        for name in ("key_offsets", "key_indices", "query_offsets", "query_indices"):
            layout_cache[name + "_i32"] = _as_index(layout_cache[name], torch.int32)
        if (n_seq_blocks_k < (1 << 28) and layout_cache["key_indices"].numel() < INT32_INDEX_MAX
                and n_head_blocks_qk <= 2 and n_head_blocks_v <= 2 and sparsity_block_size == 64):
            offsets, records, group_size = _build_forward_records(
                layout_cache, attention_layout, int(n_batches), int(n_seq_blocks_q), int(n_seq_blocks_k),
                int(n_head_blocks_qk), int(n_head_blocks_v), own_layout=True)
            layout_cache["group_offsets"], layout_cache["group_records"] = offsets, records
            layout_cache["group_size"] = group_size
        layout_cache["tables"] = _Tables(layout_cache)
        finalize_layout_cache(layout_cache)

    meta = _Meta()
    meta.tables = layout_cache["tables"]
    meta.dims = (int(n_batches), int(n_seq_blocks_q), int(n_seq_blocks_k), int(n_head_blocks_qk),
                 int(n_head_blocks_v))
    meta.sbs = sparsity_block_size
    meta.scale = scale
    meta.has_bias = has_bias
    meta.facts = _mask_facts(layout_cache, attention_layout, attention_mask, mask_bytes, lengths, meta.dims,
                             sparsity_block_size)

    needs_grad = torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad
                                              or (attention_bias is not None and attention_bias.requires_grad))
    if not needs_grad:
        # nothing to differentiate: the launch itself, without the autograd machinery around it
        return BlksprsTensor.wrap(_forward_launch(q, k, v, attention_bias, mask_bytes, lengths, meta)[0])
    return BlksprsTensor.wrap(_FlashAttention.apply(q, k, v, attention_bias, mask_bytes, lengths, meta))
