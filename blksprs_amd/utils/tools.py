"""Layout -> lookup-table builders and the caller-owned layout cache.

The lookup tables are computed on the device by the integer kernels of
libblksprs_amd.so (``csrc/lut.hip``); this module sizes their outputs and keeps
the observable results identical to the reference's torch formulations
(blksprs/utils/tools.py:33-57 for the two basic tables, :60-156 for the cache,
:159-287 for the shape and dtype helpers).
"""

import functools
from typing import Any

import torch
from torch import Tensor, Size

from .. import _capi

INT32_INDEX_MAX = 2_147_483_647

LayoutCache = dict[str, Any]

_KEY = "_blksprs_cache_key"
_REFS = "_blksprs_cache_refs"
_STATE = "_blksprs_cache_state"
_CHECKED = "_blksprs_cache_checked"  # number of entries when the recorded state was last found valid
_WATCH = "_blksprs_cache_watch"      # the recorded state once more, in a form that is cheap to compare
_SAME = "_blksprs_cache_same"        # the key once more, in a form that is cheap to compare (see _same_inputs)
_PRIVATE = frozenset((_KEY, _REFS, _STATE, _CHECKED, _WATCH, _SAME))


def as_base_tensor(value: Tensor) -> Tensor:
    """Strips a tensor subclass (same storage) so metadata is always a plain ``torch.Tensor``."""
    return value if type(value) is Tensor else Tensor(value)


# --------------------------------------------------------------------------- device LUT builders

def layout_bytes(layout: Tensor) -> Tensor:
    """The layout as contiguous 0/1 bytes on its device (a view for bool layouts)."""
    layout = as_base_tensor(layout)
    if not layout.is_contiguous():
        layout = layout.contiguous()
    if layout.dtype == torch.bool:
        return layout.view(torch.uint8)
    if layout.dtype == torch.uint8:
        return layout
    # numeric layouts hold exact 0/1 values (validated upstream)
    return (layout != 0).view(torch.uint8)


def _require_device(t: Tensor) -> None:
    if t.device.type != "cuda":
        raise RuntimeError(
            "blksprs_amd builds lookup tables with HIP kernels and needs GPU tensors; "
            f"got a layout on {t.device}")


class PackedLayout:
    """Result of one device pass over a layout.

    Attributes:
        packed: int64 reverse index over the flattened layout (``-1`` = inactive).
        count: number of active blocks.
        row_offsets: int32 CSR offsets over rows of length ``row_len`` (``None`` if not requested).
        max_per_row: largest number of active blocks in one row (0 if not requested).
    """

    __slots__ = ("packed", "count", "row_offsets", "max_per_row")

    def __init__(self, packed, count, row_offsets, max_per_row):
        self.packed, self.count, self.row_offsets, self.max_per_row = packed, count, row_offsets, max_per_row


def pack_layouts(*specs, then=None):
    """Scans several layouts on the device, ``specs`` being ``(layout, row_len)`` pairs: reverse index, block
    count and optional CSR row offsets of each.

    One stream synchronisation for all of them (the counts size the caller's next allocations).  ``then``, if
    given, is called with the reverse indices before that synchronisation: it launches what depends on them
    alone and returns an int64 device tensor of its own statistics, which are read back in the same transfer;
    the function then returns ``(infos, statistics as a list)``.
    """
    lib = _capi.load()
    results = []
    stats_dev = None
    for number, (layout, row_len) in enumerate(specs):
        _require_device(layout)
        lay = layout_bytes(layout)
        n = lay.numel()
        dev = lay.device
        if stats_dev is None:
            stats_dev = torch.empty((len(specs), 2), dtype=torch.int64, device=dev)
        packed = torch.empty(n, dtype=torch.int64, device=dev)
        n_rows = n // row_len if row_len > 0 else 0
        row_offsets = torch.empty(n_rows + 1, dtype=torch.int32, device=dev) if row_len > 0 else None
        ws_bytes = lib.bsa_lut_workspace_bytes(n)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        with _capi.on_device(dev):
            _capi.call("bsa_lut_packed", _capi.ptr(lay), n, row_len, _capi.ptr(packed),
                       row_offsets.data_ptr() if row_offsets is not None else 0,
                       stats_dev[number].data_ptr(), 0, _capi.ptr(workspace), ws_bytes, _capi.stream(dev))
        results.append((packed, row_offsets))
    if then is None:
        stats = stats_dev.tolist() if results else []
        extra = None
    else:
        more = then([packed for packed, _ in results])
        both = torch.cat([stats_dev.reshape(-1), more.reshape(-1)]).tolist()
        stats = [both[2 * i:2 * i + 2] for i in range(len(results))]
        extra = both[2 * len(results):]
    infos = [PackedLayout(packed, int(count), row_offsets, int(longest))
             for (packed, row_offsets), (count, longest) in zip(results, stats)]
    return infos if then is None else (infos, extra)


def pack_layout(layout: Tensor, row_len: int = 0) -> PackedLayout:
    """``pack_layouts`` for one layout."""
    return pack_layouts((layout, row_len))[0]


def build_packed_indices(sparsity_layout: Tensor) -> Tensor:
    """int64 reverse index of a layout: position among the active blocks, ``-1`` for inactive ones."""
    return pack_layout(sparsity_layout).packed


def nonzero_from_packed(packed: Tensor, shape, count: int) -> Tensor:
    """int64 ``[count, 3]`` coordinates of the active blocks in row-major order."""
    B, R, C = (int(s) for s in shape)
    coords = torch.empty((count, 3), dtype=torch.int64, device=packed.device)
    if count:
        with _capi.on_device(packed.device):
            _capi.call("bsa_lut_nonzero", packed.data_ptr(), B, R, C, coords.data_ptr(), _capi.stream(packed.device))
    return coords


def build_layout_indices(sparsity_layout: Tensor) -> Tensor:
    """Coordinates of the active blocks, equal to ``torch.nonzero(sparsity_layout)``."""
    info = pack_layout(sparsity_layout)
    return nonzero_from_packed(info.packed, sparsity_layout.shape, info.count)


def csr_indices_from_packed(packed: Tensor, n_cols: int, count: int) -> Tensor:
    """int32 column ids of the active blocks, row by row."""
    indices = torch.empty(count, dtype=torch.int32, device=packed.device)
    if count:
        with _capi.on_device(packed.device):
            _capi.call("bsa_lut_csr_indices", packed.data_ptr(), packed.numel(), n_cols, indices.data_ptr(),
                       _capi.stream(packed.device))
    return indices


def sorted_rows_from_offsets(row_offsets: Tensor, n_rows: int, n_cols: int) -> Tensor:
    """Per-row descending sort of the reverse index (active first), int64 flat."""
    out = torch.empty(n_rows * n_cols, dtype=torch.int64, device=row_offsets.device)
    if out.numel():
        with _capi.on_device(out.device):
            _capi.call("bsa_lut_sorted_rows", row_offsets.data_ptr(), n_rows, n_cols, out.data_ptr(),
                       _capi.stream(out.device))
    return out


class ContractionLists:
    """Per-output-block lists of (x block, y block) index pairs of a block-sparse product."""

    __slots__ = ("pair_offsets", "pairs", "n_pairs")

    def __init__(self, pair_offsets, pairs, n_pairs):
        self.pair_offsets, self.pairs, self.n_pairs = pair_offsets, pairs, n_pairs


class _ContractionCounts:
    """What phase 1 of the contraction lists leaves on the device for phase 2."""

    __slots__ = ("operands", "dims", "mask_x", "mask_y", "pos_offsets", "stats_dev")


def count_contraction_pairs(pidx_x: Tensor, pidx_y: Tensor, pidx_o: Tensor, B: int, R: int, K: int,
                            C: int) -> _ContractionCounts:
    """Phase 1 of the contraction lists (``bsa_lut_contraction_offsets``), launched without waiting for it: the
    total number of pairs lies in ``stats_dev[0]`` on the device."""
    dev = pidx_o.device
    n = B * R * C
    W = (K + 63) // 64
    c = _ContractionCounts()
    c.operands, c.dims = (pidx_x, pidx_y, pidx_o), (B, R, K, C)
    c.mask_x = torch.empty(max(B * R * W, 1), dtype=torch.int64, device=dev)
    c.mask_y = torch.empty(max(B * C * W, 1), dtype=torch.int64, device=dev)
    c.pos_offsets = torch.empty(n + 1, dtype=torch.int32, device=dev)
    c.stats_dev = torch.empty(2, dtype=torch.int64, device=dev)
    ws_bytes = _capi.load().bsa_lut_workspace_bytes(n)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with _capi.on_device(dev):
        _capi.call("bsa_lut_contraction_offsets", _capi.ptr(pidx_x), _capi.ptr(pidx_y), _capi.ptr(pidx_o),
                   B, R, K, C, c.mask_x.data_ptr(), c.mask_y.data_ptr(), c.pos_offsets.data_ptr(),
                   c.stats_dev.data_ptr(), 0, workspace.data_ptr(), ws_bytes, _capi.stream(dev))
    return c


def write_contraction_pairs(c: _ContractionCounts, total: int, nnz_o: int) -> ContractionLists:
    """Phase 2: the lists themselves, ``total`` being the number of pairs phase 1 counted."""
    if total > INT32_INDEX_MAX:
        raise RuntimeError(f"block-sparse product has {total} block pairs; at most {INT32_INDEX_MAX} are supported")
    pidx_x, pidx_y, pidx_o = c.operands
    B, R, K, C = c.dims
    dev = pidx_o.device
    pair_offsets = torch.empty(nnz_o + 1, dtype=torch.int32, device=dev)
    pairs = torch.empty((total, 2), dtype=torch.int32, device=dev)
    with _capi.on_device(dev):
        _capi.call("bsa_lut_contraction_pairs", _capi.ptr(pidx_x), _capi.ptr(pidx_y), _capi.ptr(pidx_o),
                   B, R, K, C, c.mask_x.data_ptr(), c.mask_y.data_ptr(), c.pos_offsets.data_ptr(), nnz_o,
                   pair_offsets.data_ptr(), _capi.ptr(pairs), _capi.stream(dev))
    return ContractionLists(pair_offsets, pairs, total)


def build_contraction_lists(*products) -> "ContractionLists | list":
    """Builds, on the device, for every active output block the ascending-k list of block pairs to multiply.

    ``build_contraction_lists(pidx_x, pidx_y, pidx_o, B, R, K, C, nnz_o)`` for one product, or one such tuple per
    product for several: their pair counts are read back together, one wait for the stream in all."""
    one = not isinstance(products[0], tuple)
    if one:
        products = (products,)
    counted = [count_contraction_pairs(*p[:7]) for p in products]
    totals = torch.stack([c.stats_dev[0] for c in counted]).tolist()
    lists = [write_contraction_pairs(c, int(total), p[7]) for c, total, p in zip(counted, totals, products)]
    return lists[0] if one else lists


# --------------------------------------------------------------------------- layout cache

def prepare_layout_cache(layout_cache: LayoutCache | None, operation: str, *values: object) -> LayoutCache:
    """Returns ``layout_cache`` ready for ``operation``, emptied first if it belongs to other inputs.

    The cache is keyed on the operation name, on the identity / in-place version /
    shape / stride / dtype / device / requires_grad of every tensor argument and on
    every scalar argument, and it is also dropped when any derived entry changed
    since it was finalized.  Inference tensors have no version counter, so a cache
    keyed on one never hits.
    """
    if layout_cache is None:
        layout_cache = {}
    recorded = layout_cache.get(_STATE)
    if recorded is not None and _same_inputs(layout_cache.get(_SAME), operation, values):
        stale = not _unchanged(layout_cache, recorded)
        key = refs = None
    else:
        key, refs = layout_cache_key(operation, *values)
        stale = layout_cache.get(_KEY) != key or recorded is None or not _unchanged(layout_cache, recorded)
    if stale:
        if key is None:
            key, refs = layout_cache_key(operation, *values)
        layout_cache.clear()
        layout_cache[_KEY] = key
        # holding the sources keeps their ids from being reused by other tensors
        layout_cache[_REFS] = refs
        layout_cache[_SAME] = _same_inputs_record(operation, values)
    else:
        layout_cache.setdefault(_CHECKED, None)  # counted by len() below
        layout_cache[_CHECKED] = len(layout_cache)
    return layout_cache


def _same_inputs_record(operation: str, values: tuple):
    """What ``_same_inputs`` compares against, or ``None`` when some value is neither a tensor with a version
    counter nor a plain number, string or ``None`` (the full key decides then)."""
    entries = []
    for v in values:
        if isinstance(v, Tensor):
            if v.is_inference():
                return None
            entries.append((v, v._version, v.data_ptr(), v.requires_grad, v.shape))
        elif v is None or type(v) in (int, bool, float, str):
            entries.append((None, v, 0, False, None))  # a plain value: compared as it is
        else:
            return None
    return operation, tuple(entries)


def _same_inputs(record, operation: str, values: tuple) -> bool:
    """True when every value is the very tensor object the cache was filed under, not modified in place since (its
    version counter), at the same address, of the same shape and with the same ``requires_grad``: the full key
    (``layout_cache_key``) is then the recorded one, since the stride, dtype and device of an object only change
    together with its version counter or its storage.  False means "compare the full key", not "different"."""
    if record is None or record[0] != operation or len(record[1]) != len(values):
        return False
    for (tensor, version, address, requires_grad, shape), v in zip(record[1], values):
        if tensor is None:  # a plain value (the recorded one sits in `version`)
            if type(v) is not type(version) or v != version:
                return False
        elif (v is not tensor or v._version != version or v.data_ptr() != address or v.requires_grad != requires_grad
                or v.shape != shape):
            return False
    return True


def layout_cache_key(operation: str, *values: object) -> tuple[tuple, tuple]:
    """The key ``prepare_layout_cache`` files a cache under, and the tensors it depends on."""
    refs: list[Tensor] = []
    parts = [_signature(v, refs) for v in values]
    return (operation, tuple(parts)), tuple(refs)


def _signature(value, refs: list):
    if isinstance(value, Tensor):
        refs.append(value)
        # an inference tensor has no version counter: a fresh object never equals an earlier key
        version = object() if value.is_inference() else value._version
        # torch.Size and the stride tuple compare and hash like plain tuples
        return ("tensor", id(value), version, value.shape, value.stride(), value.dtype, value.device,
                value.requires_grad)
    if isinstance(value, (tuple, list, Size)):
        return tuple(_signature(v, refs) for v in value)
    if isinstance(value, dict):
        return tuple(sorted((k, _signature(v, refs)) for k, v in value.items()))
    return value


class CacheHolder:
    """A cache of a nested operation, kept inside a caller's cache as one opaque entry: the nested operation
    validates it itself, and what it adds later (the lists of a backward pass, say) does not make the outer cache
    look modified."""

    __slots__ = ("cache",)

    def __init__(self):
        self.cache: LayoutCache = {}


def finalize_layout_cache(layout_cache: LayoutCache) -> LayoutCache:
    """Records what the cache holds now; a later change of any entry invalidates it."""
    # a cache that prepare_layout_cache has just found equal to its recorded state, and that has gained no entry
    # since, is in that state still (builders add entries, they replace none)
    if layout_cache.get(_CHECKED) == len(layout_cache) and _STATE in layout_cache:
        return layout_cache
    layout_cache[_STATE] = _snapshot(layout_cache)
    layout_cache[_CHECKED] = None
    layout_cache[_WATCH] = None
    layout_cache[_WATCH] = _watch_list(layout_cache)
    return layout_cache


def _watch_list(layout_cache: LayoutCache) -> tuple:
    """The recorded state as ``(number of entries, [(key, object, version or None), ...])`` when every entry is a
    tensor with a version counter or a value that is compared by identity; ``None`` when some entry needs the full
    comparison (containers, inference tensors)."""
    entries = []
    for key, value in layout_cache.items():
        if key in _PRIVATE:
            continue
        if isinstance(value, Tensor):
            if torch.is_inference(value):
                return None
            entries.append((key, value, value._version))
        elif isinstance(value, (dict, tuple, list, Size, PackedLayout, ContractionLists)):
            return None
        else:
            entries.append((key, value, None))
    return len(layout_cache), tuple(entries)


def _unchanged(layout_cache: LayoutCache, recorded: tuple) -> bool:
    """Whether the cache holds what it held when its state was recorded: every entry the same object with the same
    version counter (this runs on every call of an operator that is handed a cache)."""
    watch = layout_cache.get(_WATCH)
    if watch is None or len(layout_cache) != watch[0]:
        return _snapshot(layout_cache) == recorded
    get = layout_cache.get
    for key, value, version in watch[1]:
        current = get(key, _PRIVATE)
        if current is not value or (version is not None and current._version != version):
            # an equal value under another identity (an int, say) is no change: let the full comparison decide
            return _snapshot(layout_cache) == recorded
    return True


def _snapshot(layout_cache: LayoutCache) -> tuple:
    # in insertion order: builders only add entries, so an unchanged cache lists them in the same order
    return tuple((k, _entry_state(v)) for k, v in layout_cache.items() if k not in _PRIVATE)


def _entry_state(value):
    if isinstance(value, Tensor):
        # a derived tensor is the same while it is the same object with the same version counter (this runs for
        # every entry on every call: no more than that)
        try:
            return id(value), value._version
        except RuntimeError:  # an inference tensor has no version counter: never equal to an earlier state
            return object()
    if isinstance(value, dict):
        return tuple((k, _entry_state(v)) for k, v in value.items() if k not in _PRIVATE)
    if isinstance(value, (tuple, list, Size)):
        return tuple(_entry_state(v) for v in value)
    if isinstance(value, (PackedLayout, ContractionLists)):
        return tuple(_entry_state(getattr(value, s)) for s in value.__slots__)
    return value


# --------------------------------------------------------------------------- shape / dtype helpers

def do_shape_blocksparse(x: Tensor) -> tuple[Tensor, Size]:
    """Flattens all leading dimensions into one batch dimension; returns the 3-D tensor and the original shape."""
    if x.dim() < 2:
        raise ValueError("Tensor must have at least 2 dimensions")
    if x.dim() == 3:
        return x.contiguous(), x.size()
    batch = 1
    for s in x.shape[:-2]:
        batch *= s
    return x.reshape(batch, x.size(-2), x.size(-1)).contiguous(), x.size()


def undo_shape_blocksparse(x: Tensor, shape: Size | tuple[int, ...]) -> Tensor:
    """Restores the leading dimensions removed by :func:`do_shape_blocksparse` (last two taken from ``x``)."""
    if x.dim() != 3:
        raise ValueError("Tensor must have exactly 3 dimensions")
    if len(shape) < 2:
        raise ValueError("Original shape must have at least 2 dimensions")
    batch = 1
    for s in shape[:-2]:
        batch *= s
    if x.size(0) != batch:
        raise ValueError("Tensor batch dimension does not match original shape")
    if x.shape[:-2] == shape[:-2]:
        return x
    return x.reshape((*shape[:-2], *x.shape[-2:]))


def ceil_pow2(x: int) -> int:
    """Smallest power of two >= ``x``."""
    if x <= 0:
        raise ValueError("Input must be a positive integer.")
    return 1 << (x - 1).bit_length()


def can_use_int32_indexing(*values: Tensor | int | None) -> bool:
    """Whether every given buffer (tensor or element count) has at most 2**31 - 1 elements."""
    for v in values:
        if v is None:
            continue
        n = v.numel() if isinstance(v, Tensor) else int(v)
        if n > INT32_INDEX_MAX:
            return False
    return True



def eager_only(fn):
    """Makes ``fn`` run outside ``torch.compile``: the returned entry point is an ordinary function whose only
    statement calls ``torch.compiler.disable(fn)``.  A caller's compiled graph breaks at that call and resumes after
    it (the reference's wrappers break the graph as well, at their validation and cache preparation).  Decorating
    the public function with ``torch.compiler.disable`` itself is not enough: ``torch.compile(fn)`` unwraps a
    disabled function it is handed directly and traces its body."""
    disabled = torch.compiler.disable(fn)
    is_compiling = torch.compiler.is_compiling

    @functools.wraps(fn)
    def entry(*args, **kwargs):
        # outside a trace the body is called as it is (the wrapper that keeps a trace out costs two microseconds
        # per call); while this function is being traced the test is true and the trace ends at the call below
        if not is_compiling():
            return fn(*args, **kwargs)
        return disabled(*args, **kwargs)

    return entry


def cast_for_autocast(*values: Tensor):
    """Casts fp16 / bf16 / fp32 GPU tensors to the autocast dtype while autocast is on; others pass through."""
    if torch.is_autocast_enabled():
        target = torch.get_autocast_dtype("cuda")
        eligible = (torch.float16, torch.bfloat16, torch.float32)
        values = tuple(v.to(target) if v.is_cuda and v.dtype in eligible else v for v in values)
    return values[0] if len(values) == 1 else values
