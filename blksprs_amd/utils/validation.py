"""Input checks and per-thread switches of the block-sparse operators.

The error types and message texts follow the reference
(blksprs/utils/validation.py:64-386 for the checks, :8-24 and :447-472 for the
thread-local switches) because callers and tests match on them.  Every check is
a no-op while validation is disabled for the calling thread.
"""

import functools
import operator
import threading

import torch
from torch import Tensor

_state = threading.local()


def _validation_enabled() -> bool:
    return getattr(_state, "validation", True)


validation_enabled = _validation_enabled


def _contiguous_enabled() -> bool:
    return getattr(_state, "contiguous", True)


def disable_validation() -> None:
    """Switch input validation off for the calling thread."""
    _state.validation = False


def enable_validation() -> None:
    """Switch input validation on for the calling thread."""
    _state.validation = True


def disable_contiguous() -> None:
    """Stop operators from calling ``.contiguous()`` on their operands (calling thread only)."""
    _state.contiguous = False


def enable_contiguous() -> None:
    """Let operators call ``.contiguous()`` on their operands again (calling thread only)."""
    _state.contiguous = True


def mask_facts_enabled() -> bool:
    return getattr(_state, "mask_facts", True)


def disable_mask_facts() -> None:
    """Turns off, for the calling thread, everything ``flash_attention`` keeps per mask tensor (the forward lists
    without the pairs a mask's values rule out, the reuse of the backward records): every call then walks the
    lists of the layouts alone and rebuilds the backward records.  For callers that rewrite a mask's memory
    behind autograd's back (``.data``, a foreign kernel), which the version counter those facts are keyed on
    does not see.  No counterpart in the reference, whose lists do not depend on mask values."""
    _state.mask_facts = False


def enable_mask_facts() -> None:
    """Reverts :func:`disable_mask_facts` (calling thread only)."""
    _state.mask_facts = True


_kept_ds_limit = 4 << 30


def kept_ds_limit() -> int:
    return _kept_ds_limit


def set_kept_ds_limit(n_bytes: int) -> None:
    """The backward of ``flash_attention`` on 64 x 64 16-bit blocks keeps dS of every pair in a buffer that lives
    for that one backward call (8 KiB per active block of the attention layout, taken from torch's allocator and
    returned to it when the call is queued; with it dQ costs one matrix product per pair instead of three) when the
    buffer of that call takes at most ``n_bytes`` (default 4 GiB; the limit is per call and the setting is shared
    by all threads); 0: never, dS is formed twice, as the reference does
    (blksprs/ops/flash_attention.py:1228-1480)."""
    global _kept_ds_limit
    _kept_ds_limit = int(n_bytes)


def _check(fn):
    """Turns ``fn`` into a no-op while validation is disabled."""

    @functools.wraps(fn)
    def guarded(*args, **kwargs):
        if _validation_enabled():
            return fn(*args, **kwargs)
        return None

    return guarded


def ensure_contiguous(*tensors: Tensor):
    """Returns the operands made contiguous unless that was switched off."""
    if _contiguous_enabled():
        if len(tensors) == 2:  # the common call, without a generator
            return tensors[0].contiguous(), tensors[1].contiguous()
        tensors = tuple(t.contiguous() for t in tensors)
    return tensors[0] if len(tensors) == 1 else tensors


@_check
def validate_dimensions(*tensors: Tensor, dims: int = 3) -> None:
    if any(t.dim() != dims for t in tensors):
        raise ValueError(f"Tensor must have {dims} dimensions")


@_check
def validate_contiguous(*tensors: Tensor) -> None:
    if not all(t.is_contiguous() for t in tensors):
        raise ValueError("Tensor must be contiguous")


_FLOAT_DTYPES = (torch.float16, torch.bfloat16, torch.float32)


@_check
def validate_dtype_float(*tensors: Tensor) -> None:
    for t in tensors:
        if t.dtype not in _FLOAT_DTYPES:
            raise ValueError("Tensor must have either float16, bfloat16, or float32 dtype")
        if t.dtype != tensors[0].dtype:
            raise ValueError("Tensors must have same dtype")


@_check
def validate_dtype_float_32(*tensors: Tensor) -> None:
    if any(t.dtype != torch.float32 for t in tensors):
        raise ValueError("Tensor must have float32 dtype")


SUPPORTED_COPY_DTYPES = (
    torch.bool, torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64,
    torch.float16, torch.bfloat16, torch.float32, torch.float64,
)


@_check
def validate_dtype_supported(*tensors: Tensor) -> None:
    if any(t.dtype not in SUPPORTED_COPY_DTYPES for t in tensors):
        raise ValueError("Tensor dtype is not supported")


@_check
def validate_same_dtype(*tensors: Tensor) -> None:
    if any(t.dtype != tensors[0].dtype for t in tensors[1:]):
        raise ValueError("Tensors must have same dtype")


def _is_zero_one(t: Tensor) -> bool:
    return bool(torch.all((t == 0) | (t == 1)))


@_check
def validate_binary(*tensors: Tensor) -> None:
    for t in tensors:
        if not _is_zero_one(t):
            raise ValueError("Tensor values must be either 0 or 1")


@_check
def validate_device(*tensors: Tensor) -> None:
    if not tensors:
        return
    first = tensors[0].device
    if first.type != "cuda":
        raise ValueError("Tensors must be on GPU")
    if any(t.device != first for t in tensors):
        raise ValueError("Tensors must be on same device")


@_check
def validate_shape(tensor: Tensor, expected_shape, name: str = "Tensor") -> None:
    expected = torch.Size(expected_shape)
    if tensor.shape != expected:
        raise ValueError(
            f"{name} shape {tuple(tensor.shape)} doesn't match expected {tuple(expected)}")


def _require_divisible(value: int, divisor: int, value_name: str, divisor_name: str) -> None:
    if value % divisor:
        raise ValueError(f"{value_name} must be divisible by {divisor_name}")


def _check_layout_values(layout: Tensor) -> None:
    if layout.is_complex():
        raise ValueError("Sparsity layout must not have a complex dtype")
    if layout.dtype != torch.bool and not _is_zero_one(layout):
        raise ValueError("Sparsity layout values must be either 0 or 1")


def _check_layout_common(tensor: Tensor, layout: Tensor) -> None:
    _check_layout_values(layout)
    if tensor.device != layout.device:
        raise ValueError("Tensor and sparsity layout must be on same device")
    if not layout.is_contiguous():
        raise ValueError("Sparsity layout must be contiguous")
    if layout.dim() != 3:
        raise ValueError("Sparsity layout must have exactly 3 dimensions")


def count_blocks(layout: Tensor) -> int:
    """Number of active blocks, summed in int64 so half-precision layouts with
    more than 2048 ones still count exactly."""
    return int(layout.reshape(-1).to(torch.int64).sum().item())


@_check
def validate_sparsity(sparsity_block_size: int, *pairs) -> None:
    """Checks compressed tensors against their layouts."""
    for tensor, layout in pairs:
        _check_layout_common(tensor, layout)
        if not (tensor.size(-1) == tensor.size(-2) == sparsity_block_size):
            raise ValueError("Blocks not conforming to sparsity block size")
        if tensor.size(0) != count_blocks(layout):
            raise ValueError("Mismatch between sparsity layout and blocks")


@_check
def validate_sparsity_dense(sparsity_block_size: int, *pairs) -> None:
    """Checks dense tensors against the layouts they are to be compressed with."""
    for tensor, layout in pairs:
        _check_layout_common(tensor, layout)
        if tensor.size(0) != layout.size(0):
            raise ValueError("Tensor batch dimension does not match sparsity layout")
        _require_divisible(tensor.size(-1), sparsity_block_size, "Tensor sizes", "sparsity block size")
        _require_divisible(tensor.size(-2), sparsity_block_size, "Tensor sizes", "sparsity block size")
        if (tensor.size(-1) // sparsity_block_size != layout.size(-1) or
                tensor.size(-2) // sparsity_block_size != layout.size(-2)):
            raise ValueError("Tensor not conforming to sparsity layout")


@_check
def validate_sparsity_layout(*layouts: Tensor) -> None:
    for layout in layouts:
        _check_layout_values(layout)
        if layout.dim() != 3:
            raise ValueError("Sparsity layout must have exactly 3 dimensions")
        if not layout.is_contiguous():
            raise ValueError("Sparsity layout must be contiguous")
        if layout.device.type != "cuda":
            raise ValueError("Sparsity layout must be on GPU")


@_check
def validate_sparsity_block_size(sparsity_block_size: int, *values) -> None:
    if isinstance(sparsity_block_size, bool) or not isinstance(sparsity_block_size, int):
        raise TypeError("Sparsity block size must be an integer")
    if sparsity_block_size < 16:
        raise ValueError("Sparsity block size must be at least 16")
    if sparsity_block_size & (sparsity_block_size - 1):
        raise ValueError("Sparsity block size must be a power of 2")
    for value in values:
        size = value if isinstance(value, (torch.Size, tuple, list)) else value.size()
        _require_divisible(size[-1], sparsity_block_size, "Tensor sizes", "sparsity block size")
        _require_divisible(size[-2], sparsity_block_size, "Tensor sizes", "sparsity block size")


@_check
def validate_positive_integer(value, name: str) -> None:
    if isinstance(value, bool):
        raise TypeError(f"{name} must be an integer")
    try:
        value = operator.index(value)
    except TypeError as exc:
        raise TypeError(f"{name} must be an integer") from exc
    if value < 1:
        raise ValueError(f"{name} must be a positive integer")
