"""ctypes binding of libblksprs_amd.so (the C ABI declared in include/blksprs_amd.h).

The library is the only compute path of this package: there is no fallback.  If
it has not been built, every operator raises ``RuntimeError`` on first use.
"""

import ctypes
import os
from pathlib import Path

import torch

_LIB_PATH = Path(__file__).resolve().parent / "lib" / "libblksprs_amd.so"

ABI_VERSION = 3
F32, F16, BF16 = 0, 1, 2
DTYPE_CODES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

c_void_p, c_int, c_int64, c_size_t, c_uint64, c_float = (
    ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t, ctypes.c_uint64, ctypes.c_float)


class AttnArgs(ctypes.Structure):
    """Mirror of ``struct bsa_attn_args``."""

    _fields_ = (
        [(n, c_void_p) for n in ("q", "k", "v", "o", "d_o", "dq", "dk", "dv", "lse", "delta", "mask", "bias", "dbias",
                                 "pidx_q", "pidx_k", "pidx_v", "pidx_o", "pidx_mask", "pidx_bias",
                                 "key_offsets", "key_indices", "query_offsets", "query_indices", "causal_lengths")]
        + [(n, c_int64) for n in ("B", "nq", "nk", "nh", "nhv", "n_q_blocks", "n_k_blocks", "n_v_blocks",
                                  "n_o_blocks", "n_mask_blocks", "n_bias_blocks")]
        + [("sbs", ctypes.c_int32), ("dtype", ctypes.c_int32), ("mask_kind", ctypes.c_int32), ("scale", c_float)]
        + [("group_offsets", c_void_p), ("group_records", c_void_p), ("group_size", ctypes.c_int32)]
        + [("bwd_scratch", c_void_p), ("n_layout_blocks", c_int64), ("bwd_scratch_ready", c_int64),
           ("bwd_scratch_bytes", c_int64), ("bwd_ds", c_void_p), ("bwd_ds_bytes", c_int64)]
    )


class LinesArgs(ctypes.Structure):
    """Mirror of ``struct bsa_lines_args``."""

    _fields_ = (
        [(n, c_void_p) for n in ("streamed", "priv", "out", "pidx_streamed", "pidx_private", "pidx_out",
                                 "part_table")]
        + [(n, c_int64) for n in ("n_batches", "lines_per_batch", "n_streamed", "n_outputs")]
        + [("streamed_strides", c_int64 * 3), ("out_strides", c_int64 * 3), ("private_strides", c_int64 * 3)]
        + [(n, c_int64) for n in ("nnz_streamed", "nnz_private", "nnz_out")]
        + [("error", c_void_p)]
    )


ATTN_RECORD_INTS = 16  # BSA_ATTN_RECORD_INTS
ROWS_RECORD_INTS = 128  # BSA_ROWS_RECORD_INTS

# name -> (restype, argtypes); must list every symbol of include/blksprs_amd.h
SIGNATURES = {
    "bsa_abi_version": (c_int, []),
    "bsa_last_error": (ctypes.c_char_p, []),
    "bsa_build_info": (ctypes.c_char_p, []),
    "bsa_lut_workspace_bytes": (c_size_t, [c_int64]),
    "bsa_lut_packed": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_size_t, c_void_p]),
    "bsa_lut_packed_static_max_entries": (c_int64, []),
    "bsa_lut_packed_static": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "bsa_lut_nonzero": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "bsa_lut_csr_indices": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "bsa_lut_sorted_rows": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "bsa_lut_pair_union": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "bsa_lut_pair_entries": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "bsa_layout_matmul": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "bsa_lut_contraction_offsets": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                                            c_void_p]),
    "bsa_lut_contraction_pairs": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                          c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "bsa_to_sparse": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p]),
    "bsa_to_dense": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_int,
                             c_uint64, c_void_p]),
    "bsa_matmul_lines_parts": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "bsa_matmul_lines": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p]),
    "bsa_transpose_blocks": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                     c_int, c_int, c_void_p]),
    "bsa_layout_from_dense": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "bsa_row_reduce": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_int,
                               c_int, c_void_p]),
    "bsa_row_add": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                            c_int, c_int, c_int, c_void_p]),
    "bsa_softmax_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "bsa_softmax_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "bsa_matmul": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int,
                           c_int, c_int, c_int, c_void_p]),
    "bsa_lut_order_workspace_bytes": (c_size_t, [c_int64]),
    "bsa_lut_block_order": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "bsa_lut_row_work_table": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_int64, c_int, c_void_p,
                                       c_int64, c_void_p, c_size_t, c_void_p]),
    "bsa_matmul_rows_records": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                        c_int64, c_void_p, c_void_p]),
    "bsa_matmul_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64,
                                c_int64, c_int64, c_int, c_int, c_void_p]),
    "bsa_attn_fwd_records": (c_int, [ctypes.POINTER(AttnArgs), c_void_p, c_void_p, c_void_p]),
    "bsa_attn_mask_dead": (c_int, [c_void_p, c_int64, ctypes.c_int32, c_void_p, c_void_p]),
    "bsa_attn_bwd_scratch_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64, c_int64]),
    "bsa_attn_bwd_ds_bytes": (c_size_t, [c_int64, ctypes.c_int32]),
    "bsa_attn_fwd": (c_int, [ctypes.POINTER(AttnArgs), c_void_p]),
    "bsa_attn_bwd": (c_int, [ctypes.POINTER(AttnArgs), c_void_p]),
}

_lib = None


def library_path() -> Path:
    return Path(os.environ.get("BLKSPRS_AMD_LIB", _LIB_PATH))


def load():
    """Loads the shared library once and binds every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not path.exists():
        raise RuntimeError(
            f"{path} is missing: build it with `python -m blksprs_amd.csrc.build` "
            "(hipcc, --offload-arch=gfx950). blksprs_amd has no other compute path.")
    lib = ctypes.CDLL(str(path))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.bsa_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{path} has ABI version {lib.bsa_abi_version()}, expected {ABI_VERSION}")
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().bsa_last_error()
        raise RuntimeError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")


def ptr(t) -> int:
    """Device pointer of a tensor, or NULL for ``None`` / empty tensors."""
    if t is None or t.numel() == 0:
        return 0
    return t.data_ptr()


def stream(device) -> int:
    """The current torch stream of ``device`` as a raw hipStream_t."""
    index = device.index
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if index is None else index)


# entry points that wait for the stream when their `stats_host` argument (at the given position) is not NULL
_WAITS_WITH_STATS_HOST = {"bsa_lut_packed": 6, "bsa_lut_contraction_offsets": 11}
host_waits = 0  # calls so far that made the host wait for the device inside the library


_bound = {}  # entry point name -> bound foreign function (looked up once)


def call(name: str, *args) -> None:
    global host_waits
    fn = _bound.get(name)
    if fn is None:
        fn = _bound[name] = getattr(load(), name)
    if name in _WAITS_WITH_STATS_HOST and args[_WAITS_WITH_STATS_HOST[name]]:
        host_waits += 1
    rc = fn(*args)
    if rc != 0:
        check(rc, name)


class on_device:
    """``with on_device(device):`` makes ``device`` the current one for the launches inside, and does nothing at
    all when it already is (the common case; torch's own context manager costs two microseconds either way)."""

    __slots__ = ("index", "previous")

    def __init__(self, device):
        self.index = device.index

    def __enter__(self):
        self.previous = -1
        index = self.index
        if index is not None and torch._C._cuda_getDevice() != index:
            self.previous = torch._C._cuda_getDevice()
            torch._C._cuda_setDevice(index)

    def __exit__(self, *exc):
        if self.previous >= 0:
            torch._C._cuda_setDevice(self.previous)
        return False
