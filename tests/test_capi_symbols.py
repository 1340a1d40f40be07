"""The C-ABI library loads and exports exactly what include/blksprs_amd.h declares (no compute calls)."""

import ctypes
import re
from pathlib import Path

from blksprs_amd import _capi

HEADER = Path(__file__).resolve().parent.parent / "include" / "blksprs_amd.h"


def _declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(bsa_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_entry_points():
    assert _declared() == sorted(_capi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(str(_capi.library_path()))
    for name in _declared():
        assert hasattr(lib, name), name
    assert _capi.load().bsa_abi_version() == _capi.ABI_VERSION


def test_argument_block_matches_the_header_layout():
    # 24 pointers, 11 int64, 3 int32 and one float, then 2 pointers and one int32 (padded to 8 bytes), a pointer
    # and an int64
    assert ctypes.sizeof(_capi.AttnArgs) == 24 * 8 + 11 * 8 + 4 * 4 + 2 * 8 + 8 + 2 * 8
    assert _capi.AttnArgs.bwd_scratch.offset == 40 * 8 and _capi.AttnArgs.n_layout_blocks.offset == 41 * 8
    assert _capi.AttnArgs.group_offsets.offset == 37 * 8 and _capi.AttnArgs.group_size.offset == 39 * 8
    assert _capi.AttnArgs.sbs.offset == 35 * 8


def test_bad_arguments_are_rejected_on_the_host():
    lib = _capi.load()
    # sbs = 24 is not a power of two; nothing is launched
    rc = lib.bsa_matmul(0, 0, 0, 0, 0, 0, 0, 0, 0, 24, 0, 0, 0, 0)
    assert rc == -1 and b"power of two" in lib.bsa_last_error()
    rc = lib.bsa_to_sparse(0, 0, 0, 0, 32, 32, 16, 3, 0)
    assert rc == -1 and b"element size" in lib.bsa_last_error()
    # empty problems are accepted without touching the device
    assert lib.bsa_matmul(0, 0, 0, 0, 0, 0, 0, 0, 0, 64, 2, 0, 0, 0) == 0
    assert lib.bsa_softmax_fwd(0, 0, 0, 0, 0, 32, 0) == 0
