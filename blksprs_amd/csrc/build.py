"""Builds libblksprs_amd.so from the HIP sources in this directory.

    python -m blksprs_amd.csrc.build

One hipcc invocation per translation unit (run in parallel), then one link.  The
library lands in ``blksprs_amd/lib/`` and is what ``blksprs_amd._capi`` loads.
"""

import concurrent.futures
import os
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT_DIR = HERE.parent / "lib"
LIB = OUT_DIR / "libblksprs_amd.so"
SOURCES = ["common.hip", "lut.hip", "lut_order.hip", "convert.hip", "softmax.hip", "matmul.hip", "matmul_rows.hip", "matmul_lines.hip", "row_wise.hip",
           "attention.hip", "attn_generic.hip", "attn_mfma.hip", "attn_bwd_mfma.hip", "attn_f32mma.hip", "attn_f32mma_bwd.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "-std=c++17", "-fno-strict-aliasing", "--offload-arch=gfx950", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]


def _build_info() -> str:
    """What ``bsa_build_info()`` returns: the compiler's own version line and the flags."""
    try:
        out = subprocess.run([HIPCC, "--version"], capture_output=True, text=True).stdout.splitlines()
        version = next((line.strip() for line in out if "HIP version" in line), out[0].strip() if out else "unknown")
        clang = next((line.strip() for line in out if "clang version" in line), "")
    except OSError:
        version, clang = "unknown", ""
    text = f"hipcc: {version}; {clang}; flags: {' '.join(FLAGS)}"
    return "".join(c for c in text if c.isprintable() and c not in '"\\')


def _compile(src: str) -> Path:
    obj = OUT_DIR / "obj" / (Path(src).stem + ".o")
    extra = [f'-DBSA_BUILD_INFO="{_build_info()}"'] if src == "common.hip" else []
    cmd = [HIPCC, *FLAGS, *extra, "-c", str(HERE / src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = True) -> Path:
    (OUT_DIR / "obj").mkdir(parents=True, exist_ok=True)
    jobs = min(len(SOURCES), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = list(pool.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objects)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stderr)
    if verbose:
        print(f"built {LIB} ({LIB.stat().st_size} bytes)")
    return LIB


if __name__ == "__main__":
    build()
