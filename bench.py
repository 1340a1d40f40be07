"""Benchmark of the block-sparse compute path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2]

A step is one pass of the hot path over one batch of synthetic, seeded input that is already resident in
HBM, with the lookup tables built beforehand (their build time is reported separately).  The default
workload is configuration 2 of BASELINE.json (bf16 block-sparse matmul, B=16, 4096^3, sbs 64, 25 % operand
density, product output layout), the configuration the headline metric is quoted on; ``--config`` selects
c1 (fp32 matmul 256^3), c2bwd (the two backward products of c2), c3 / c3bwd (fp32 softmax forward / backward),
c4 / c4bwd (bf16 flash attention forward / forward+backward), c5 (fp16 matmul, sbs 16) or one of the data
movement rows instead.  Without ``--config`` the line also carries, under ``other_configs``, the roofline objects of
c4 (forward), c3 and c5, timed in the same process.  One JSON line is printed on stdout; everything else goes to
stderr.

Every configuration is first checked on a sample against the CPU oracle (``correct``), then run untimed for 0.3 s
(a card that has idled starts below its sustained clock), then timed.  ``launch_ms_flushed`` / ``frac_flushed``
repeat the timing with 1 GiB written between launches, so that no launch finds its operands in the memory-side cache.

The ``roofline`` object prices the dominant kernel against the roofline that bounds it, from the average
launch duration measured with events on the launch stream; ``cpu_baseline`` times the CPU oracle on a
bounded sample of the same workload on the host cores (reported, not a target).
"""

import argparse
import json
import math
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

import torch

# MI355X published peaks (dense)
PEAK_HBM_GBS = 8000.0
PEAK_MFMA_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}


# HBM bytes per step: FETCH_SIZE and WRITE_SIZE (KiB per dispatch, summed over the kernels of one step) from the
# rocprofv3 --pmc runs summarised under profiles/ (one text file per configuration; the figures this script uses
# are collected in profiles/traffic.json, which `bench.py --summarise DIR --config X` writes from rocprofv3's output
# together with the text summary), scaled by what the same counters read for a plain copy kernel of known size
# (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  FETCH_SIZE counts what leaves an L2, so reads served by the memory-side
# cache are included.  Not re-measured by a timing run of this script.
TRAFFIC_FILE = ROOT / "profiles" / "traffic.json"
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0


def traffic_bytes(config):
    try:
        entry = json.loads(TRAFFIC_FILE.read_text()).get(config)
    except (OSError, ValueError):
        return None
    if not entry or entry.get("fetch_kib") is None or entry.get("write_kib") is None:
        return None
    return int((FETCH_SCALE * entry["fetch_kib"] + WRITE_SCALE * entry["write_kib"]) * 1024)


# file stem of the summary of a configuration under profiles/: the kernel(s) and the workload
PROFILE_STEMS = {
    "c1": "matmul_mfma_kernel_c1_fp32_matmul",
    "c2": "matmul_rows_kernel_c2_bf16_matmul",
    "c2bwd": "matmul_lines_kernel_c2bwd_bf16_matmul_backward",
    "c3": "softmax_fwd_kernel_c3_fp32_softmax",
    "c3bwd": "softmax_bwd_kernel_c3bwd_fp32_softmax_backward",
    "c4": "attn_fwd_mfma_kernel_c4_bf16_attention_forward",
    "c4cl": "attn_fwd_mfma_kernel_c4cl_bf16_attention_forward_causal_lengths",
    "c4bwd": "attn_kernels_c4_bf16_attention_forward_backward",
    "c5": "matmul_small16_kernel_c5_fp16_sbs16",
    "a1": "attn_f32mma_kernels_a1_fp32_reference_benchmark",
    "a1bwd": "attn_f32mma_kernels_a1bwd_fp32_reference_benchmark_backward",
    "m32": "matmul_mfma_kernel_m32_bf16_sbs32",
    "m128": "matmul_mfma_kernel_m128_bf16_sbs128",
    "mf32": "matmul_mfma_kernel_mf32_fp32_sbs64",
    "v1": "to_sparse_kernel_v1_bf16_to_sparse",
    "v2": "to_dense_kernel_v2_bf16_to_dense",
    "t1": "transpose_blocks16_kernel_t1_bf16_transpose",
    "l1": "layout_from_dense_kernel_l1_bf16_build_sparsity_layout",
    "r1": "row_reduce_kernel_r1_bf16_row_wise_sum",
    "r2": "row_add_kernel_r2_bf16_row_wise_add",
}
# kernels of this library by a piece of their name (rocprofv3 reports everything the process launches)
LIBRARY_KERNELS = ("matmul_", "softmax_", "attn_", "to_sparse", "to_dense", "transpose_blocks", "layout_from_dense",
                   "row_reduce", "row_add", "lines_", "rows_records", "lut_", "packed", "records_kernel")


def summarise_profile(directory, config, note, side_name=None):
    """Turns rocprofv3's output for one configuration into the text summary under profiles/ and the entry of
    profiles/traffic.json.  ``directory`` holds one sub-directory per run of the SAME command (`python3 bench.py
    --config X --steps S --warmup W --no-cpu-baseline`): ``trace`` (--kernel-trace --stats) and any number of
    counter runs (--pmc ...), among them FETCH_SIZE and WRITE_SIZE; each sub-directory may hold a file ``command``
    with the full command line, which is quoted.  Durations are averages over all dispatches, counters medians
    per dispatch (the first dispatches of a run may do one-off work)."""
    import collections
    import glob
    import sqlite3
    import statistics

    directory = Path(directory)
    lines = [f"# configuration {config} of bench.py: rocprofv3 (ROCm 7.2) on one MI355X, one run per counter set, "
             f"each run the full command shown; durations in microseconds, counters are medians per dispatch.",
             f"# FETCH_SIZE / WRITE_SIZE are in KiB as reported; calibration against a plain copy kernel of known "
             f"size: FETCH_SIZE x {FETCH_SCALE}, WRITE_SIZE x {WRITE_SCALE} give bytes."]
    if note:
        lines.append("# " + note)
    step_kernels, counters = {}, collections.defaultdict(dict)
    for sub in sorted((p for p in directory.iterdir() if p.is_dir()), key=lambda p: (p.name != "trace", p.name)):
        dbs = sorted(glob.glob(str(sub / "**" / "*_results.db"), recursive=True))
        if not dbs:
            continue
        command = (sub / "command").read_text().strip() if (sub / "command").exists() else f"(run {sub.name})"
        lines.append("# " + command)
        cur = sqlite3.connect(dbs[0]).cursor()
        if sub.name == "trace":
            rows = cur.execute("select name, count(*), avg(duration), min(duration), max(duration) from kernels "
                               "group by name order by sum(duration) desc").fetchall()
            for name, n, avg, lo, hi in rows:
                if any(k in name for k in LIBRARY_KERNELS):
                    step_kernels[name] = {"n": n, "avg_us": round(avg / 1e3, 1)}
                    lines.append(f"  kern {name[:110]:110s} n={n} avg={avg / 1e3:.1f}us min={lo / 1e3:.1f} max={hi / 1e3:.1f}")
        else:
            raw = cur.execute("select kernel_name, counter_name, value from counters_collection").fetchall()
            grouped = collections.defaultdict(list)
            for kernel, counter, value in raw:
                grouped[(kernel, counter)].append(value)
            per_kernel = collections.defaultdict(dict)
            for (kernel, counter), values in grouped.items():
                if any(k in kernel for k in LIBRARY_KERNELS):
                    per_kernel[kernel][counter] = round(statistics.median(values), 1)
                    counters[kernel][counter] = per_kernel[kernel][counter]
            for kernel in sorted(per_kernel):
                lines.append(f"  pmc {kernel[:110]:110s} {per_kernel[kernel]}")
    # the kernels of a step: those that ran about once per step or more (one-off table builders ran a few times)
    most = max((k["n"] for k in step_kernels.values()), default=0)
    per_step = {name: k for name, k in step_kernels.items() if k["n"] * 4 >= most}
    fetch = sum(counters[name].get("FETCH_SIZE", 0.0) for name in per_step if name in counters)
    write = sum(counters[name].get("WRITE_SIZE", 0.0) for name in per_step if name in counters)
    have = any("FETCH_SIZE" in counters[name] for name in per_step if name in counters)
    lines.append(f"# kernels of one step: {len(per_step)}; sum of their average durations "
                 f"{sum(k['avg_us'] for k in per_step.values()):.1f} us; FETCH_SIZE {fetch:.1f} KiB + WRITE_SIZE "
                 f"{write:.1f} KiB per step = {(FETCH_SCALE * fetch + WRITE_SCALE * write) * 1024 / 1e6:.1f} MB")
    stem = side_name or PROFILE_STEMS.get(config, config)
    out = ROOT / "profiles" / (stem + ".txt")
    out.parent.mkdir(exist_ok=True)
    if side_name:  # a side experiment (runs that differ in an option): the runs as they are, no totals, no table entry
        out.write_text("\n".join(lines[:-1]) + "\n")
        print(f"wrote {out}")
        return
    out.write_text("\n".join(lines) + "\n")
    try:
        table = json.loads(TRAFFIC_FILE.read_text())
    except (OSError, ValueError):
        table = {}
    table[config] = {"profile": out.name, "fetch_kib": round(fetch, 1) if have else None,
                     "write_kib": round(write, 1) if have else None,
                     "kernels": {name[:100]: {**k, **counters.get(name, {})} for name, k in per_step.items()}}
    TRAFFIC_FILE.write_text(json.dumps(table, indent=1, sort_keys=True) + "\n")
    print(f"wrote {out} and {TRAFFIC_FILE}")


def log(*a):
    print(*a, file=sys.stderr, flush=True)


CPU_SAMPLE_SECONDS = 12.0  # the CPU baseline repeats its sample until this much time has gone by


def _repeat_for(seconds, fn):
    """Calls ``fn`` until ``seconds`` have passed (at least once); returns (passes, mean seconds per pass)."""
    t0 = time.perf_counter()
    reps = 0
    while True:
        fn()
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= seconds:
            return reps, dt / reps


def _events(n):
    return [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]


def _sleep_cycles_per_ms():
    """How many cycles of torch.cuda._sleep make one millisecond on this card."""
    probe = 2_000_000
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda._sleep(probe)
    torch.cuda.synchronize()
    a.record()
    torch.cuda._sleep(probe)
    b.record()
    torch.cuda.synchronize()
    return probe / max(a.elapsed_time(b), 1e-3)


PREROLL_MS = 300.0   # untimed work in front of the warm-up steps, whatever --warmup says
FLUSH_BYTES = 1 << 30  # written between launches of the flushed timing: 4x the 256 MB memory-side cache


def preroll(step):
    """Runs ``step`` untimed until the card has worked for PREROLL_MS: a card that has idled runs its first tens of
    milliseconds below its sustained clock, and the driver's run has only a few warm-up steps.  Returns
    (milliseconds, launches)."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n = 0
    while True:
        for _ in range(20):
            step()
        n += 20
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3
        if ms >= PREROLL_MS:
            return ms, n


def _percentile(sorted_values, q):
    return sorted_values[min(len(sorted_values) - 1, int(q * len(sorted_values)))]


def time_steps(step, steps, warmup):
    """Times exactly ``steps`` steps after ``warmup`` untimed ones.  Returns a dict: wall ms per step, per-launch
    mean / median / p20 / p80 from stream events (p20 and p80 as the reference's own timing helper reports them,
    blksprs/utils/benchmarking.py:15, :22-23), and the host's enqueue time per step.

    The per-launch figure must not contain the time the card waits for the host: a step whose kernels are
    shorter than the host's work per call leaves the stream empty between launches, and an event recorded on an
    empty stream fires at once, long before the kernel behind it is enqueued.  When the host is the slower side,
    the timed launches are therefore enqueued in chunks behind a short delay kernel, so that every event pair
    brackets kernels that are already waiting in the stream.  (Not otherwise: the card clocks down during the
    delays, which slows a long kernel.)
    """
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    host_ms = (time.perf_counter() - t0) * 1e3 / steps  # what the host needs to enqueue a step
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev = _events(steps)
    if host_ms < 0.7 * wall_ms:
        # the card is the slower side: the stream never runs empty, events between the steps see the kernels only
        for s, e in ev:
            s.record()
            step()
            e.record()
        torch.cuda.synchronize()
    else:
        per_ms = _sleep_cycles_per_ms()
        chunk = 20
        for c in range(0, steps, chunk):
            # long enough for the host to enqueue the whole chunk (the wall time per step bounds its work per step)
            torch.cuda._sleep(int(per_ms * (1.0 + 2.0 * wall_ms * chunk)))
            for s, e in ev[c:c + chunk]:
                s.record()
                step()
                e.record()
            torch.cuda.synchronize()
    per = sorted(s.elapsed_time(e) for s, e in ev)
    return {"wall_ms": wall_ms, "mean_ms": sum(per) / len(per), "median_ms": per[len(per) // 2],
            "p20_ms": _percentile(per, 0.2), "p80_ms": _percentile(per, 0.8), "host_ms": host_ms}


def time_steps_flushed(step, steps, scratch):
    """Mean per-launch ms with the caches emptied in front of every launch: FLUSH_BYTES are written between the
    launches, outside the event pair (the fill also keeps the stream busy while the host enqueues the step).  What a
    launch finds in the 256 MB memory-side cache and the L2s is then what the fill left, not its own operands from
    the launch before."""
    ev = _events(steps)
    for i, (s, e) in enumerate(ev):
        scratch.fill_(i & 1)
        s.record()
        step()
        e.record()
    torch.cuda.synchronize()
    per = sorted(s.elapsed_time(e) for s, e in ev)
    return sum(per) / len(per)


def count_host_syncs(fn):
    """Runs ``fn`` and returns (milliseconds, number of calls that made the host wait for the device: those torch's
    sync debug mode reports plus the library calls that wait for the stream themselves)."""
    import warnings
    from blksprs_amd import _capi
    inside_library = _capi.host_waits
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("warn")
    try:
        with warnings.catch_warnings(record=True) as seen:
            warnings.simplefilter("always")
            t0 = time.perf_counter()
            fn()
            torch.cuda.set_sync_debug_mode("default")
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3
    finally:
        torch.cuda.set_sync_debug_mode("default")
    return ms, sum("synchroniz" in str(w.message).lower() for w in seen) + _capi.host_waits - inside_library


# --------------------------------------------------------------------------- workloads


def matmul_workload(name, B, n, sbs, dtype, density, ensure_rows, value_scale, dev, cpu_sample_batches,
                    backward=False, check_batch=0):
    import blksprs_amd as bs
    from blksprs_amd.ops.matmul import matmul_build_layout_cache
    from oracle import blksprs_oracle as orc

    g = torch.Generator().manual_seed(0)
    lx = orc.random_layout((B, n, n), density, g, ensure_rows=ensure_rows)
    ly = orc.random_layout((B, n, n), density, g, ensure_rows=ensure_rows)
    lxd, lyd = lx.to(dev), ly.to(dev)
    lod = bs.layouting.build_sparsity_layout_matmul(lxd, lyd)
    nnz_x, nnz_y, nnz_o = int(lx.sum()), int(ly.sum()), int(lod.sum())
    gd = torch.Generator(device=dev).manual_seed(1)
    x = (torch.randn((nnz_x, sbs, sbs), generator=gd, device=dev) * value_scale).to(dtype)
    y = torch.randn((nnz_y, sbs, sbs), generator=gd, device=dev).to(dtype)
    go = (torch.randn((nnz_o, sbs, sbs), generator=gd, device=dev) / math.sqrt(n * sbs)).to(dtype)

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    cache = {}
    out = bs.ops.matmul(x, lxd, y, lyd, lod, sbs, layout_cache=cache)
    torch.cuda.synchronize()
    first_ms = (time.perf_counter() - t0) * 1e3  # holds the load of the library and of its code objects
    # the lookup tables of a second, empty cache: what a new triple of layouts costs once the library is loaded
    lut_ms, lut_syncs = count_host_syncs(lambda: matmul_build_layout_cache(None, lxd, lyd, lod))
    pairs = int(cache["contraction_pairs"].size(0))
    es = x.element_size()
    flops = pairs * 2.0 * sbs ** 3
    alg_bytes = (nnz_x + nnz_y + nnz_o) * sbs * sbs * es
    log(f"[{name}] nnz_x={nnz_x} nnz_y={nnz_y} nnz_o={nnz_o} ({nnz_o / (B * n * n):.1%} of output) "
        f"pairs={pairs} (mean {pairs / max(nnz_o, 1):.2f}/block) flops={flops / 1e9:.2f}G "
        f"algorithmic bytes={alg_bytes / 1e6:.1f}MB; first call {first_ms:.2f} ms, lookup tables of a fresh cache "
        f"{lut_ms:.2f} ms with {lut_syncs} host syncs")

    generations = ROW_GENERATIONS if not backward and cache["plan"].row_records is not None else None
    if generations is not None:
        # measurement only: the launch ends after the first entries of every XCD's list (32 compute units per XCD
        # take 32 entries at a time; entry k of XCD c sits at position 8 k + c), the rest of the output is not
        # computed, so the result is not checked and the rates of the line mean nothing: the counters per launch do
        plan = cache["plan"]
        plan.row_records = plan.row_records[:256 * generations * plan.row_items]
        log(f"[{name}] row kernel limited to {plan.row_records.size(0)} of its work table's entries")

    bs.utils.disable_validation()
    if backward:
        xg, yg = x.requires_grad_(True), y.requires_grad_(True)
        graph_out = bs.ops.matmul(xg, lxd, yg, lyd, lod, sbs, layout_cache=cache)

        def step():  # dX = dO Y^T and dY = X^T dO, nothing else
            return torch.autograd.grad(graph_out, (xg, yg), go, retain_graph=True)

        flops = 2.0 * flops
        alg_bytes = (2 * nnz_o + 2 * nnz_x + 2 * nnz_y) * sbs * sbs * es
    else:
        def step():
            return bs.ops.matmul(x, lxd, y, lyd, lod, sbs, layout_cache=cache)

    def slices(b):
        sl = lambda lay, t: t[int(lay[:b].sum()):int(lay[:b + 1].sum())].detach().cpu()
        lo = lod.cpu()
        return lo, sl(lx, x), sl(ly, y), sl(lo, go), sl

    def check():
        """Batch entry ``check_batch`` against the CPU oracle (fp64 accumulation of the rounded operands)."""
        b = check_batch
        lo, xs, ys, gs, sl = slices(b)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        close = lambda got, want: bool(torch.allclose(got.double().cpu(), want.double(), rtol=tol, atol=tol))
        lxb, lyb, lob = lx[b:b + 1].numpy(), ly[b:b + 1].numpy(), lo[b:b + 1].numpy()
        if not backward:
            want = orc.matmul(xs.double(), lxb, ys.double(), lyb, lob, sbs, acc_dtype=torch.float64)
            return close(sl(lo, step()), want)
        x64, y64 = xs.double().requires_grad_(True), ys.double().requires_grad_(True)
        orc.matmul(x64, lxb, y64, lyb, lob, sbs, acc_dtype=torch.float64).backward(gs.double())
        dx, dy = step()
        return close(sl(lx, dx), x64.grad) and close(sl(ly, dy), y64.grad)

    def cpu_baseline():
        nb = min(cpu_sample_batches, B)
        sl = lambda lay, t: t[:int(lay[:nb].sum())].detach().float().cpu()
        lo = lod.cpu()
        xs, ys = sl(lx, x), sl(ly, y)
        reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.matmul(
            xs, lx[:nb].numpy(), ys, ly[:nb].numpy(), lo[:nb].numpy(), sbs, acc_dtype=torch.float32))
        sample_pairs = int(torch.einsum("bik,bkj,bij->", lx[:nb].float(), ly[:nb].float(), lo[:nb].float()))
        return {"value": sample_pairs * 2.0 * sbs ** 3 / dt / 1e12, "unit": "TFLOP/s",
                "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"{'forward of ' if backward else ''}{nb} of {B} batches x {reps} passes, dense-masked fp32 "
                          f"torch matmul + to_sparse, {dt * reps:.1f} s"}

    dt_name = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}[dtype]
    if backward:
        kernel = ("matmul_lines_kernel (two launches: dX by rows of dO, dY by its columns)"
                  if sbs == 64 and dtype != torch.float32 else
                  "matmul_mfma_kernel (two launches: dX with y read transposed, dY with x read transposed)")
    elif sbs > 16:
        kernel = "matmul_rows_kernel" if sbs == 64 and dtype != torch.float32 else "matmul_mfma_kernel"
    else:
        kernel = "matmul_small16_kernel" if dtype != torch.float32 else "matmul_small_kernel"
    # 172 FLOP per byte at sbs 64 and 25 % density: below the balance of the 16-bit matrix cores (312 FLOP/B), above
    # that of the fp32 ones (20 FLOP/B): fp32 products of large problems are bound by the fp32 matrix-core peak
    bound = "mfma" if dtype == torch.float32 and sbs >= 32 and B * n * sbs >= 16 * 4096 else "hbm"
    if generations is not None:
        check = lambda: None
    return dict(step=step, flops=flops, alg_bytes=alg_bytes, dtype=dt_name, bound=bound, cpu_baseline=cpu_baseline,
                check=check, kernel=kernel,
                config={"workload": name, "B": B, "M": n * sbs, "K": n * sbs, "N": n * sbs,
                        "sparsity_block_size": sbs, "density": density, "nnz_x": nnz_x, "nnz_y": nnz_y,
                        "nnz_o": nnz_o, "block_pairs": pairs, "first_call_ms": round(first_ms, 3),
                        "lut_build_ms": round(lut_ms, 3), "lut_build_host_syncs": lut_syncs})


def linear_workload(dev):
    """``apply_torch_linear_cached`` on configuration 2's x operand: a 4096 -> 4096 linear layer with bias over a
    bf16 input of 16 x 4096 x 4096 at 25 % block density (dense output, one un-replicated copy of the weight)."""
    import blksprs_amd as bs
    from oracle import blksprs_oracle as orc

    B, n, sbs = 16, 64, 64
    g = torch.Generator().manual_seed(0)
    layout = orc.random_layout((B, n, n), 0.25, g)
    ld = layout.to(dev)
    nnz = int(layout.sum())
    gd = torch.Generator(device=dev).manual_seed(1)
    x = (torch.randn((nnz, sbs, sbs), generator=gd, device=dev) * 0.25).to(torch.bfloat16)
    torch.manual_seed(2)
    linear = torch.nn.Linear(n * sbs, n * sbs, bias=True, device=dev, dtype=torch.bfloat16)
    cache = {}
    with torch.no_grad():
        bs.utils.apply_torch_linear_cached(x, ld, sbs, linear, layout_cache=cache)
    nnz_o = B * n * n
    flops = nnz * n * 2.0 * sbs ** 3
    alg_bytes = (nnz + n * n + nnz_o) * sbs * sbs * 2
    bs.utils.disable_validation()

    def step():
        with torch.no_grad():
            return bs.utils.apply_torch_linear_cached(x, ld, sbs, linear, layout_cache=cache)

    def cpu_baseline():
        nb = 1
        cnt = int(layout[:nb].sum())
        xs = x[:cnt].float().cpu()
        w, b = linear.weight.detach().float().cpu(), linear.bias.detach().float().cpu()
        reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.linear(xs, layout[:nb].numpy(), w, b, sbs))
        return {"value": cnt * n * 2.0 * sbs ** 3 / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                "kind": "port", "sample": f"{nb} of {B} batches x {reps} passes, dense fp64 torch linear + to_sparse, "
                                          f"{dt * reps:.1f} s (flops counted over non-zero input blocks)"}

    return dict(step=step, flops=flops, alg_bytes=alg_bytes, dtype="bf16", bound="mfma", cpu_baseline=cpu_baseline,
                kernel="matmul_rows_kernel",
                config={"workload": "p1_apply_torch_linear_bf16", "B": B, "rows": n * sbs, "in_features": n * sbs,
                        "out_features": n * sbs, "sparsity_block_size": sbs, "density": 0.25, "nnz_x": nnz,
                        "nnz_o": nnz_o})


def softmax_workload(dev, backward=False):
    import blksprs_amd as bs
    from oracle import blksprs_oracle as orc

    B, n, sbs = 32, 32, 64
    g = torch.Generator().manual_seed(0)
    tri = torch.tril(torch.ones((n, n), dtype=torch.bool))
    layout = tri.unsqueeze(0) | ((torch.rand((B, n, n), generator=g) < 0.1) & ~tri)
    ld = layout.to(dev)
    nnz = int(layout.sum())
    x = torch.randn((nnz, sbs, sbs), device=dev) * 2.0  # N(0, 4): sigma = 2
    go = torch.randn((nnz, sbs, sbs), device=dev)
    cache = {}
    bs.ops.softmax(x, ld, sbs, layout_cache=cache)
    lut_ms, lut_syncs = count_host_syncs(lambda: bs.ops.softmax(x, ld, sbs, layout_cache={}))
    alg_bytes = (3 if backward else 2) * nnz * sbs * sbs * 4
    log(f"[c3] nnz={nnz} algorithmic bytes={alg_bytes / 1e6:.1f}MB; call with a fresh cache {lut_ms:.2f} ms, "
        f"{lut_syncs} host syncs")
    bs.utils.disable_validation()
    if backward:
        xg = x.requires_grad_(True)
        graph_out = bs.ops.softmax(xg, ld, sbs, layout_cache=cache)

        def step():  # reads y and dy, writes dx
            return torch.autograd.grad(graph_out, xg, go, retain_graph=True)[0]
    else:
        def step():
            return bs.ops.softmax(x, ld, sbs, layout_cache=cache)

    def check():
        """Batch entry 0 against the CPU oracle at rtol = atol = 1e-5."""
        cnt = int(layout[:1].sum())
        xs = x[:cnt].detach().cpu()
        ys = orc.softmax(xs, layout[:1].numpy(), sbs)
        want = orc.softmax_backward(go[:cnt].cpu(), ys, layout[:1].numpy(), sbs) if backward else ys
        return bool(torch.allclose(step()[:cnt].cpu().double(), want.double(), rtol=1e-5, atol=1e-5))

    def cpu_baseline():
        nb = 8
        cnt = int(layout[:nb].sum())
        xs = x[:cnt].detach().cpu()
        reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.softmax(xs, layout[:nb].numpy(), sbs))
        return {"value": 2 * cnt * sbs * sbs * 4 / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                "kind": "port", "sample": f"{'forward of ' if backward else ''}{nb} of {B} batches x {reps} passes, "
                                          f"dense -inf-masked torch softmax (fp64), {dt * reps:.1f} s"}

    return dict(step=step, flops=0.0, alg_bytes=alg_bytes, dtype="f32", bound="hbm", cpu_baseline=cpu_baseline,
                check=check, kernel="softmax_bwd_kernel" if backward else "softmax_fwd_kernel",
                config={"workload": "c3_softmax_fp32" + ("_backward" if backward else ""), "B": B, "rows": n * sbs,
                        "cols": n * sbs, "sparsity_block_size": sbs, "nnz": nnz, "lut_build_ms": round(lut_ms, 3),
                        "lut_build_host_syncs": lut_syncs})


def movement_workload(dev, which):
    """The HBM-bound rows next to the hot path, at the size of configuration 2's x operand (bf16, 25 % of
    16 x 64 x 64 blocks of 64): ``transpose``, ``row_wise_sum`` and ``row_wise_add`` of the compressed x, and
    ``build_sparsity_layout`` of its dense form (16 x 4096 x 4096 bf16)."""
    import blksprs_amd as bs
    from oracle import blksprs_oracle as orc

    B, n, sbs = 16, 64, 64
    g = torch.Generator().manual_seed(0)
    layout = orc.random_layout((B, n, n), 0.25, g)
    ld = layout.to(dev)
    nnz = int(layout.sum())
    gd = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn((nnz, sbs, sbs), device=dev, dtype=torch.bfloat16, generator=gd)
    bs.utils.disable_validation()
    if which == "transpose":
        cache = {}
        bs.ops.transpose(x, ld, sbs, layout_cache=cache)
        alg_bytes = 2 * nnz * sbs * sbs * 2

        def step():
            return bs.ops.transpose(x, ld, sbs, layout_cache=cache)

        def cpu_baseline():
            nb = 2
            cnt = int(layout[:nb].sum())
            xs = x[:cnt].cpu()
            reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.transpose(xs, layout[:nb].numpy(), sbs))
            return {"value": 2 * cnt * sbs * sbs * 2 / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                    "kind": "port", "sample": f"{nb} of {B} batches x {reps} passes, per-block torch transpose, {dt * reps:.1f} s"}

        def check():
            cnt = int(layout[:1].sum())
            want, _ = orc.transpose(x[:cnt].cpu(), layout[:1].numpy(), sbs)
            return bool(torch.equal(step()[0][:cnt].cpu(), want))

        return dict(step=step, flops=0.0, alg_bytes=alg_bytes, dtype="bf16", bound="hbm", cpu_baseline=cpu_baseline,
                    check=check, kernel="transpose_blocks16_kernel",
                    config={"workload": "t1_transpose_bf16", "B": B, "rows": n * sbs, "cols": n * sbs,
                            "sparsity_block_size": sbs, "nnz": nnz})
    if which in ("row_sum", "row_add"):
        n_rows = int(layout.any(-1).sum())
        lnp = layout.numpy()
        nb = 2
        cnt = int(layout[:nb].sum())
        xs = x[:cnt].cpu()
        if which == "row_sum":
            alg_bytes = (nnz + n_rows) * sbs * sbs * 2

            def step():
                return bs.ops.misc.row_wise_sum(x, ld, sbs)

            def cpu_baseline():
                reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.row_wise_reduce(xs, lnp[:nb], sbs, "sum"))
                return {"value": (cnt + nb * n) * sbs * sbs * 2 / dt / 1e9, "unit": "GB/s",
                        "cores": torch.get_num_threads(), "kind": "port",
                        "sample": f"{nb} of {B} batches x {reps} passes, per-block torch sums, {dt * reps:.1f} s"}

            def check():
                want = orc.row_wise_reduce(xs, lnp[:nb], sbs, "sum")[0]
                got = step()[0][:want.size(0)].cpu()
                return bool(torch.allclose(got.double(), want.double(), rtol=2e-2, atol=2e-2))

            return dict(step=step, flops=0.0, alg_bytes=alg_bytes, dtype="bf16", bound="hbm",
                        cpu_baseline=cpu_baseline, check=check, kernel="row_reduce_kernel",
                        config={"workload": "r1_row_wise_sum_bf16", "B": B, "rows": n * sbs, "cols": n * sbs,
                                "sparsity_block_size": sbs, "nnz": nnz})
        y = torch.randn((n_rows, sbs, 1), device=dev, dtype=torch.bfloat16, generator=gd)
        alg_bytes = 2 * nnz * sbs * sbs * 2 + n_rows * sbs * 2
        ys = y[:nb * n].cpu()

        def step():
            return bs.ops.misc.row_wise_add(x, ld, y, sbs)

        def cpu_baseline():
            reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.row_wise_add(xs, lnp[:nb], ys, sbs))
            return {"value": 2 * cnt * sbs * sbs * 2 / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                    "kind": "port",
                    "sample": f"{nb} of {B} batches x {reps} passes, per-block torch adds, {dt * reps:.1f} s"}

        def check():
            want = orc.row_wise_add(xs, lnp[:nb], ys, sbs)
            return bool(torch.allclose(step()[:cnt].cpu().double(), want.double(), rtol=2e-2, atol=2e-2))

        return dict(step=step, flops=0.0, alg_bytes=alg_bytes, dtype="bf16", bound="hbm", cpu_baseline=cpu_baseline,
                    check=check, kernel="row_add_kernel",
                    config={"workload": "r2_row_wise_add_bf16", "B": B, "rows": n * sbs, "cols": n * sbs,
                            "sparsity_block_size": sbs, "nnz": nnz})
    dense = bs.ops.to_dense(x, ld, sbs)
    if which in ("to_sparse", "to_dense"):
        nb = 2
        cnt = int(layout[:nb].sum())
        lnp = layout.numpy()
        cache = {}
        if which == "to_sparse":
            bs.ops.to_sparse(dense, ld, sbs, layout_cache=cache)
            alg_bytes = 2 * nnz * sbs * sbs * 2

            def step():
                return bs.ops.to_sparse(dense, ld, sbs, layout_cache=cache)

            ds = dense[:nb].cpu()

            def cpu_baseline():
                reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.to_sparse(ds, lnp[:nb], sbs))
                return {"value": 2 * cnt * sbs * sbs * 2 / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                        "kind": "port", "sample": f"{nb} of {B} batches x {reps} passes, torch reshape / permute / "
                                                  f"boolean index, {dt * reps:.1f} s"}

            check = lambda: bool(torch.equal(step()[:cnt].cpu(), orc.to_sparse(ds, lnp[:nb], sbs)))
            kernel, workload = "to_sparse_kernel", "v1_to_sparse_bf16"
        else:
            bs.ops.to_dense(x, ld, sbs, layout_cache=cache)
            alg_bytes = dense.numel() * 2 + nnz * sbs * sbs * 2

            def step():
                return bs.ops.to_dense(x, ld, sbs, layout_cache=cache)

            xs = x[:cnt].cpu()

            def cpu_baseline():
                reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.to_dense(xs, lnp[:nb], sbs))
                return {"value": (nb * n * n + cnt) * sbs * sbs * 2 / dt / 1e9, "unit": "GB/s",
                        "cores": torch.get_num_threads(), "kind": "port",
                        "sample": f"{nb} of {B} batches x {reps} passes, torch fill / boolean index / permute, "
                                  f"{dt * reps:.1f} s"}

            check = lambda: bool(torch.equal(step()[:nb].cpu(), orc.to_dense(xs, lnp[:nb], sbs)))
            kernel, workload = "to_dense_kernel", "v2_to_dense_bf16"
        return dict(step=step, flops=0.0, alg_bytes=alg_bytes, dtype="bf16", bound="hbm", cpu_baseline=cpu_baseline,
                    check=check, kernel=kernel, config={"workload": workload, "B": B, "rows": n * sbs, "cols": n * sbs,
                                           "sparsity_block_size": sbs, "nnz": nnz})
    alg_bytes = dense.numel() * 2 + B * n * n

    def step():
        return bs.layouting.build_sparsity_layout(dense, sbs)

    def cpu_baseline():
        nb = 2
        ds = dense[:nb].cpu()
        reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.build_sparsity_layout(ds, sbs))
        return {"value": ds.numel() * 2 / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"{nb} of {B} batches x {reps} passes, torch != 0 and any over blocks, {dt * reps:.1f} s"}

    def check():
        want = torch.from_numpy(orc.build_sparsity_layout(dense[:1].cpu(), sbs))
        return bool(torch.equal(step()[:1].cpu().to(torch.bool), want.to(torch.bool)))

    return dict(step=step, flops=0.0, alg_bytes=alg_bytes, dtype="bf16", bound="hbm", cpu_baseline=cpu_baseline,
                check=check, kernel="layout_from_dense_kernel",
                config={"workload": "l1_build_sparsity_layout_bf16", "B": B, "rows": n * sbs, "cols": n * sbs,
                        "sparsity_block_size": sbs, "active_blocks": nnz})


def attention_workload(dev, backward, native_causal=False):
    import blksprs_amd as bs
    from oracle import blksprs_oracle as orc

    BH, n, sbs, nh = 64, 128, 64, 2
    g = torch.Generator().manual_seed(0)
    la = orc.bigbird_layout(BH, n, g)
    lmask = la & torch.ones((n, n), dtype=torch.bool).triu()
    nnz = int(la.sum())
    lad, lmd = la.to(dev), lmask.to(dev)
    full = torch.ones((BH, n, nh), dtype=torch.bool, device=dev)
    # causal mask inside every mask block (key position > query position), built on the device
    midx = torch.nonzero(lmd)
    r = torch.arange(sbs, device=dev)
    qpos = midx[:, 1].view(-1, 1, 1) * sbs + r.view(1, -1, 1)
    kpos = midx[:, 2].view(-1, 1, 1) * sbs + r.view(1, 1, -1)
    mask = kpos > qpos
    q, k, v = (torch.randn((BH * n * nh, sbs, sbs), device=dev).to(torch.bfloat16) for _ in range(3))
    d_o = torch.randn((BH * n * nh, sbs, sbs), device=dev).to(torch.bfloat16)
    cache = {}
    if backward:
        q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    # the same causal attention two ways (blksprs/ops/flash_attention.py:1128-1142): an explicit mask tensor (the
    # headline), or the native predicate on causal_lengths, without any mask tensor
    lengths = torch.full((BH,), n * sbs, dtype=torch.int64, device=dev)
    if native_causal:
        mask_args = dict(causal_lengths=lengths)
    else:
        mask_args = dict(attention_mask=mask, sparsity_layout_mask=lmd)
    bs.ops.flash_attention(q, full, k, full, v, full, lad, sbs, layout_cache=cache, **mask_args)
    fwd_flops = nnz * 4.0 * sbs * sbs * (nh * sbs)
    flops = fwd_flops * (3.5 if backward else 1.0)
    alg_bytes = 4 * BH * n * nh * sbs * sbs * 2 + (0 if native_causal else int(lmask.sum()) * sbs * sbs)
    # pairs in which some score survives the mask: the others are in the layout (and in the metric's flop count,
    # which follows the reference, whose kernels visit them) but the kernels here neither fetch nor compute them
    live_pairs = int((la & torch.ones((n, n), dtype=torch.bool).tril()).sum())
    log(f"[c4] layout blocks={nnz} ({nnz / (BH * n):.1f}/row) causal-useful={live_pairs} "
        f"mask blocks={int(lmask.sum())} fwd flops={fwd_flops / 1e9:.1f}G")
    bs.utils.disable_validation()

    def step():
        o = bs.ops.flash_attention(q, full, k, full, v, full, lad, sbs, layout_cache=cache, **mask_args)
        if backward:
            q.grad = k.grad = v.grad = None
            o.backward(d_o)
        return o

    def check():
        """Head 0 against the CPU oracle (dense masked attention, fp32 accumulation) at rtol = atol = 2e-2."""
        cnt = int(lmask[:1].sum())
        fl = full[:1].cpu().numpy()
        leaves = [t[:n * nh].detach().float().cpu().requires_grad_(backward) for t in (q, k, v)]
        if native_causal:
            want = orc.flash_attention(leaves[0], fl, leaves[1], fl, leaves[2], fl, la[:1].numpy(), sbs,
                                       causal_lengths=lengths[:1].cpu())
        else:
            want = orc.flash_attention(leaves[0], fl, leaves[1], fl, leaves[2], fl, la[:1].numpy(), sbs,
                                       mask=mask[:cnt].cpu(), layout_mask=lmask[:1].numpy())
        close = lambda got, ref: bool(torch.allclose(got[:n * nh].detach().float().cpu(), ref, rtol=2e-2, atol=2e-2))
        ok = close(step(), want.detach())
        if backward:
            want.backward(d_o[:n * nh].float().cpu())
            ok = ok and all(close(t.grad, ref.grad) for t, ref in zip((q, k, v), leaves))
        return ok

    def cpu_baseline():
        heads = 1
        qs, ks, vs = (t[:heads * n * nh].detach().float().cpu() for t in (q, k, v))
        cnt = int(lmask[:heads].sum())
        fl = full[:heads].cpu().numpy()
        mk = mask[:cnt].cpu()
        reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.flash_attention(
            qs, fl, ks, fl, vs, fl, la[:heads].numpy(), sbs, mask=mk, layout_mask=lmask[:heads].numpy()))
        return {"value": int(la[:heads].sum()) * 4.0 * sbs * sbs * nh * sbs / dt / 1e12, "unit": "TFLOP/s",
                "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"forward of {heads} of {BH} heads x {reps} passes, dense masked fp32 torch attention, "
                          f"{dt * reps:.1f} s"}

    return dict(step=step, flops=flops, alg_bytes=alg_bytes, dtype="bf16", bound="mfma", cpu_baseline=cpu_baseline,
                check=check, executed_flops=flops * live_pairs / nnz,
                kernel="attn_fwd_mfma_kernel" if not backward else
                "attn_fwd_mfma_kernel + attn_bwd_delta_kernel + attn_bwd_kv8_walk_kernel + attn_bwd_dq_kernel (one step; the mask_dead / records / order kernels ran once, in the warm-up)",
                config={"workload": "c4_flash_attention_bf16" + ("_fwd_bwd" if backward else "_fwd")
                        + ("_causal_lengths" if native_causal else ""),
                        "batch_heads": BH, "seq": n * sbs, "head_dim": nh * sbs, "sparsity_block_size": sbs,
                        "layout_blocks": nnz,
                        "mask": "native causal predicate (causal_lengths)" if native_causal else "explicit causal blocks"})


def reference_attention_benchmark(dev, m=2048, backward=False):
    """The reference's own attention benchmark (test/cases/test_blocksparse.py:1481-1579): fp32, batch * heads = 8,
    sequence ``m``, head_dim 64, sbs 32, half of the attention layout's blocks active (every row at least one).  The
    step is ``flash_attention``; the same result by ``matmul -> scale -> softmax -> matmul`` of this library is timed
    next to it (``unfused_ms``), and the reference asserts flash <= 1.1 x unfused."""
    import blksprs_amd as bs
    from oracle import blksprs_oracle as orc

    bh, hd, sbs = 8, 64, 32
    n, nh = m // sbs, hd // sbs
    g = torch.Generator().manual_seed(0)
    la = orc.random_layout((bh, n, n), 0.5, g, ensure_rows=True).to(dev)
    lqkv = torch.ones((bh, n, nh), dtype=torch.bool, device=dev)
    gd = torch.Generator(device=dev).manual_seed(1)
    q, k, v = (bs.ops.to_sparse(torch.randn((bh, m, hd), generator=gd, device=dev), lqkv, sbs) for _ in range(3))
    d_o = torch.randn(q.shape, generator=gd, device=dev)
    if backward:
        q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    k_t, lkt = bs.ops.transpose(k, lqkv, sbs)
    lo = bs.layouting.build_sparsity_layout_matmul(la, lqkv)
    scale = 1.0 / hd ** 0.5
    caches = [{}, {}, {}, {}]

    def unfused():
        k_now, _ = bs.ops.transpose(k, lqkv, sbs) if backward else (k_t, None)
        scores = bs.ops.matmul(q, lqkv, k_now, lkt, la, sbs, layout_cache=caches[0]) * scale
        probs = bs.ops.softmax(scores, la, sbs, layout_cache=caches[1])
        out = bs.ops.matmul(probs, la, v, lqkv, lo, sbs, layout_cache=caches[2])
        if backward:
            q.grad = k.grad = v.grad = None
            out.backward(d_o)
        return out

    def step():
        out = bs.ops.flash_attention(q, lqkv, k, lqkv, v, lqkv, la, sbs, scale=scale, layout_cache=caches[3])
        if backward:
            q.grad = k.grad = v.grad = None
            out.backward(d_o)
        return out

    unfused_out = unfused().detach()
    unfused_grads = [t.grad.clone() for t in (q, k, v)] if backward else []
    same = bool(torch.allclose(unfused_out, step().detach(), rtol=1e-4, atol=1e-4))
    same = same and all(torch.allclose(g, t.grad, rtol=1e-3, atol=1e-4) for g, t in zip(unfused_grads, (q, k, v)))
    bs.utils.disable_validation()
    for _ in range(20):
        unfused()
    torch.cuda.synchronize()
    ev = _events(20)
    for s_, e_ in ev:
        s_.record()
        unfused()
        e_.record()
    torch.cuda.synchronize()
    unfused_ms = sorted(a.elapsed_time(b) for a, b in ev)[10]
    nnz = int(la.sum())
    flops = nnz * 4.0 * sbs * sbs * hd * (3.5 if backward else 1.0)
    alg_bytes = (9 if backward else 4) * bh * m * hd * 4

    def check():
        """Batch entry 0 against the CPU oracle at rtol = atol = 1e-5 (gradients: 2e-5 on O(1) values), and flash
        against the unfused path."""
        cnt = n * nh
        fl = lqkv[:1].cpu().numpy()
        leaves = [t[:cnt].detach().cpu().requires_grad_(backward) for t in (q, k, v)]
        want = orc.flash_attention(leaves[0], fl, leaves[1], fl, leaves[2], fl, la[:1].cpu().numpy(), sbs, scale=scale)
        ok = same and bool(torch.allclose(step()[:cnt].detach().cpu(), want.detach(), rtol=1e-5, atol=1e-5))
        if backward:
            want.backward(d_o[:cnt].cpu())
            ok = ok and all(torch.allclose(t.grad[:cnt].cpu(), ref.grad, rtol=2e-5, atol=2e-5)
                            for t, ref in zip((q, k, v), leaves))
        return ok

    def cpu_baseline():
        cnt = n * nh
        fl = lqkv[:1].cpu().numpy()
        qs, ks, vs, lay = (*(t[:cnt].detach().cpu() for t in (q, k, v)), la[:1].cpu().numpy())
        reps, dt = _repeat_for(CPU_SAMPLE_SECONDS, lambda: orc.flash_attention(qs, fl, ks, fl, vs, fl, lay, sbs,
                                                                                scale=scale))
        return {"value": int(la[:1].sum()) * 4.0 * sbs * sbs * hd / dt / 1e12, "unit": "TFLOP/s",
                "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"1 of {bh} heads x {reps} passes, dense masked fp32 torch attention, {dt * reps:.1f} s"}

    return dict(step=step, flops=flops, alg_bytes=alg_bytes, dtype="f32", bound="mfma", cpu_baseline=cpu_baseline,
                check=check, kernel="attn_fwd_f32mma_kernel" + (" + attn_f32mma_delta / dkdv / dq kernels" if backward else ""),
                config={"workload": "a1_flash_attention_fp32_reference_benchmark" + ("_fwd_bwd" if backward else ""),
                        "batch_heads": bh, "seq": m,
                        "head_dim": hd, "sparsity_block_size": sbs, "layout_blocks": nnz,
                        "unfused_ms": round(unfused_ms, 4)})


def make_workload(name, dev):
    if name == "c1":
        return matmul_workload("c1_matmul_fp32", 2, 8, 32, torch.float32, 0.5, True, 1.0, dev, 2)
    if name == "c2":
        return matmul_workload("c2_matmul_bf16", 16, 64, 64, torch.bfloat16, 0.25, False, 1.0 / 64.0, dev, 16,
                               check_batch=3)
    if name == "c2bwd":
        return matmul_workload("c2_matmul_bf16_backward", 16, 64, 64, torch.bfloat16, 0.25, False, 1.0 / 64.0, dev,
                               16, backward=True, check_batch=3)
    # the C2 problem (4096^3, 25 % density, product layout) off the one shape the row kernel takes: other block
    # sizes and fp32 run on the tile kernel (blksprs/ops/matmul.py:148-253 serves every dtype and block size)
    if name == "m32":
        return matmul_workload("c2_problem_bf16_sbs32", 16, 128, 32, torch.bfloat16, 0.25, False, 1.0 / 64.0, dev, 4,
                               check_batch=3)
    if name == "m128":
        return matmul_workload("c2_problem_bf16_sbs128", 16, 32, 128, torch.bfloat16, 0.25, False, 1.0 / 64.0, dev, 4,
                               check_batch=3)
    if name == "mf32":
        return matmul_workload("c2_problem_fp32_sbs64", 16, 64, 64, torch.float32, 0.25, False, 1.0 / 64.0, dev, 4,
                               check_batch=3)
    if name == "c3":
        return softmax_workload(dev)
    if name == "c3bwd":
        return softmax_workload(dev, backward=True)
    if name == "c4":
        return attention_workload(dev, backward=False)
    if name == "c4bwd":
        return attention_workload(dev, backward=True)
    if name == "c4cl":
        return attention_workload(dev, backward=False, native_causal=True)
    if name == "c4clbwd":
        return attention_workload(dev, backward=True, native_causal=True)
    if name == "a1":
        return reference_attention_benchmark(dev)
    if name == "a1bwd":
        return reference_attention_benchmark(dev, backward=True)
    if name == "c5":
        return matmul_workload("c5_matmul_fp16", 64, 128, 16, torch.float16, 0.05, True, 1.0, dev, 8)
    if name == "t1":
        return movement_workload(dev, "transpose")
    if name == "l1":
        return movement_workload(dev, "layout")
    if name == "v1":
        return movement_workload(dev, "to_sparse")
    if name == "v2":
        return movement_workload(dev, "to_dense")
    if name == "p1":
        return linear_workload(dev)
    if name == "r1":
        return movement_workload(dev, "row_sum")
    if name == "r2":
        return movement_workload(dev, "row_add")
    raise SystemExit(f"unknown config {name}")


CONFIGS = ["a1", "a1bwd", "c1", "c2", "c2bwd", "c3", "c3bwd", "c4", "c4bwd", "c4cl", "c4clbwd", "c5", "m32", "m128", "mf32", "t1", "l1", "r1", "r2", "p1", "v1", "v2"]
# the configurations a default run times behind the headline one, with fewer steps (their roofline objects ride
# along in the same JSON line so that they are timed by whoever runs the script, not quoted from elsewhere)
COMPANIONS = ["c2bwd", "c4", "c4cl", "c4bwd", "c3", "c5"]


ROW_GENERATIONS = None  # --row-generations


def measure(config, dev, steps, warmup, scratch):
    """Builds the workload, checks a sample against the oracle, times it.  Returns (workload, result dict)."""
    import blksprs_amd as bs

    w = make_workload(config, dev)
    try:
        correct = w["check"]() if "check" in w else None
    finally:
        bs.utils.disable_validation()
    preroll_ms, preroll_launches = preroll(w["step"])
    t = time_steps(w["step"], steps, warmup)
    flushed_ms = time_steps_flushed(w["step"], min(steps, 50), scratch)
    mean_ms = t["mean_ms"]
    if w["bound"] == "hbm":
        gbs = w["alg_bytes"] / (mean_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": round(gbs / PEAK_HBM_GBS, 4)}
        roofline["frac_flushed"] = round(w["alg_bytes"] / (flushed_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
    else:
        ach = w["flops"] / (mean_ms * 1e-3) / 1e12
        peak = PEAK_MFMA_TFLOPS[w["dtype"]]
        roofline = {"bound": "mfma", "achieved": round(ach, 1), "peak": peak, "unit": "TFLOP/s",
                    "frac": round(ach / peak, 4)}
        roofline["frac_flushed"] = round(w["flops"] / (flushed_ms * 1e-3) / 1e12 / peak, 4)
    if "executed_flops" in w:
        # the matrix-core work the kernels really do (pairs that the mask rules out as a whole are skipped): this,
        # not the metric's count over all pairs of the layout, is the utilisation of the matrix cores
        executed = w["executed_flops"] / (mean_ms * 1e-3) / 1e12
        roofline["achieved_executed"] = round(executed, 1)
        roofline["frac_executed"] = round(executed / roofline["peak"], 4)
    roofline["traffic"] = traffic_bytes(config)
    roofline["algorithmic_bytes"] = int(w["alg_bytes"])
    roofline["kernel"] = w["kernel"]
    roofline["launch_ms_mean"] = round(mean_ms, 4)
    roofline["launch_ms_median"] = round(t["median_ms"], 4)
    roofline["launch_ms_p20"] = round(t["p20_ms"], 4)
    roofline["launch_ms_p80"] = round(t["p80_ms"], 4)
    roofline["launch_ms_flushed"] = round(flushed_ms, 4)  # caches emptied in front of every launch
    roofline["host_ms_per_step"] = round(t["host_ms"], 4)  # what the host needs to enqueue one step
    roofline["preroll_ms"] = round(preroll_ms, 1)
    roofline["preroll_launches"] = preroll_launches
    return w, {"wall_ms": t["wall_ms"], "roofline": roofline, "correct": correct}


def measured_ceilings(dev):
    """What plain library kernels reach on this card, next to the published peaks the roofline fractions use: a
    dense bf16 and fp32 GEMM of 8192^3 through torch (hipBLASLt / rocBLAS) and a device-to-device copy of 2 GiB."""
    def timed(fn, reps):
        for _ in range(3):
            fn()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for s, e in ev:
            s.record()
            fn()
            e.record()
        torch.cuda.synchronize()
        return sorted(s.elapsed_time(e) for s, e in ev)[reps // 2]

    out = {}
    n = 8192
    for name, dtype in (("dense_gemm_bf16_tflops", torch.bfloat16), ("dense_gemm_fp32_tflops", torch.float32)):
        a = torch.randn((n, n), device=dev, dtype=dtype)
        b = torch.randn((n, n), device=dev, dtype=dtype)
        c = torch.empty((n, n), device=dev, dtype=dtype)
        ms = timed(lambda: torch.matmul(a, b, out=c), 10)
        out[name] = round(2.0 * n ** 3 / (ms * 1e-3) / 1e12, 1)
        del a, b, c
    src = torch.empty(2 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    ms = timed(lambda: dst.copy_(src), 10)
    out["copy_2gib_read_plus_write_gbs"] = round(2.0 * src.numel() / (ms * 1e-3) / 1e9, 1)
    # one direction at a time over the same 2 GiB: a kernel that only reads (this library's layout builder: every
    # byte once, one byte written per 8 KiB read) and one that only writes (torch's fill)
    import blksprs_amd as bs
    dense = src.view(torch.bfloat16).view(16, 8192, 8192)
    ms = timed(lambda: bs.layouting.build_sparsity_layout(dense, 64), 10)
    out["read_2gib_gbs"] = round(src.numel() / (ms * 1e-3) / 1e9, 1)
    ms = timed(lambda: dst.zero_(), 10)
    out["write_2gib_gbs"] = round(dst.numel() / (ms * 1e-3) / 1e9, 1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default=None, choices=CONFIGS,
                    help="one configuration only; without it: c2 as the headline, then " + ", ".join(COMPANIONS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--summarise", default=None, metavar="DIR",
                    help="no timing: write the summary under profiles/ (and the entry of profiles/traffic.json) of "
                         "--config from rocprofv3's output in DIR (sub-directories trace, fetch, write, ...)")
    ap.add_argument("--row-generations", type=int, default=None, metavar="G",
                    help="measurement of the row kernel's memory traffic: launch only the first 32 G entries of every "
                         "XCD's work list (forward matmul configurations on the row kernel; result unchecked)")
    ap.add_argument("--summary-name", default=None, metavar="STEM",
                    help="with --summarise: write profiles/STEM.txt (the runs of a side experiment as they are) and "
                         "leave profiles/traffic.json alone")
    ap.add_argument("--note", default="", help="a line of text for the summary written by --summarise")
    args = ap.parse_args()
    if args.summarise:
        if not args.config:
            raise SystemExit("--summarise needs --config")
        summarise_profile(args.summarise, args.config, args.note, args.summary_name)
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py measures one GPU: the block-sparse path has no cross-GPU step in this build "
                         "(it would shard on the batch dimension with no collective); run with --gpus 1")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU (the product has no CPU path)")
    global ROW_GENERATIONS
    ROW_GENERATIONS = args.row_generations
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    scratch = torch.empty(FLUSH_BYTES, dtype=torch.uint8, device=dev)
    headline = args.config or "c2"
    w, r = measure(headline, dev, args.steps, args.warmup, scratch)
    wall_ms = r["wall_ms"]
    tflops = w["flops"] / (wall_ms * 1e-3) / 1e12
    gbs = w["alg_bytes"] / (wall_ms * 1e-3) / 1e9
    line = {
        "metric": "effective TFLOP/s on nonzero blocks" if w["flops"] else "achieved GB/s on nonzero blocks",
        "value": round(tflops, 3) if w["flops"] else round(gbs, 1),
        "unit": "TFLOP/s" if w["flops"] else "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": w["dtype"], "data": "synthetic",
        "config": w["config"], "roofline": r["roofline"], "correct": r["correct"],
    }
    if w["flops"]:
        line["pct_of_mfma_peak"] = round(100.0 * tflops / PEAK_MFMA_TFLOPS[w["dtype"]], 2)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = w["cpu_baseline"]()
    del w
    if args.config is None:
        others = {}
        for name in COMPANIONS:
            torch.cuda.empty_cache()
            wo, ro = measure(name, dev, min(args.steps, 50), args.warmup, scratch)
            entry = {"workload": wo["config"]["workload"], "dtype": wo["dtype"], "ms_per_step": round(ro["wall_ms"], 4),
                     "roofline": ro["roofline"], "correct": ro["correct"]}
            if wo["flops"]:
                entry["tflops"] = round(wo["flops"] / (ro["wall_ms"] * 1e-3) / 1e12, 3)
            for key in ("lut_build_ms", "lut_build_host_syncs"):
                if key in wo["config"]:
                    entry[key] = wo["config"][key]
            others[name] = entry
            del wo
        line["other_configs"] = others
        del scratch
        torch.cuda.empty_cache()
        line["measured_ceilings"] = measured_ceilings(dev)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
