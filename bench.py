#!/usr/bin/env python3
"""Benchmark of the table-batched int4/int8/fp16 embedding forward on one MI355X.

    python bench.py [--steps K] [--warmup W] [--config 3|5|1|2|4] [--scale S]

A step is one forward over one batch of synthetic, seeded input already
resident in HBM (fbgemm_amd/bench_configs.py). The printed JSON line reports
useful row bytes per second (unpadded row data + scale/bias of every lookup
that reads a row; indices, offsets, weights, padding and output are not
credited), the same figure as a fraction of the 8 TB/s HBM peak, pooled rows
per second, and a CPU baseline timed on this machine's host cores.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--clock-warmup-s", type=float, default=0.3,
                    help="seconds of untimed forwards in front of the warm-up steps of every timed leg, to bring an idle "
                         "device's clocks up (0: none)")
    ap.add_argument("--config", type=int, default=3, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--scale", type=float, default=1.0, help="shrink rows and batch (1.0 = the real configuration)")
    ap.add_argument("--rows-scale", type=float, default=None,
                    help="config 3 only: shrink the tables but not the batch (cache-resident experiment)")
    ap.add_argument("--only-type", type=int, default=None,
                    help="config 3 only: give every table this row type (1 fp16, 2 int8, 3 int4); experiment")
    ap.add_argument("--per-table", action="store_true",
                    help="config 4 only: one row-wise-sparse kernel call per table (the reference's core-library "
                         "API) instead of one table-batched forward with the remap fused in")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="also run one plain copy of this many MiB (yardstick for hardware byte counters)")
    ap.add_argument("--graph", action="store_true",
                    help="capture one forward in a HIP graph after the warm-up and time replays of it "
                         "(what a serving loop would do; the default times eager launches)")
    ap.add_argument("--no-check", dest="check", action="store_false",
                    help="skip the parity gate (by default a sample of tables of the first forward is compared with "
                         "the oracle before anything is timed, and the line says \"checked\": true)")
    ap.add_argument("--accumulate", default="auto", choices=["auto", "exact", "fast"],
                    help="exact = the reference's sequence of fp32 roundings, bit-identical to the CPU path (the library's "
                         "default; the parity gate compares bit for bit); fast = the biases of a bag summed apart, the "
                         "mode a plan is switched to for throughput (tolerance grade: the gate holds fp16 / bf16 output to "
                         "one unit in the last place and fp32 output to 1e-5, the bound the path states); auto = exact, "
                         "except for config 5, where the arithmetic is not hidden behind the memory system and fast "
                         "is a sixth quicker. A table-batched run also times the other mode on the same inputs and "
                         "prints it under \"other_accumulate\" (--one-mode skips that)")
    ap.add_argument("--one-mode", "--no-exact", dest="other_mode", action="store_false",
                    help="do not also time the other accumulate mode")
    ap.add_argument("--wide4", choices=["auto", "on", "off"], default="auto",
                    help="large forwards whose lean tables all have 4-bit rows in bags of 8 lanes and more (config 5): the lean "
                         "kernel's four-waves-per-SIMD instance always / never, or (auto, the library's default) whichever of the "
                         "two kernels the first forwards measure as the faster one")
    ap.add_argument("--int8-output", action="store_true",
                    help="table-batched configurations: the operator's 8-bit pooled output ([B, total_D + 8 T]: every table's "
                         "pooled vector quantized row-wise in the lookup's output stage) instead of the configuration's float "
                         "output; needs --no-check --one-mode (the tests hold that output to the oracles, the gate here does not)")
    ap.add_argument("--no-rank-records", action="store_true",
                    help="config 4 only: read the int32 mapping arrays in the forward instead of the compact "
                         "bitmap-and-rank form of the (order-preserving) mappings")
    ap.add_argument("--no-kernel-events", dest="kernel_events", action="store_false",
                    help="skip the second timed region, the one with a pair of HIP events around the lookup kernels of "
                         "every forward (roofline.kernel_ms is then the forward time)")
    ap.add_argument("--no-also", dest="also", action="store_false",
                    help="default run only: do not append the driver-timed figures of config 5 under \"also\"")
    ap.add_argument("--ceiling-table-gib", default="1,4,32",
                    help="--op gather_ceiling: table sizes in GiB, comma separated (one size per run separates the counters of a profile)")
    ap.add_argument("--ceiling-index", default="both", choices=["uniform", "zipf", "both"],
                    help="--op gather_ceiling: row streams of the 128-byte-line cases")
    ap.add_argument("--ceiling-lines-only", action="store_true",
                    help="--op gather_ceiling: only the aligned 128-byte-line cases (no streaming read, no row shapes)")
    ap.add_argument("--op", default="lookup",
                    choices=["lookup", "quantize", "dequantize", "bounds_check", "pruned_array_lookup",
                             "pruned_hashmap_lookup", "float_to_hfp8", "hfp8_to_float", "rowwise_prune",
                             "compressed_indices_remap", "sequence", "no_bag", "inplace_update", "gather_ceiling", "ref_microbench"],
                    help="lookup = the table-batched forward (the metric); the others time one operator beside "
                         "the path at the shape config 4 / config 3 gives it and print the same kind of line")
    return ap.parse_args()


# the lookup kernels of a forward as the summaries name them (the last one is the general kernel)
LOOKUP_KERNELS = ("lookup_lean_kernel", "lookup_lean_wide4_kernel", "lookup_lean_wide4_redo_kernel", "lookup_kernel")


def traffic_from_profile(config_id):
    """HBM bytes the lookup kernels of one forward move (lookup_lean_kernel, and lookup_kernel for
    the tables the lean kernel does not take), from the committed hardware-counter
    summary of this configuration (profiles/lookup_kernel_config<N>.txt): FETCH_SIZE
    and WRITE_SIZE (KiB per dispatch), each scaled by what the same counter read
    for the plain copy of known size that ran in the same process. None when the
    summary is not there."""
    import re
    path = os.path.join(ROOT, "profiles", f"lookup_kernel_config{config_id}.txt")
    if not os.path.exists(path):
        return None
    text = open(path).read()
    m = re.search(r"--calibration-copy-mib (\d+)", text)
    vals = {}
    for kern, ctr, v in re.findall(r"pmc\s+(\w+)(?:<\w+>)?: (FETCH_SIZE|WRITE_SIZE) avg_per_dispatch=([0-9.e+]+)", text):
        vals[(kern, ctr)] = float(v)
    try:
        copy_bytes = int(m.group(1)) << 20
        total = 0.0
        for ctr in ("FETCH_SIZE", "WRITE_SIZE"):
            factor = copy_bytes / (vals[("calibration_copy_kernel", ctr)] * 1024.0)
            kib = [vals[(k, ctr)] for k in LOOKUP_KERNELS if (k, ctr) in vals]
            if not kib:
                return None
            total += sum(kib) * 1024.0 * factor
        return int(total)
    except (AttributeError, KeyError, ZeroDivisionError):
        return None


def profile_kernel_us(config_id):
    """Average duration (microseconds) of the lookup kernels of one forward in the committed kernel trace of
    this configuration (the `stats` lines of profiles/lookup_kernel_config<N>.txt), so that the line's own
    figure can be held against it. None when the summary is not there."""
    import re
    path = os.path.join(ROOT, "profiles", f"lookup_kernel_config{config_id}.txt")
    if not os.path.exists(path):
        return None
    rows = re.findall(r"stats\s+(\w+)(?:<\w+>)?: calls=(\d+) avg_ns=([0-9.e+]+)", open(path).read())
    calls = {k: int(c) for k, c, _ in rows}
    total = {k: int(c) * float(v) for k, c, v in rows}
    # every forward launches one of the two lean kernels (the trace holds both while the plan is still
    # choosing between them); the redo kernel goes with the four-wave instance
    forwards = calls.get("lookup_lean_kernel", 0) + calls.get("lookup_lean_wide4_kernel", 0)
    lean = sum(total.get(k, 0.0) for k in LOOKUP_KERNELS[:-1]) / forwards if forwards else 0.0
    general = total.get("lookup_kernel", 0.0) / calls["lookup_kernel"] if calls.get("lookup_kernel") else 0.0
    if not lean and not general:
        return None
    # with kernels of both kinds the general one runs beside the lean one (side stream): the longer of the two
    return round(max(lean, general) / 1e3, 2)


def tbe_runner(p, torch, accumulate="exact", rank_records=True, int8_output=False):
    """Returns (launch, out, status, plan) for a TbeProblem: launch() enqueues one forward."""
    from fbgemm_amd import _lib, ops

    lib = _lib.lib()
    dev = p.dev_weights.device
    plan = ops.TbePlan(torch.from_numpy(p.weights_offsets), torch.from_numpy(p.tys), torch.from_numpy(p.D_offsets),
                       torch.zeros(p.T, dtype=torch.int32), p.dev_weights.numel(), 0, p.row_alignment)
    _lib.check(lib.fbgemm_amd_tbe_plan_set_accumulate(plan.handle, 1 if accumulate == "fast" else 0))
    out_dt = {0: torch.float32, 1: torch.float16, 5: torch.bfloat16}[p.output_dtype]
    out = torch.empty((p.B, p.total_D), dtype=out_dt, device=dev)
    if int8_output:
        out = torch.empty((p.B, p.total_D + 8 * p.T), dtype=torch.uint8, device=dev)
    st = ops.Status(dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = (plan.handle, C.c_void_p(p.dev_weights.data_ptr()), None, C.c_void_p(p.indices.data_ptr()),
            C.c_void_p(p.offsets.data_ptr()), 64 if p.indices.dtype == torch.int64 else 32, p.indices.numel(),
            p.offsets.numel(), p.pooling_mode,
            None if p.indice_weights is None else C.c_void_p(p.indice_weights.data_ptr()),
            ops.INT8 if int8_output else p.output_dtype, C.c_void_p(out.data_ptr()),
            C.c_void_p(p.extra["remap"].data_ptr()) if "remap" in p.extra else None, 32,
            C.c_void_p(p.extra["remap_offsets"].data_ptr()) if "remap" in p.extra else None,
            p.extra["remap_offsets"].numel() if "remap" in p.extra else 0,
            C.c_void_p(st.buf.data_ptr()), stream)
    if "remap" in p.extra and rank_records:
        plan.set_index_remappings(p.extra["remap"], p.extra["remap_offsets"])

    def launch():
        # the stream of the moment: under graph capture it is the capturing stream
        rc = lib.fbgemm_amd_tbe_forward_pruned(*args[:-1], C.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc:
            raise RuntimeError(lib.fbgemm_amd_last_error().decode())

    return launch, out, st, plan


def spmdm_runner(probs, torch):
    """Single-table configurations: one launch per table."""
    from fbgemm_amd import _lib, ops
    from fbgemm_amd._lib import SpmdmConfig

    lib = _lib.lib()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    st = ops.Status(probs[0].table.device)
    calls, outs = [], []
    for p in probs:
        out_dt = {0: torch.float32, 1: torch.float16, 5: torch.bfloat16}[p.out_ty]
        out = torch.empty(p.num_bags * p.D, dtype=out_dt, device=p.table.device)
        cfg = SpmdmConfig(weight_ty=p.ty, output_ty=p.out_ty, index_bits=64, offset_bits=32, block_size=p.D,
                          output_stride=-1, input_stride=-1, normalize_by_lengths=int(p.normalize),
                          is_weight_positional=0, use_offsets=1, scale_bias_last=1)
        calls.append((cfg, (p.num_bags, p.lookups, p.data_size, C.c_void_p(p.table.data_ptr()),
                            C.c_void_p(p.indices.data_ptr()), C.c_void_p(p.offsets.data_ptr()), None,
                            C.c_void_p(out.data_ptr()),
                            None if p.remap is None else C.c_void_p(p.remap.data_ptr()),
                            C.c_void_p(st.buf.data_ptr()), stream)))
        outs.append(out)

    def launch():
        now = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        for cfg, a in calls:
            rc = lib.fbgemm_amd_spmdm_launch(C.byref(cfg), *a[:-1], now)
            if rc:
                raise RuntimeError(lib.fbgemm_amd_last_error().decode())

    return launch, outs, st


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_counts():
    """What the host has: logical CPUs, physical cores (distinct (package, core) pairs of
    /proc/cpuinfo), and the CPUs this process may run on."""
    cores, phys, core = set(), None, None
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("physical id"):
                phys = line.split(":", 1)[1].strip()
            elif line.startswith("core id"):
                core = line.split(":", 1)[1].strip()
            elif not line.strip():
                if core is not None:
                    cores.add((phys, core))
                phys = core = None
        if core is not None:
            cores.add((phys, core))
    except OSError:
        pass
    try:
        allowed = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        allowed = os.cpu_count() or 1
    return {"os_cpu_count": os.cpu_count(), "physical_cores": len(cores) or None, "cpus_allowed": allowed}


def cpu_baseline_tbe(p, seconds, torch):
    """Time the CPU path on this machine's host cores, on the same workload: as
    many of the problem's tables, from the first on, as fit half of the free
    host memory (all of them for config 3's 33 GB on the benchmark box), all
    their bags. Protocol after the reference's own microbenchmark
    (bench/EmbeddingSpMDMNBitBenchmark.cc:210-266): cache-warm repeats AND
    passes with the last-level cache flushed before each (a 1 GiB buffer
    rewritten, untimed; bench/BenchUtils.cc:64-69), one core and all cores.
    Preferred engine: the reference's AVX2/AVX-512 kernels through
    libtorch_cpu.so, run the way the CPU operator runs them (one table after
    the other; all cores = OpenMP over tables). Fallbacks: the reference's
    scalar code built from its sources, then the C oracle."""
    import numpy as np
    import oracle
    from fbgemm_amd.bench_configs import unpadded_row_bytes

    try:
        import psutil
        budget = int(psutil.virtual_memory().available * 0.5)
    except Exception:
        budget = 6 << 30
    budget = max(budget, 1 << 30)
    nt = 0
    while nt < p.T and int(p.weights_offsets[nt] + p.rows[nt] * p.row_bytes[nt]) <= budget:
        nt += 1
    nt = max(nt, 1)
    end = int(p.weights_offsets[nt - 1] + p.rows[nt - 1] * p.row_bytes[nt - 1])
    host_w = np.empty(end, np.uint8)
    step = 1 << 30
    for s0 in range(0, end, step):  # in pieces: no second 33 GB staging copy
        host_w[s0:min(end, s0 + step)] = p.dev_weights[s0:min(end, s0 + step)].cpu().numpy()
    idx = np.ascontiguousarray(p.physical_indices, dtype=np.int64)  # after the remap, where there is one
    off = np.ascontiguousarray(p.host_offsets, dtype=np.int64)
    kept = p.kept_per_table()[:nt]
    sample_bytes = int(sum(int(k) * unpadded_row_bytes(int(D), int(ty)) for k, D, ty in zip(kept, p.Ds[:nt], p.tys[:nt])))
    sample_rows = int(off[nt * p.B] - off[0])
    out = np.zeros((p.B, p.total_D), dtype=np.float32 if p.output_dtype == 0 else np.uint16)

    jit = None
    try:
        from oracle import jit_baseline as jit
        jit.lib()
    except Exception:
        jit = None

    def one_pass(threads):
        if jit is not None:
            rc = jit.tbe_tables(0, nt, host_w, p.weights_offsets, p.tys, p.D_offsets, p.row_bytes, p.rows,
                                p.total_D, idx, off, p.B, p.pooling_mode, p.host_weights, p.output_dtype, out, threads)
            assert rc == 0
        else:
            for t in range(nt):
                s, e = int(off[t * p.B]), int(off[(t + 1) * p.B])
                ty, rb = int(p.tys[t]), int(p.row_bytes[t])
                elem = 4 if ty == 0 else 2 if ty == 1 else 1
                w0 = int(p.weights_offsets[t])
                ok, _ = oracle.spmdm(ty, int(p.Ds[t]), host_w[w0:w0 + int(p.rows[t]) * rb], idx[s:e],
                                     off[t * p.B:(t + 1) * p.B + 1] - off[t * p.B],
                                     weights=None if p.host_weights is None else p.host_weights[s:e],
                                     normalize=p.pooling_mode == 1, out_ty=p.output_dtype, input_stride=rb // elem,
                                     scale_bias_last=False, data_size=int(p.rows[t]), output_size=p.B,
                                     impl="ref" if oracle.have_ref() else "oracle")
                assert ok

    flush_buf = np.zeros(1 << 30, np.uint8)

    def timed(threads, secs, flush):
        one_pass(threads)  # warm-up: code generation, page faults
        n, spent, t_start = 0, 0.0, time.perf_counter()
        while True:
            if flush:
                np.add(flush_buf, 1, out=flush_buf)  # untimed: pushes tables, indices and output out of the LLC
            t0 = time.perf_counter()
            one_pass(threads)
            spent += time.perf_counter() - t0
            n += 1
            if time.perf_counter() - t_start >= secs or n >= 1000:
                return spent / n

    # threads of the all-core leg: what OMP_NUM_THREADS grants (the benchmark boxes set it to their
    # share of the host), else every physical core this process may run on
    counts = cpu_counts()
    omp = os.environ.get("OMP_NUM_THREADS")
    cores = int(omp) if omp and omp.isdigit() and int(omp) > 0 else min(counts["physical_cores"] or counts["cpus_allowed"], counts["cpus_allowed"])
    cores = max(1, min(cores, counts["cpus_allowed"]))
    if jit is not None:
        cores = min(cores, jit.max_threads())
        kind = "reference"
        impl = ("fbgemm AVX2/AVX-512 run-time generated kernels as shipped in libtorch_cpu.so "
                "(GenerateEmbeddingSpMDM[NBit]WithStrides, THREAD_LOCAL, prefetch 16), table after table "
                "as the CPU operator runs them; all-core figure = OpenMP over tables")
    else:
        cores = 1
        kind = "reference" if oracle.have_ref() else "port"
        impl = ("reference scalar EmbeddingSpMDM*_ref built from its sources (oracle/_ref)" if kind == "reference"
                else "C restatement of the reference's scalar loop (oracle/)")
    t1_warm = timed(1, seconds / 4, False)
    tn_warm = timed(cores, seconds / 4, False) if cores > 1 else t1_warm
    t1_cold = timed(1, seconds / 4, True)
    tn_cold = timed(cores, seconds / 4, True) if cores > 1 else t1_cold
    fig = lambda t: {"value": round(sample_bytes / t / 1e9, 3), "unit": "GB/s", "pooled_rows_per_s": round(sample_rows / t, 1)}
    return {
        **fig(tn_warm), "cores": cores, "kind": kind, "cpu_model": cpu_model(), **counts,
        "omp_num_threads": os.environ.get("OMP_NUM_THREADS"),
        "llc_flushed": fig(tn_cold),
        "single_core": {**fig(t1_warm), "llc_flushed": fig(t1_cold)},
        "sample": f"first {nt} of {p.T} tables of the same problem, all {p.B} bags each "
                  f"({sample_rows} lookups, {sample_bytes} useful row bytes per pass); `value` = cache-warm repeats, "
                  f"`llc_flushed` = a 1 GiB buffer rewritten before every pass (untimed); {impl}",
    }


def calibration_copy(a, torch):
    """One plain copy of a known size: the yardstick the hardware byte counters are scaled against."""
    if not a.calibration_copy_mib:
        return
    from fbgemm_amd import _lib
    n = a.calibration_copy_mib << 20
    src = torch.zeros(n, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    _lib.bench_check(_lib.bench_lib().fbgemm_amd_bench_calibration_copy(
        C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), n,
        C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()


def gather_ceiling(a):
    """What this GPU sustains for the access patterns of a pooled lookup, measured with the
    yardstick kernels of the benchmark-only library (bench_kernels.hip): a streaming read, and
    gathers of random rows with 16-byte lanes, from tables of --ceiling-table-gib GiB (1, 4 and 32
    by default: a table the address translation covers easily, and tables far beyond it), with
    uniform and with Zipf(1.1)-skewed row streams, 8 or 16 rows per lane group in flight, into
    registers or straight into LDS. One JSON line: `value` is the rate of uniform random aligned
    128-byte lines from the largest table, every case is under "cases"."""
    import numpy as np
    import torch

    from fbgemm_amd import _lib
    lib = _lib.bench_lib()
    torch.cuda.set_device(0)
    stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)
    sizes = [int(g) for g in a.ceiling_table_gib.split(",")]
    biggest = int((max(sizes) << 30) * a.scale)
    table = torch.empty(biggest, dtype=torch.uint8, device="cuda")
    table.view(torch.int32).random_(0, 1 << 30)
    sink = torch.zeros(1 << 20, dtype=torch.int32, device="cuda")
    gen = torch.Generator(device="cuda")
    gen.manual_seed(99)
    n = int((1 << 25) * a.scale)
    ptr = lambda t: C.c_void_p(t.data_ptr())
    steps, warm = max(3, a.steps // 10), max(1, a.warmup // 4)

    def timed(fn):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(steps):
            fn()
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) / steps

    def zipf_rows(rows):
        """Row ids the way the benchmark configurations draw them: Zipf(1.1) ranks, folded into the
        table, sent through a seeded permutation (an affine map with an odd multiplier modulo a power
        of two, folded again: hot rows land all over the table)."""
        rng = np.random.Generator(np.random.PCG64(4242))
        z = (rng.zipf(1.1, size=n) - 1) % rows
        z = (z * 2654435761 + 12345) % rows
        return torch.from_numpy(z.astype(np.int32)).cuda()

    modes = [(0, "registers, 8 rows in flight", "gather_lines_kernel<8>"), (1, "registers, 16 rows in flight", "gather_lines_kernel<16>"),
             (2, "LDS-direct 16-byte loads, 8 rows in flight", "gather_lines_lds_kernel")]
    cases = []
    if not a.ceiling_lines_only:
        ms = timed(lambda: _lib.bench_check(lib.fbgemm_amd_bench_stream_read(ptr(table), biggest, ptr(sink), sink.numel(), stream())))
        cases.append({"case": f"streaming read of {biggest >> 30} GiB, 16 bytes per lane, 8 loads in flight",
                      "kernel": "stream_read_kernel", "ms": round(ms, 4), "GB/s": round(biggest / ms / 1e6, 1)})

    def gather_case(what, table_bytes, stride, lanes, off, idx, mode):
        rows = table_bytes // stride
        waves = 256 * 64
        ms = timed(lambda: _lib.bench_check(lib.fbgemm_amd_bench_gather(ptr(table), rows, stride, lanes, off, ptr(idx), n,
                                                                         ptr(sink), sink.numel(), waves, mode[0], stream())))
        useful = n * lanes * 16
        first, last = off, off + lanes * 16 - 1
        g = np.gcd(stride, 128)
        starts = (np.arange(128 // g) * g) % 128
        lines = float(np.mean((starts + last) // 128 - (starts + first) // 128 + 1))
        rec = {"case": what, "table_GiB": round(table_bytes / 2**30, 2), "fetch": mode[1], "kernel": mode[2], "rows": n,
               "ms": round(ms, 4), "useful_GB/s": round(useful / ms / 1e6, 1), "lines_per_row": round(lines, 3),
               "G_lines/s": round(n * lines / ms / 1e6, 2), "G_rows/s": round(n / ms / 1e6, 2)}
        cases.append(rec)
        return rec

    headline = None
    for gib in sorted(sizes):
        tb = int((gib << 30) * a.scale)
        rows = tb // 128
        uni = torch.randint(0, rows, (n,), dtype=torch.int32, device="cuda", generator=gen)
        if a.ceiling_index in ("uniform", "both"):
            rec = gather_case("uniform random 128-byte lines (aligned)", tb, 128, 8, 0, uni, modes[0])
            if gib == max(sizes):
                headline = rec
        if a.ceiling_index in ("zipf", "both"):
            rec = gather_case("Zipf(1.1) 128-byte lines (aligned)", tb, 128, 8, 0, zipf_rows(rows), modes[0])
            if gib == max(sizes) and headline is None:
                headline = rec
        if gib == max(sizes) and a.ceiling_index != "zipf":
            gather_case("uniform random 128-byte lines (aligned)", tb, 128, 8, 0, uni, modes[1])
            gather_case("uniform random 128-byte lines (aligned)", tb, 128, 8, 0, uni, modes[2])
        del uni
    if not a.ceiling_lines_only:
        # (what, row stride, lanes per row, byte offset of the first lane's load), largest table
        shapes = [("128 bytes at byte 4 of rows 144 bytes apart (4-bit rows of 256 columns, data after the header)", 144, 8, 4),
                  ("144-byte rows whole, as 8 aligned lanes of the first 128 bytes", 144, 8, 0),
                  ("random 64-byte half lines (aligned)", 64, 4, 0),
                  ("random 512-byte rows (fp16 rows of 256 columns)", 512, 32, 0),
                  ("32 bytes at byte 4 of rows 48 bytes apart (4-bit rows of 64 columns)", 48, 2, 4)]
        for what, stride, lanes, off in shapes:
            idx = torch.randint(0, biggest // stride, (n,), dtype=torch.int32, device="cuda", generator=gen)
            gather_case(what, biggest, stride, lanes, off, idx, modes[0])
    res = {"metric": "random 128-byte line gathers, G lines/s on 1 MI355X", "value": headline["G_lines/s"], "unit": "G lines/s",
           "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": headline["ms"],
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
           "config": {"workload": f"yardstick kernels over tables of {sorted(sizes)} GiB, {n} rows per launch"},
           "roofline": {"bound": "hbm", "achieved": headline["useful_GB/s"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                        "frac": round(headline["useful_GB/s"] / HBM_PEAK_GBPS, 4), "traffic": None,
                        "kernel": "gather_lines_kernel<8>", "kernel_ms": headline["ms"],
                        "algorithmic_bytes_per_launch": n * 128},
           "cases": cases, "cpu_baseline": None}
    print(json.dumps(res))


def ref_microbench(a):
    """The shapes of the reference's own microbenchmark (bench/EmbeddingSpMDMNBitBenchmark.cc:47-63):
    10 bags, lengths U{1..201}, indices unique inside a bag, a 4-bit table of 4,000,000 rows (fp16
    scale/bias last) x D in {32, 64, 128, 256}, unweighted sum, fp32 output. Few, long bags: per call
    the GPU is bound by launches and dependent memory round trips, not by bandwidth. Timed per D:
    the default (exact) mode, the tolerance-grade mode (bags cut into segments), and the reference's
    AVX kernel on one host core the way its benchmark runs it (cache-warm and LLC-flushed)."""
    import numpy as np
    import torch

    from fbgemm_amd import ops
    torch.cuda.set_device(0)
    rng = np.random.default_rng(123)
    rows, nb = int(4_000_000 * a.scale), 10
    jit = None
    if not a.no_cpu:
        try:
            from oracle import jit_baseline as jit
            jit.lib()
        except Exception:
            jit = None
    cases = []
    flush = np.zeros(1 << 28, np.uint8)
    for D in (32, 64, 128, 256):
        lens = rng.integers(1, 202, size=nb)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        idx = np.concatenate([rng.permutation(rows)[:l] for l in lens]).astype(np.int64)
        stride = D // 2 + 4
        table = torch.randint(0, 256, (rows, stride), dtype=torch.uint8, device="cuda")
        table[:, D // 2:] = torch.tensor([2.0, 1.0], dtype=torch.float16).view(torch.uint8).cuda()
        d_idx, d_off = torch.from_numpy(idx).cuda(), torch.from_numpy(off).cuda()
        out = torch.empty(nb * D, dtype=torch.float32, device="cuda")
        kern = ops.generate_embedding_spmdm_nbit(4, D, False, False)
        st = ops.Status()
        rec = {"D": D, "lookups": int(off[-1]), "useful_row_bytes": int(off[-1]) * stride}
        ref_out = None
        for mode, acc in (("exact", ops.ACC_EXACT), ("fast", ops.ACC_FAST)):
            call = lambda: kern(nb, len(idx), rows, table.view(-1), d_idx, d_off, None, out, status=st, accumulate=acc)
            for _ in range(a.warmup):
                call()
            torch.cuda.synchronize()
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ev0.record()
            for _ in range(a.steps):
                call()
            ev1.record()
            torch.cuda.synchronize()
            rec[f"gpu_{mode}_us"] = round(ev0.elapsed_time(ev1) / a.steps * 1e3, 2)
            if mode == "exact":
                ref_out = out.clone()
            else:
                rel = ((out - ref_out).abs() / ref_out.abs().clamp_min(1e-30)).max().item()
                rec["fast_vs_exact_max_rel"] = float(f"{rel:.3g}")
        assert st.read()[0] == 0
        if jit is not None:
            host = table.cpu().numpy().reshape(-1)
            idx64, off64 = idx, off.astype(np.int64)
            for name, fl in (("cpu_warm_us", False), ("cpu_flushed_us", True)):
                jit.spmdm(3, D, host, idx64, off64, out_ty=0, data_size=rows)
                n, spent = 0, 0.0
                while spent < 0.5 and n < 2000:
                    if fl:
                        np.add(flush, 1, out=flush)
                    t0 = time.perf_counter()
                    jit.spmdm(3, D, host, idx64, off64, out_ty=0, data_size=rows)
                    spent += time.perf_counter() - t0
                    n += 1
                rec[name] = round(spent / n * 1e6, 2)
            del host
        cases.append(rec)
        del table
    head = cases[2]
    res = {"metric": "time per call, reference microbenchmark shapes (10 bags x ~100 rows, 4M-row 4-bit table) on 1 MI355X",
           "value": head["gpu_fast_us"], "unit": "us", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
           "ms_per_step": head["gpu_fast_us"] / 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
           "dtype": "f32", "data": "synthetic",
           "config": {"workload": "bench/EmbeddingSpMDMNBitBenchmark.cc shapes; value = D 128, tolerance-grade mode", "rows": rows},
           "roofline": {"bound": "hbm", "achieved": round(head["useful_row_bytes"] / head["gpu_fast_us"] / 1e3, 3), "peak": HBM_PEAK_GBPS,
                        "unit": "GB/s", "frac": round(head["useful_row_bytes"] / head["gpu_fast_us"] / 1e3 / HBM_PEAK_GBPS, 6),
                        "traffic": None, "kernel": "split_offsets + lookup + combine_segments", "kernel_ms": head["gpu_fast_us"] / 1e3,
                        "algorithmic_bytes_per_launch": head["useful_row_bytes"]},
           "cases": cases,
           "cpu_baseline": None if jit is None else {
               "value": head["cpu_warm_us"], "unit": "us", "cores": 1, "kind": "reference", "cpu_model": cpu_model(),
               "sample": "the whole call (D 128), fbgemm's AVX2/AVX-512 generated kernel from libtorch_cpu.so, cache-warm; "
                         "cpu_flushed_us in cases = a 256 MiB buffer rewritten before every call"}}
    print(json.dumps(res))


def side_op(a):
    """One operator beside the lookup, timed with events on the launch stream.

    Shapes: the index operators see config 4's batch (32 tables x 4096 bags,
    3.6 M int64 indices, 2 M-row mappings); the quantizers see 1 M rows x 128
    columns (a table of config 2's shape), 4-bit rows in the table-batched layout;
    so do the hfp8 converters and the single-table no_bag kernel (8-bit rows);
    rowwise_prune sees 2 M x 64 fp32 with half of the rows kept; sequence
    (PoolingMode.NONE) sees 32 int4 tables x 1 M rows x 128 with config 4's bags;
    inplace_update overwrites 1 M random rows of those tables."""
    import numpy as np
    import torch

    from fbgemm_amd import ops

    torch.cuda.set_device(0)
    rng = np.random.default_rng(4242)
    cu = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()
    cpu = None
    if a.op in ("quantize", "dequantize"):
        rows, cols = int((1 << 20) * a.scale), 128
        x = torch.randn(rows, cols, device="cuda", dtype=torch.float32)
        stride = ops.padded_row_size_in_bytes(cols, ops.INT4, 16)
        q = torch.zeros(rows, stride, dtype=torch.uint8, device="cuda")
        ops.quantize_rowwise(x, 4, False, ops.QLAYOUT_TBE, out=q)
        row_bytes = cols * 4 + cols // 2 + 4
        if a.op == "quantize":
            launch = lambda: ops.quantize_rowwise(x, 4, False, ops.QLAYOUT_TBE, out=q)
            kernel, workload = "quantize_rowwise_kernel", f"fp32 [{rows}, {cols}] -> 4-bit rows, fp16 scale/bias first"
        else:
            launch = lambda: ops.dequantize_rowwise(q, cols, 4, False, ops.QLAYOUT_TBE, torch.float32)
            kernel, workload = "dequantize_rowwise_kernel", f"4-bit rows, fp16 scale/bias first [{rows}, {cols}] -> fp32"
        alg_bytes, units = rows * row_bytes, rows

        def cpu():  # the oracle's scalar restatement on a sample, one core
            import oracle
            n = min(rows, 200_000)
            xs = x[:n].cpu().numpy()
            qs = q[:n].cpu().numpy()
            t0 = time.perf_counter()
            if a.op == "quantize":
                oracle.quantize_rowwise(xs, 4, False, oracle.LAYOUT_TBE, out_stride=stride)
            else:
                oracle.dequantize_rowwise(qs, cols, 4, False, oracle.LAYOUT_TBE)
            dt = time.perf_counter() - t0
            return {"value": round(n * row_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                    "sample": f"first {n} rows, one pass"}
    elif a.op in ("float_to_hfp8", "hfp8_to_float"):
        rows, cols = int((1 << 20) * a.scale), 128
        x = torch.randn(rows, cols, device="cuda", dtype=torch.float32)
        codes = ops.float_to_hfp8_quantized(x, 4, 7, 240.0)
        if a.op == "float_to_hfp8":
            launch = lambda: ops.float_to_hfp8_quantized(x, 4, 7, 240.0)
            kernel, workload = "float_to_hfp8_kernel", f"fp32 [{rows}, {cols}] -> hfp8 (4 exponent bits, bias 7)"
        else:
            launch = lambda: ops.hfp8_quantized_to_float(codes, 4, 7)
            kernel, workload = "hfp8_to_float_kernel", f"hfp8 (4 exponent bits, bias 7) [{rows}, {cols}] -> fp32"
        alg_bytes, units = rows * cols * 5, rows
    elif a.op == "rowwise_prune":
        rows, cols = int(2_000_000 * a.scale), 64
        w = torch.randn(rows, cols, device="cuda", dtype=torch.float32)
        ind = torch.rand(rows, device="cuda", dtype=torch.float32)
        kept = int((ind > 0.5).sum())
        launch = lambda: ops.embedding_bag_rowwise_prune(w, ind, 0.5, torch.int32, True, 0, None)
        # indicator in, remap out, the kept rows in and out
        alg_bytes, units = 4 * rows + 4 * rows + 2 * kept * cols * 4, rows
        kernel, workload = "prune_gather_kernel", f"fp32 [{rows}, {cols}], {kept} rows kept, int32 remap (map + gather, output allocated per call)"
    elif a.op == "no_bag":
        rows, cols = int((1 << 20) * a.scale), 128
        table = torch.randint(0, 256, (rows, cols + 8), dtype=torch.uint8, device="cuda")
        table[:, cols:] = torch.tensor([0.01, -0.5], dtype=torch.float32).view(torch.uint8).cuda()
        n = rows
        idx = torch.randint(0, rows, (n,), dtype=torch.int64, device="cuda")
        out = torch.empty(n, cols, dtype=torch.float32, device="cuda")
        kern = ops.generate_embedding_spmdm_with_strides(ops.INT8, cols, False, False, no_bag=True)
        st = ops.Status()
        launch = lambda: kern(n, n, rows, table, idx, None, None, out, status=st)
        alg_bytes, units = n * (cols + 8 + cols * 4 + 8), n
        kernel, workload = "row_lookup_kernel", f"8-bit rows [{rows}, {cols}] (fp32 scale/bias last), {n} int64 indices -> fp32 rows"
    elif a.op == "inplace_update":
        T, D = 32, 128
        E = max(1000, int(1_000_000 * a.scale))
        n = max(1, int(1_000_000 * a.scale))
        rb = ops.padded_row_size_in_bytes(D, ops.INT4, 16)
        weights = torch.randint(0, 256, (T * E * rb,), dtype=torch.uint8, device="cuda")
        tables = rng.integers(0, T, size=n).astype(np.int32)
        # distinct rows per table: two updates of one row in a call race
        rows = (rng.permutation(T * E)[:n] // T).astype(np.int64)
        upd = torch.randint(0, 256, (n * rb,), dtype=torch.uint8, device="cuda")
        args = (weights, torch.zeros(0, dtype=torch.uint8, device="cuda"), torch.zeros(T, dtype=torch.int32, device="cuda"),
                (torch.arange(T, dtype=torch.int64) * (E * rb)).cuda(), torch.full((T,), ops.INT4, dtype=torch.uint8, device="cuda"),
                torch.arange(T + 1, dtype=torch.int32, device="cuda") * D, upd, cu(tables), cu(rows),
                cu(np.arange(n + 1, dtype=np.int64) * rb), 16)
        st = ops.Status()
        launch = lambda: ops.emb_inplace_update(*args, status=st)
        alg_bytes, units = n * (2 * rb + 4 + 8 + 8), n
        kernel, workload = "inplace_update_kernel", f"{n} rows of {rb} bytes into {T} int4 tables x {E} rows x {D} (random rows)"
    elif a.op == "sequence":
        T, B, D = 32, max(1, int(4096 * a.scale)), 128
        E = max(1000, int(1_000_000 * a.scale))
        rb = ops.padded_row_size_in_bytes(D, ops.INT4, 16)
        lens = rng.integers(5, 51, size=T * B)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        n = int(off[-1])
        idx = rng.integers(0, E, size=n).astype(np.int64)
        weights = torch.randint(0, 256, (T * E * rb,), dtype=torch.uint8, device="cuda")
        weights.view(T * E, rb)[:, :4] = torch.tensor([0.01, -0.5], dtype=torch.float16).view(torch.uint8).cuda()
        wo = torch.arange(T, dtype=torch.int64) * (E * rb)
        args = (weights, torch.zeros(0, dtype=torch.uint8, device="cuda"), torch.zeros(T, dtype=torch.int32, device="cuda"),
                wo.cuda(), torch.full((T,), ops.INT4, dtype=torch.uint8, device="cuda"),
                torch.arange(T + 1, dtype=torch.int32, device="cuda") * D, T * D, 0, D, 0, 0, 0, cu(idx), cu(off), ops.POOL_NONE,
                None, ops.FP16)
        st = ops.Status()
        launch = lambda: ops.int_nbit_split_embedding_codegen_lookup_function(*args, row_alignment=16, status=st)
        alg_bytes, units = n * (D // 2 + 4 + D * 2 + 8), n
        kernel, workload = "sequence_lookup_kernel", f"PoolingMode.NONE, {T} int4 tables x {E} rows x {D}, {n} int64 indices -> fp16 rows (output allocated per call)"
    else:
        T, B = 32, max(1, int(4096 * a.scale))
        E = max(1000, int(2_000_000 * a.scale))
        lens = rng.integers(5, 51, size=T * B)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
        n = int(off[-1])
        idx = rng.integers(0, E, size=n).astype(np.int64)
        d_idx, d_off = cu(idx), cu(off)
        units = n
        if a.op == "bounds_check":
            rows_per_table = cu(np.full(T, E, np.int64))
            warning = torch.zeros(1, dtype=torch.int64, device="cuda")
            launch = lambda: ops.bounds_check_indices(rows_per_table, d_idx, d_off, ops.BOUNDS_WARNING, warning)
            alg_bytes = 8 * n + 8 * (T * B + 1)
            kernel, workload = "bounds_check_bags_kernel", f"WARNING mode, {T} tables x {B} bags, {n} int64 indices in range"
        elif a.op == "compressed_indices_remap":
            # one table's mapping, all bags: the core library's remap takes one table at a time
            mapping = np.where(rng.random(E) < 0.5, -1, 1).astype(np.int32)
            mapping[mapping > 0] = np.arange(int((mapping > 0).sum()), dtype=np.int32)
            d_map = cu(mapping)
            w = torch.rand(n, device="cuda", dtype=torch.float32)
            launch = lambda: ops.compressed_indices_remap(d_idx, d_map, d_off, w)
            kept = int((mapping[idx] != -1).sum())
            alg_bytes = 8 * n + 4 * n + 4 * n + 12 * kept + 16 * (T * B + 1)
            kernel, workload = "remap_move_kernel", f"one mapping of {E} int32 entries (half pruned), {T * B} bags, {n} int64 indices + weights (outputs allocated per call)"
        elif a.op == "pruned_array_lookup":
            remap = cu(np.where(rng.random(T * E) < 0.5, -1, 1).astype(np.int32))
            ro = cu(np.arange(T + 1, dtype=np.int64) * E)
            launch = lambda: ops.pruned_array_lookup(d_idx, d_off, remap, ro)
            alg_bytes = 8 * n + 4 * n + 8 * n
            kernel, workload = "pruned_array_lookup_kernel", f"{T} mappings x {E} int32 entries, {n} int64 indices"
        else:
            cap = int(E * 0.5 / 0.6) + 1  # the map is built on the host, as the reference's module does
            hto = np.arange(T + 1, dtype=np.int64) * cap
            table = np.full((T * cap, 2), -1, np.int64)
            keys = np.concatenate([rng.choice(E, size=E // 2, replace=False) for _ in range(T)]).astype(np.int64)
            dense = np.concatenate([np.arange(E // 2) for _ in range(T)]).astype(np.int64)
            h_table = torch.from_numpy(table)
            ops.pruned_hashmap_insert(torch.from_numpy(keys), torch.from_numpy(dense),
                                      torch.from_numpy((np.arange(T + 1) * (E // 2)).astype(np.int64)), h_table, torch.from_numpy(hto))
            d_table, d_hto = h_table.cuda(), cu(hto)
            launch = lambda: ops.pruned_hashmap_lookup(d_idx, d_off, d_table, d_hto)
            alg_bytes = 8 * n + 16 * n + 8 * n
            kernel, workload = "pruned_hashmap_lookup_kernel", f"{T} maps x {cap} slots (load 0.6), {n} int64 indices"
    for _ in range(a.warmup):
        launch()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(a.steps):
        launch()
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / a.steps
    calibration_copy(a, torch)
    ms = ev0.elapsed_time(ev1) / a.steps
    gbps = alg_bytes / (ms * 1e-3) / 1e9
    res = {"metric": f"achieved HBM GB/s, {a.op} on 1 MI355X", "value": round(gbps, 2), "unit": "GB/s", "n_gpus": 1,
           "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(wall_ms, 5), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "f32" if a.op in ("quantize", "dequantize", "float_to_hfp8", "hfp8_to_float", "sequence", "no_bag") else "int64", "data": "synthetic",
           "config": {"workload": workload, "units_per_step": units},
           "roofline": {"bound": "hbm", "achieved": round(gbps, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                        "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None, "kernel": kernel,
                        "kernel_ms": round(ms, 5), "algorithmic_bytes_per_launch": alg_bytes},
           "cpu_baseline": cpu() if (cpu is not None and not a.no_cpu) else None}
    print(json.dumps(res))


def sample_tables(p):
    """Tables the parity gate compares: first, last, the middle, and the first of every (type, D) pair."""
    seen = {}
    for t in range(p.T):
        seen.setdefault((int(p.tys[t]), int(p.Ds[t])), t)
    return sorted(set(seen.values()) | {0, p.T // 2, p.T - 1})


def parity_gate(p, out, launch, torch, np, accumulate="exact"):
    """One forward, then the sampled tables' blocks of its output against the
    oracle on the same inputs: bit for bit (exact), or to the stated tolerance
    (fast). Raises before anything is timed."""
    import oracle
    launch()
    torch.cuda.synchronize()
    from fbgemm_amd import tolerance
    tables = sample_tables(p)
    worst, worst_block, needed, cancels = 0, 0.0, 0, 0
    for t in tables:
        s, e = int(p.host_offsets[t * p.B]), int(p.host_offsets[(t + 1) * p.B])
        elem = 4 if int(p.tys[t]) == 0 else 2 if int(p.tys[t]) == 1 else 1
        ok, want = oracle.spmdm(int(p.tys[t]), int(p.Ds[t]), p.table_host_bytes(t), p.physical_indices[s:e],
                                p.host_offsets[t * p.B:(t + 1) * p.B + 1] - p.host_offsets[t * p.B],
                                weights=None if p.host_weights is None else p.host_weights[s:e],
                                normalize=p.pooling_mode == 1, out_ty=p.output_dtype,
                                input_stride=int(p.row_bytes[t]) // elem, scale_bias_last=False,
                                data_size=int(p.rows[t]), output_size=p.B)
        got = out[:, int(p.D_offsets[t]):int(p.D_offsets[t + 1])].contiguous().cpu()
        got = got.numpy() if p.output_dtype == 0 else got.view(torch.int16).numpy().view(np.uint16)
        if accumulate == "exact":
            same = ok and (got.reshape(-1).view(want.dtype) == want).all()
        else:
            r = tolerance.grade(got.reshape(p.B, -1), want.reshape(p.B, -1), p.output_dtype, np)
            worst, worst_block = max(worst, r["worst"]), max(worst_block, r["worst_block"])
            needed, cancels = needed + r["needed_block_clause"], cancels + r["cancellations"]
            same = ok and r["ok"]
        if not same:
            raise AssertionError(f"parity gate: table {t} of {p.name} differs from the oracle; nothing was timed")
    how = "bit for bit" if accumulate == "exact" else (
        f"to tolerance (worst element-wise: {worst} {'units in the last place' if p.output_dtype else 'relative'}; "
        f"{needed} of {cancels} cancellations needed the block-relative clause, worst {worst_block:.3g} of the block)")
    print(f"parity gate: tables {tables} of {p.name} match the oracle {how}", file=sys.stderr)
    return tables


def time_tbe(p, a, torch, np, steps, warmup, graph, accumulate):
    """Parity gate, warm-up, `steps` timed forwards of one table-batched problem.
    Returns the figures of the JSON line that depend on the measurement."""
    from fbgemm_amd import _lib
    if a.int8_output:
        assert not a.check and not a.other_mode, "--int8-output needs --no-check --one-mode"
    _lib.check(_lib.lib().fbgemm_amd_set_wide4({"auto": -1, "on": 2, "off": 0}[getattr(a, "wide4", "auto")]))
    launch, out, st, plan = tbe_runner(p, torch, accumulate, not a.no_rank_records, a.int8_output)
    torch.cuda.synchronize()
    checked = parity_gate(p, out, launch, torch, np, accumulate) if a.check else None
    # The parity gate leaves the device idle for seconds while the host computes the expected
    # values, and a device that has been idle runs its first forwards 2-3 % slower than it does
    # once its clocks are up (about a hundred forwards of the headline configuration). The
    # benchmark is of the steady state: forwards for `--clock-warmup-s` seconds (untimed,
    # reported in the line's config) come before the W warm-up steps.
    t_end = time.perf_counter() + a.clock_warmup_s
    while time.perf_counter() < t_end:
        for _ in range(16):
            launch()
        torch.cuda.synchronize()
    for _ in range(warmup):
        launch()
    torch.cuda.synchronize()
    step = launch
    if graph:
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                launch()
        torch.cuda.synchronize()
        step = g.replay
        step()
        torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    bits, pos = st.read()
    assert bits == 0, f"the lookup rejected its inputs: status {bits:#x} at {pos}"
    ms_per_step = wall * 1e3 / steps
    forward_ms = ev0.elapsed_time(ev1) / steps  # events on the launch stream, back-to-back forwards
    kernel_ms, kernel_name = forward_ms, "lookup_lean_kernel / lookup_kernel (+ bag_order_kernel), per graph replay"
    if not graph and a.kernel_events:
        # The lookup kernels' own duration: a second region of `steps` forwards that skip the bag
        # scheduler (the order the last forward left is still valid: same offsets), bracketed by one
        # pair of HIP events on the stream the kernels are launched on. What is timed is the lookup
        # kernels back to back, so the figure includes the gap between two launches and can only
        # read longer than a kernel trace does.
        _lib.check(_lib.lib().fbgemm_amd_tbe_plan_reuse_order(plan.handle, 1))
        for _ in range(max(3, warmup // 10)):
            launch()
        torch.cuda.synchronize()
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        k0.record()
        for _ in range(steps):
            launch()
        k1.record()
        torch.cuda.synchronize()
        _lib.check(_lib.lib().fbgemm_amd_tbe_plan_reuse_order(plan.handle, 0))
        bits, pos = st.read()
        assert bits == 0, f"the lookup rejected its inputs: status {bits:#x} at {pos}"
        kernel_ms = k0.elapsed_time(k1) / steps
        kernel_name = "lookup_lean_kernel or lookup_lean_wide4_kernel (+ lookup_kernel for tables of other shapes, beside it), back to back"
    return {"ms_per_step": ms_per_step, "forward_ms": forward_ms, "kernel_ms": kernel_ms, "kernel": kernel_name,
            "checked": checked}


def accumulate_mode(a, config_id):
    if a.accumulate != "auto":
        return a.accumulate
    return "fast" if config_id == 5 else "exact"


def other_leg(p, a, torch, np, useful, steps, warmup, mode):
    """The same problem in the other accumulate mode, gated the way that mode is, for the line of a run."""
    mode = "fast" if mode == "exact" else "exact"
    m = time_tbe(p, a, torch, np, steps, warmup, False, mode)
    return {"accumulate": mode, "steps": steps, "warmup": warmup, "ms_per_step": round(m["ms_per_step"], 5),
            "value": round(useful / (m["ms_per_step"] * 1e-3) / 1e9, 2), "kernel_ms": round(m["kernel_ms"], 5),
            "forward_ms": round(m["forward_ms"], 5),
            "roofline_frac": round(useful / (m["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "checked": bool(m["checked"])}


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this path is measured on ONE GPU (no sharding, no collectives); "
              f"--gpus {a.gpus} is not supported", file=sys.stderr)
        sys.exit(2)
    if a.op == "gather_ceiling":
        return gather_ceiling(a)
    if a.op == "ref_microbench":
        return ref_microbench(a)
    if a.op != "lookup":
        return side_op(a)
    import numpy as np
    import torch

    from fbgemm_amd import bench_configs as bc

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    t_build = time.time()
    tbe = a.config in (3, 5) or (a.config == 4 and not a.per_table)
    if tbe:
        p = (bc.config3("cuda", a.scale, a.rows_scale, a.only_type) if a.config == 3 else
             bc.config5("cuda", a.scale) if a.config == 5 else bc.config4_batched("cuda", a.scale))
        lookups, useful = p.lookups, p.useful_row_bytes()
        other = p.other_bytes()
        name, dtype_out = p.name, {0: "fp32", 1: "fp16", 5: "bf16"}[p.output_dtype]
        if a.int8_output:
            dtype_out = "int8 rows with fp32 scale and bias per (bag, table)"
        launches_per_step = 1
        torch.cuda.synchronize()
        build_s = time.time() - t_build
        mode = accumulate_mode(a, a.config)
        m = time_tbe(p, a, torch, np, a.steps, a.warmup, a.graph, mode)
        ms_per_step, forward_ms, kernel_ms, kernel_name = m["ms_per_step"], m["forward_ms"], m["kernel_ms"], m["kernel"]
        checked = m["checked"]
    else:
        probs = {1: lambda: [bc.config1("cuda", a.scale)], 2: lambda: [bc.config2("cuda", a.scale)],
                 4: lambda: bc.config4("cuda", a.scale)}[a.config]()
        launch, out, st = spmdm_runner(probs, torch)
        lookups = sum(q.lookups for q in probs)
        useful = sum(q.useful_row_bytes() for q in probs)
        other = {}
        name = probs[0].name.split("[")[0] if len(probs) > 1 else probs[0].name
        dtype_out = {0: "fp32", 1: "fp16", 5: "bf16"}[probs[0].out_ty]
        launches_per_step = len(probs)
        p = None
        torch.cuda.synchronize()
        build_s = time.time() - t_build
        checked = None
        if a.check:  # the first table against the oracle, bit for bit
            import oracle
            launch()
            torch.cuda.synchronize()
            q = probs[0]
            ok, want = oracle.spmdm(q.ty, q.D, q.table.cpu().numpy(), q.host_indices, q.host_offsets,
                                    normalize=q.normalize, out_ty=q.out_ty, remap=q.host_remap, data_size=q.data_size)
            got = out[0].cpu()
            got = got.numpy() if q.out_ty == 0 else got.view(torch.int16).numpy().view(np.uint16)
            if not (ok and (got.view(want.dtype) == want).all()):
                raise AssertionError(f"parity gate: {q.name} differs from the oracle; nothing was timed")
            checked = [0]
        for _ in range(a.warmup):
            launch()
        torch.cuda.synchronize()
        step = launch
        if a.graph:
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    launch()
            torch.cuda.synchronize()
            step = graph.replay
            step()
            torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record()
        for _ in range(a.steps):
            step()
        ev1.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        bits, pos = st.read()
        assert bits == 0, f"the lookup rejected its inputs: status {bits:#x} at {pos}"
        ms_per_step = wall * 1e3 / a.steps
        forward_ms = ev0.elapsed_time(ev1) / a.steps
        kernel_ms = forward_ms
        kernel_name = "lookup_kernel (+ bag_order_kernel), per " + ("graph replay" if a.graph else "forward")
    calibration_copy(a, torch)

    gbps = useful / (ms_per_step * 1e-3) / 1e9
    kern_gbps = useful / (kernel_ms * 1e-3) / 1e9
    res = {
        "metric": "achieved HBM GB/s (% peak) + pooled rows/s, int4 TBE fwd on 1 MI355X",
        "value": round(gbps, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": name, "config_id": a.config, "scale": a.scale, "lookups_per_step": lookups,
                   "useful_row_bytes_per_step": useful, "other_bytes_per_step": other,
                   "output_dtype": dtype_out, "launches_per_step": launches_per_step, "hip_graph": bool(a.graph),
                   "accumulate": mode if tbe else "exact",
                   "untimed_clock_warmup_s": a.clock_warmup_s if tbe else 0.0},
        "checked": bool(checked), "checked_tables": checked,
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "pooled_rows_per_s": round(lookups / (ms_per_step * 1e-3), 1),
        "roofline": {"bound": "hbm", "achieved": round(kern_gbps, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(kern_gbps / HBM_PEAK_GBPS, 4),
                     "traffic": traffic_from_profile(a.config) if (a.scale == 1.0 and p is not None and not a.rows_scale
                                                                   and a.only_type is None) else None,
                     "kernel": kernel_name, "kernel_ms": round(kernel_ms / launches_per_step, 5),
                     "forward_ms": round(forward_ms, 5),
                     "kernel_ms_source": "HIP events around `steps` lookup launches without the scheduler" if tbe and not a.graph and a.kernel_events
                     else "HIP events around the timed forwards",
                     "profile_kernel_us": profile_kernel_us(a.config) if (a.scale == 1.0 and p is not None and not a.rows_scale
                                                                          and a.only_type is None) else None,
                     "algorithmic_bytes_per_launch": useful // launches_per_step},
        "setup_s": round(build_s, 1),
    }
    if p is not None and a.other_mode and not a.graph:
        res["other_accumulate"] = other_leg(p, a, torch, np, useful, a.steps, a.warmup, mode)
    if not a.no_cpu and p is not None:
        res["cpu_baseline"] = cpu_baseline_tbe(p, a.cpu_seconds, torch)
    elif not a.no_cpu:
        res["cpu_baseline"] = None
    # The default run also times config 5 (the HBM-sized int4 workload) so that its figure is
    # measured by whoever runs the default command; it is a second measurement, not part of `value`.
    default_run = (a.config == 3 and a.scale == 1.0 and not a.rows_scale and a.only_type is None and not a.graph)
    if default_run and a.also:
        del p
        torch.cuda.empty_cache()
        t5 = time.time()
        p5 = bc.config5("cuda")
        torch.cuda.synchronize()
        setup5 = time.time() - t5
        steps5, warm5 = max(5, min(a.steps, 30)), max(1, min(a.warmup, 3))
        mode5 = accumulate_mode(a, 5)
        m5 = time_tbe(p5, a, torch, np, steps5, warm5, False, mode5)
        useful5 = p5.useful_row_bytes()
        res["also"] = {"config5": {
            "workload": p5.name, "accumulate": mode5, "steps": steps5, "warmup": warm5, "ms_per_step": round(m5["ms_per_step"], 5),
            "value": round(useful5 / (m5["ms_per_step"] * 1e-3) / 1e9, 2), "unit": "GB/s",
            "pooled_rows_per_s": round(p5.lookups / (m5["ms_per_step"] * 1e-3), 1),
            "lookups_per_step": p5.lookups, "useful_row_bytes_per_step": useful5,
            "checked": bool(m5["checked"]), "checked_tables": m5["checked"],
            "roofline": {"bound": "hbm", "achieved": round(useful5 / (m5["kernel_ms"] * 1e-3) / 1e9, 2),
                         "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(useful5 / (m5["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                         "traffic": traffic_from_profile(5), "kernel": m5["kernel"],
                         "kernel_ms": round(m5["kernel_ms"], 5), "forward_ms": round(m5["forward_ms"], 5),
                         "profile_kernel_us": profile_kernel_us(5),
                         "algorithmic_bytes_per_launch": useful5},
            "setup_s": round(setup5, 1)}}
        if a.other_mode:
            res["also"]["config5"]["other_accumulate"] = other_leg(p5, a, torch, np, useful5, steps5, warm5, mode5)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
