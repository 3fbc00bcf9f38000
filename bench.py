#!/usr/bin/env python3
"""Benchmark of the int8 quantized-GEMM inference path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]
                    [--only gemm|gemv|ln|softmax|other|pipeline|c1|chains|ceilings|calib]

One "step" is one pass of the path over the north-star workload: activations A fp16
[1,4096,4096] ~N(0,1) and weights W fp16 [1,10240,4096] ~N(0,0.02) (seed 1000, generated on
the CPU and resident in HBM before timing) through ``bmm(A, False, W, True, int8=True)`` --
row-absmax scales and int8 rounding of both operands, int8 MFMA GEMM with int32 accumulation,
fp16 dequantisation -- exactly what the reference's GEMMInt8.forward does per call.

Prints ONE JSON line.  `value` is 2*M*N*K / step time in TOP/s for that whole step (W warm-up and K
timed steps on the device kept busy by the per-kernel legs; `from_idle` is the same W + K run first
thing in the process, while the device's clock is still rising); the
`roofline` object is the GEMM kernel alone against the dense int8 MFMA peak; `components`
carries the decode GEMV, layernorm and softmax kernels (and, after them, every other kernel of
the path) against the HBM peak; `cpu_baseline`
is the torch formulation of the same step timed on the host cores (a reported baseline);
`ceilings` holds what yardstick kernels that do nothing else reach on the same chip in the same
run (matrix pipe on zero / random operands, plain and tiled copies, a cold 42 MB read) and the
vendor library's int8 product on the same shapes (calibration only; the library does not use it).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0      # MI355X dense int8 MFMA, published
PEAK_HBM_GBS = 8000.0        # MI355X HBM3E, published
M, K, N = 4096, 4096, 10240  # north-star GEMM

# Hardware-counter figures cannot be taken from inside this process.  They come from offline runs --
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` over `python3 bench.py --no-cpu --only <workload>`,
# each counter scaled by what it reads for the 256 MiB device copy of `--only calib`; MFMA pipe busy
# cycles / kernel cycles from SQ_VALU_MFMA_BUSY_CYCLES and SQ_BUSY_CYCLES -- whose summaries are the
# text files under profiles/.  The figures are read from those files at run time (never typed in here)
# and emitted with their source, so that they are not mistaken for measurements of this run.
PROFILES = os.path.join(ROOT, "profiles")
OFFLINE_SOURCE = {"traffic": "profiles/hbm_traffic_counters.txt (offline rocprofv3 --pmc run of this bench, read at run time, not measured by this process)",
                  "mfma": "profiles/gemm_mfma_utilisation.txt (offline rocprofv3 --pmc run of this bench, read at run time, not measured by this process)"}
# which row of profiles/hbm_traffic_counters.txt belongs to which workload (a substring of the kernel's name)
TRAFFIC_KERNELS = {"gemm_fused": "k_gemm_dma<2, 4, 4, 2, 128, 1,", "gemv": "k_gemv_coalescedILi8ELi3ELi2ELb0", "layernorm": "k_layernorm_teamILi1024ELi8ELb0", "softmax": "k_softmax_stream"}


def offline_counters():
    """({workload: HBM bytes per launch}, MFMA busy fraction of the fused GEMM kernel's cycles) from the
    summaries under profiles/; a missing or unreadable figure is None."""
    traffic = {k: None for k in TRAFFIC_KERNELS}
    try:
        for ln in open(os.path.join(PROFILES, "hbm_traffic_counters.txt")):
            f = ln.split()
            if len(f) < 8:
                continue
            try:
                total_mb, calls = float(f[-1]), int(f[-6])
            except ValueError:
                continue
            for k, sub in TRAFFIC_KERNELS.items():
                if sub in ln and calls > 1 and traffic[k] is None:      # (single-call rows are the set-up launches)
                    traffic[k] = round(total_mb * 1e6)
    except OSError:
        pass
    busy = None
    try:
        fused = False
        for ln in open(os.path.join(PROFILES, "gemm_mfma_utilisation.txt")):
            if ln.startswith("k_gemm_dma"):
                fused = TRAFFIC_KERNELS["gemm_fused"] in ln
            elif fused and "MFMA utilisation" in ln and busy is None:
                busy = float(ln.split()[3])
    except (OSError, ValueError, IndexError):
        pass
    return traffic, busy


TRAFFIC_BYTES, MFMA_BUSY_FRAC = offline_counters()


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--only", default="", help="run only one leg (for profiling): gemm|gemv|ln|softmax|other|pipeline|c1|chains|ceilings|calib "
                        "(calib = a plain 256 MiB device copy, the known-size kernel that scales the HBM counters)")
    p.add_argument("--reps", type=int, default=200, help="launches per timed batch in the per-kernel loops")
    return p.parse_args()


SETTLE_S = 0.05     # the device raises its clock over the first ~30 ms of load; per-kernel loops are timed after this much of it


def settle(fn, seconds=SETTLE_S):
    """Keep the device busy with fn for `seconds` (host clock), so that what follows is timed at the clock a
    sustained load runs at.  Not used for the W + K steps of `value`, whose warm-up is W steps by definition."""
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()


def event_ms(fn, reps, warmup=3, batches=5):
    """Milliseconds per call of fn from HIP events on torch's current stream (the stream every
    launcher is given): `reps` back-to-back calls split into `batches` timed batches, median batch.
    (One long batch is at the mercy of a single stall -- a monitoring tool sampling the device
    takes tens of milliseconds now and then -- which the median discards.)"""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    settle(fn)
    per = max(1, reps // batches)
    times = []
    for _ in range(batches):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(per):
            fn()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) / per)
    return sorted(times)[len(times) // 2]


def sclk_under_load(fn, seconds):
    """Median shader clock in MHz that the driver reports (the current level of pp_dpm_sclk in sysfs, the file the
    monitoring tools read) while fn is launched back to back for `seconds`; None if no such file can be read.
    The file is read in this process: nothing is spawned."""
    import glob
    import re
    import threading
    import torch
    paths = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
    samples, stop = [], [False]

    def current_mhz():
        for p in paths:
            try:
                with open(p) as f:
                    m = re.search(r"(\d+)Mhz\s*\*", f.read())
            except OSError:
                continue
            if m:
                return int(m.group(1))
        return None

    def sampler():
        while not stop[0]:
            v = current_mhz()
            if v is None:
                return
            samples.append(v)
            time.sleep(0.05)
    th = threading.Thread(target=sampler)
    th.start()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
    stop[0] = True
    th.join()
    samples = sorted(samples[2:] or samples)      # (the first samples may predate the load)
    return samples[len(samples) // 2] if samples else None


GRAPH_NODES = 64    # kernel launches per captured graph


def graph_ms(launches, reps):
    """Capture the launch closures into a HIP graph (no host launch overhead between kernels) and time replays;
    returns ms per launch.  The list is repeated until the graph holds GRAPH_NODES launches: between two graph
    launches the device idles for several microseconds, which a short graph charges to its few kernels (an empty
    kernel costs 2.55 us per launch in a graph of 8 and 1.67 us in a graph of 64).  `reps` = launches of each
    closure per timed batch.  Falls back to eager timing if capture is unavailable."""
    import torch
    n = len(launches)
    copies = max(1, GRAPH_NODES // n) if n < GRAPH_NODES else 1
    try:
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for f in launches:
                f()
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(copies):
                for f in launches:
                    f()
        g.replay()
        torch.cuda.synchronize()
        settle(g.replay)
        per = max(2, (reps // 3 + copies - 1) // copies)
        times = []
        for _ in range(3):                   # three timed batches of replays, median batch
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(per):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) / (per * n * copies))
        return sorted(times)[1], "hipgraph of %d launches" % (n * copies)
    except Exception as ex:   # pragma: no cover
        sys.stderr.write("graph capture failed (%s); eager timing\n" % ex)
        i = [0]

        def one():
            launches[i[0] % len(launches)]()
            i[0] += 1
        return event_ms(one, reps * len(launches)), "eager"


def main():
    args = parse()
    if args.gpus != 1:
        sys.stderr.write("bench.py measures one GPU: the path has no collectives and every GPU box of this "
                         "build has a single MI355X; --gpus %d is not supported\n" % args.gpus)
        sys.exit(2)
    import torch
    from cpm_kernels_amd.build import library_path, build_library
    if not os.path.exists(library_path()):
        build_library(verbose=False)
    from cpm_kernels_amd.library import cpmk
    import cpm_kernels_amd.kernels as ck
    import cpm_kernels_amd.torch as ct
    assert cpmk.lib.loaded, "libcpmk_hip.so missing"
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    st = lambda: torch.cuda.current_stream().cuda_stream   # noqa: E731
    only = args.only
    result = {}

    # peaks: the published ones every `frac` divides by, and the ones this device's own clocks give
    props = cpmk.device_props(0)
    peak_int8_clock = props["compute_units"] * props["clock_khz"] * 1e3 * 8192 / 1e12          # CUs x clock x 8192 int8 ops/clk/CU
    peak_hbm_clock = props["mem_clock_khz"] * 1e3 * 2 * props["mem_bus_bits"] / 8 / 1e9        # memory clock x 2 (double data rate) x bus width
    result["peaks"] = {
        "int8_tops_published": PEAK_INT8_TOPS, "hbm_gbs_published": PEAK_HBM_GBS,
        "int8_tops_clock_derived": round(peak_int8_clock, 1), "hbm_gbs_clock_derived": round(peak_hbm_clock, 1),
        "formula": "int8: compute_units x clock_khz x 8192 ops/clk/CU; hbm: mem_clock_khz x 2 x mem_bus_bits / 8",
        "compute_units": props["compute_units"], "clock_khz": props["clock_khz"], "mem_clock_khz": props["mem_clock_khz"],
        "mem_bus_bits": props["mem_bus_bits"], "l2_bytes": props["l2_bytes"], "arch": props["name"]}

    if only == "calib":
        # a copy of known size: FETCH_SIZE / WRITE_SIZE read for it give the counters' scale
        src = torch.randint(-128, 128, (256 << 20,), dtype=torch.int8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calib": "5 device copies of %d bytes (read + write each)" % src.numel()}), flush=True)
        return

    # ---- north-star workload ---------------------------------------------------------------
    g = torch.Generator().manual_seed(1000)
    A_cpu = torch.randn(1, M, K, generator=g).half()
    W_cpu = (torch.randn(1, N, K, generator=g) * 0.02).half()
    A, W = A_cpu.to(dev), W_cpu.to(dev)
    ops = 2.0 * M * N * K

    def leg_pipeline():
        """W untimed warm-up steps, then exactly K timed steps between synchronisations: (ms per step from HIP events, from the host clock)."""
        def step():
            return ct.bmm(A, False, W, True, int8=True)
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            step()
        e1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / args.steps
        return max(e0.elapsed_time(e1) / args.steps, 0.0), wall

    def leg_gemm():
        """The GEMM kernel alone (roofline)."""
        sA = torch.empty((1, M), dtype=torch.half, device=dev); qA = torch.empty((1, M, K), dtype=torch.int8, device=dev)
        sW = torch.empty((1, N), dtype=torch.half, device=dev); qW = torch.empty((1, N, K), dtype=torch.int8, device=dev)
        ck.gemm_quantize(1, M, K, A.data_ptr(), sA.data_ptr(), qA.data_ptr(), False, st())
        ck.gemm_quantize(1, N, K, W.data_ptr(), sW.data_ptr(), qW.data_ptr(), False, st())
        out16 = torch.empty((1, M, N), dtype=torch.half, device=dev)

        def gemm():
            ck.gemm_int8_scale(N, K, M, 1, 1, True, False, qW.data_ptr(), qA.data_ptr(), sA.data_ptr(), sW.data_ptr(),
                               True, True, out16.data_ptr(), st())
        # The shader clock under this kernel, as the driver reports it while the kernel runs back to back for a
        # second (not inside a timed loop: a sample may stall the device for a moment), on the step's operands and on all-zero
        # ones: the kernel needs the same number of cycles for both, the chip clocks lower on the operands that toggle.
        qz_a, qz_w = torch.zeros_like(qA), torch.zeros_like(qW)

        def gemm_zero():
            ck.gemm_int8_scale(N, K, M, 1, 1, True, False, qz_w.data_ptr(), qz_a.data_ptr(), sA.data_ptr(), sW.data_ptr(),
                               True, True, out16.data_ptr(), st())
        clocks = {}
        for label, fn in (("step_operands", gemm), ("zero_operands", gemm_zero)):
            mhz = sclk_under_load(fn, 1.2)
            ms_l = event_ms(fn, 20, warmup=3)
            clocks[label] = {"sclk_mhz": mhz, "kernel_us": round(ms_l * 1e3, 2),
                             "kilocycles": round(ms_l * 1e3 * mhz / 1e3, 1) if mhz else None}
        clock_under_load = dict(clocks, source="current level of /sys/class/drm/card*/device/pp_dpm_sclk sampled while the kernel runs back to back; kilocycles = kernel_us x sclk")
        del qz_a, qz_w
        ms = event_ms(gemm, max(20, args.steps), warmup=max(3, args.warmup))
        tops = ops / (ms * 1e-3) / 1e12
        roofline = {"kernel": "k_gemm_dma<2,4,4,2,128,1,true,2,0,16> (int8 MFMA GEMM + fused fp16 dequant), M=%d K=%d N=%d" % (M, K, N),
                    "bound": "mfma", "achieved": round(tops, 2), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                    "ops": "int8 multiply-accumulates counted as 2 ops",
                    "frac": round(tops / PEAK_INT8_TOPS, 4), "avg_kernel_us": round(ms * 1e3, 2),
                    "peak_clock_derived": round(peak_int8_clock, 1), "frac_of_clock_derived": round(tops / peak_int8_clock, 4),
                    "operands": "MALL-resident (one 58.7 MB operand pair and one 83.9 MB output reused by every launch)",
                    "traffic": TRAFFIC_BYTES["gemm_fused"], "traffic_unit": "bytes per launch (HBM fetch + write counters)",
                    "traffic_source": OFFLINE_SOURCE["traffic"],
                    "mfma_busy_frac_of_cycles": MFMA_BUSY_FRAC, "mfma_busy_source": OFFLINE_SOURCE["mfma"],
                    "algorithmic_bytes": M * K + N * K + 2 * M * N, "clock_under_load": clock_under_load}
        out32 = torch.empty((1, M, N), dtype=torch.int32, device=dev)

        def gemm32():
            ck.gemm_int8(N, K, M, 1, 1, True, False, qW.data_ptr(), qA.data_ptr(), out32.data_ptr(), st())
        ms32 = event_ms(gemm32, max(20, args.steps), warmup=3)
        roofline["int32_out_tops"] = round(ops / (ms32 * 1e-3) / 1e12, 2)
        roofline["timing"] = "HIP events around back-to-back eager launches, median of 5 batches (replayed from a graph without launch gaps the kernel runs 3-4 % slower: the clock follows the sustained load)"
        return roofline

    # The device raises its clock over the first ~30 ms of load (the same step takes 212, 190, 178, 172, 168 us
    # in consecutive batches of 25 right after start or half a second of idling; the GEMM alone 160 ... 135 us).
    # The W + K steps are therefore run twice: first thing in the process ("from_idle", reported beside the
    # result) and, for `value`, at the end of the per-kernel legs, right after the roofline loop of the GEMM
    # kernel has kept the device busy -- the state a serving loop is in.  With --only pipeline there is only
    # the first.
    step_ms = None
    roofline = None
    if only in ("", "pipeline"):
        step_ms, wall_ms = leg_pipeline()
        result["wall_ms_per_step"] = round(wall_ms, 4)
        result["from_idle"] = {"ms_per_step": round(step_ms, 4), "value": round(ops / (step_ms * 1e-3) / 1e12, 2),
                               "note": "the same W warm-up + K timed steps as `value`, run first thing in the process: the device's clock is still rising"}
    if only == "gemm":
        roofline = leg_gemm()

    components = {}
    reps = args.reps

    # ---- config 1: the reference's own test shape, A [1,512,4096] x W [1,4096,4096] ----------------
    if only in ("", "c1"):
        gg = torch.Generator().manual_seed(1001)
        A1 = torch.randn(1, 512, 4096, generator=gg).half().to(dev)
        W1c = (torch.randn(1, 4096, 4096, generator=gg) * 0.02).half().to(dev)
        ops1 = 2.0 * 512 * 4096 * 4096
        sA1 = torch.empty((1, 512), dtype=torch.half, device=dev); qA1 = torch.empty((1, 512, 4096), dtype=torch.int8, device=dev)
        sW1 = torch.empty((1, 4096), dtype=torch.half, device=dev); qW1 = torch.empty((1, 4096, 4096), dtype=torch.int8, device=dev)
        acc1 = torch.empty((1, 512, 4096), dtype=torch.int32, device=dev); o1 = torch.empty((1, 512, 4096), dtype=torch.half, device=dev)

        def c1_kernel_by_kernel():      # the six launches of the reference's pipeline (tests/test_gemm.py, torch/gemm.py:40-66)
            ck.gemm_calc_scale(1, 512, 4096, A1.data_ptr(), sA1.data_ptr(), st())
            ck.gemm_calc_scale(1, 4096, 4096, W1c.data_ptr(), sW1.data_ptr(), st())
            ck.gemm_round(1, 512, 4096, A1.data_ptr(), sA1.data_ptr(), qA1.data_ptr(), st())
            ck.gemm_round(1, 4096, 4096, W1c.data_ptr(), sW1.data_ptr(), qW1.data_ptr(), st())
            ck.gemm_int8(4096, 4096, 512, 1, 1, True, False, qW1.data_ptr(), qA1.data_ptr(), acc1.data_ptr(), st())
            ck.gemm_scale(1, 512, 4096, acc1.data_ptr(), sA1.data_ptr(), sW1.data_ptr(), o1.data_ptr(), True, True, st())
        # ten launches per captured graph, so that the replay overhead is shared like in the other legs
        ms_six, how = graph_ms([c1_kernel_by_kernel] * 10, max(5, reps // 10))
        ms_g32, _ = graph_ms([lambda: ck.gemm_int8(4096, 4096, 512, 1, 1, True, False, qW1.data_ptr(), qA1.data_ptr(), acc1.data_ptr(), st())] * 10, max(5, reps // 10))
        ms_g16, _ = graph_ms([lambda: ck.gemm_int8_scale(4096, 4096, 512, 1, 1, True, False, qW1.data_ptr(), qA1.data_ptr(), sA1.data_ptr(),
                                                         sW1.data_ptr(), True, True, o1.data_ptr(), st())] * 10, max(5, reps // 10))
        ms_pair, _ = graph_ms([lambda: ck.gemm_quantize_pair(512, A1.data_ptr(), sA1.data_ptr(), qA1.data_ptr(), 4096, W1c.data_ptr(), sW1.data_ptr(),
                                                            qW1.data_ptr(), 4096, st())] * 10, max(5, reps // 10))
        ms_bmm = event_ms(lambda: ct.bmm(A1, False, W1c, True, int8=True), max(20, reps // 2), warmup=10)
        components["config 1 pipeline (A [1,512,4096] x W [1,4096,4096])"] = {
            "bound": "mfma", "ops": ops1, "seed": 1001, "operands": "MALL-resident",
            "gemm_int8_us": round(ms_g32 * 1e3, 2), "gemm_int8_tops": round(ops1 / (ms_g32 * 1e-3) / 1e12, 1),
            "gemm_int8_scale_fused_us": round(ms_g16 * 1e3, 2), "gemm_int8_scale_fused_tops": round(ops1 / (ms_g16 * 1e-3) / 1e12, 1),
            "frac": round(ops1 / (ms_g16 * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
            "six_kernel_pipeline_us": round(ms_six * 1e3, 2), "quantize_pair_us": round(ms_pair * 1e3, 2), "bmm_int8_us": round(ms_bmm * 1e3, 2),
            "bmm_int8_tops": round(ops1 / (ms_bmm * 1e-3) / 1e12, 1), "timing": how + " (kernels), events (bmm)"}
        del A1, W1c, qA1, qW1, acc1, o1

    # ---- configs 4 and 5 as whole chains through the torch wrappers, native (batch, hidden, seq) layout ----
    if only in ("", "chains"):
        with torch.no_grad():
            d, dff = 4096, 10240
            gg = torch.Generator().manual_seed(1004)
            b4, s4 = 8, 512
            x4 = torch.randn(b4, d, s4, generator=gg).half().to(dev)
            W1f = (torch.randn(1, dff, d, generator=gg) * 0.02).half().to(dev); W2f = (torch.randn(1, d, dff, generator=gg) * 0.02).half().to(dev)
            ln4 = ct.LayerNorm(d, bias=True).half().to(dev)
            ln4.weight.copy_((1 + 0.1 * torch.randn(d, generator=gg)).half()); ln4.bias.copy_((0.1 * torch.randn(d, generator=gg)).half())

            def ffn(x, ln, Wa, Wb):
                h = ct.bmm(Wa, False, ln(x), False, int8=True)
                h = ct.bmm(Wb, False, ct.gelu(h), False, int8=True)
                return ct.element_add(h, x)
            ms4 = event_ms(lambda: ffn(x4, ln4, W1f, W2f), 20)
            ops4 = 2.0 * 2 * b4 * s4 * d * dff
            components["config 4 FFN block (tokens 8 x 512)"] = {
                "chain": "LayerNorm -> int8 bmm 4096->10240 -> gelu -> int8 bmm 10240->4096 -> residual add (weights and activations quantised in every call)",
                "seed": 1004, "avg_us": round(ms4 * 1e3, 1), "tops_over_the_two_products": round(ops4 / (ms4 * 1e-3) / 1e12, 1),
                "tokens_per_s": round(b4 * s4 / (ms4 * 1e-3), 0), "timing": "events, whole chain"}
            del x4

            gg = torch.Generator().manual_seed(1005)
            b5, H, dh, s5 = 16, 64, 64, 1024
            x5 = torch.randn(b5, d, s5, generator=gg).half().to(dev)
            Wp = {n_: (torch.randn(1, d, d, generator=gg) * 0.02).half().to(dev) for n_ in "qkvo"}
            ln1 = ct.LayerNorm(d, bias=True).half().to(dev); ln2 = ct.LayerNorm(d, bias=True).half().to(dev)
            pe = ct.PositionEmbedding(H, 32, 128, True).half().to(dev)
            pe.weight.copy_((torch.randn(H, 32, generator=gg) * 0.02).half())
            lens = torch.randint(512, 1025, (b5,), generator=gg)
            pad = (torch.arange(s5)[None, :] < lens[:, None]).to(dev)

            def layer(x):
                h = ln1(x)
                q, k, v = (ct.bmm(Wp[n_], False, h, False, int8=True).view(b5 * H, dh, s5) for n_ in "qkv")
                ct.global_scale_inplace(q, 1.0 / dh ** 0.5)      # 1/8: exact in fp16, so scaling q (134 MB) instead of the scores (2 GB) gives the same bits
                scores = ct.bmm(k, True, q, False, int8=False)                       # (b*H, len_k, len_q)
                bias = pe(s5, s5)
                scores = ct.batched_add(scores.view(b5, H * s5 * s5), bias.view(-1)).view(b5, H * s5, s5)
                ct.mask_inplace(scores, pad, float("-inf"))
                scores = scores.view(b5 * H, s5, s5)
                ct.softmax_inplace(scores)
                ctx = ct.bmm(v, False, scores, False, int8=False).view(b5, d, s5)
                y = ct.element_add(ct.bmm(Wp["o"], False, ctx, False, int8=True), x)
                return ffn(y, ln2, W1f, W2f)
            ms5 = event_ms(lambda: layer(x5), 5, warmup=2)
            ops5 = 2.0 * b5 * s5 * (4 * d * d + 2 * d * dff) + 2.0 * 2 * b5 * H * s5 * s5 * dh
            components["config 5 transformer layer (batch 16, seq 1024)"] = {
                "chain": "LayerNorm -> int8 q,k,v -> q / sqrt(d_head) -> fp16 scores -> T5 bias, padding mask, softmax (one launch each) -> fp16 PV -> int8 out-proj + residual -> LayerNorm -> int8 FFN with gelu + residual",
                "seed": 1005, "avg_ms": round(ms5, 3), "tops_overall": round(ops5 / (ms5 * 1e-3) / 1e12, 1),
                "tokens_per_s": round(b5 * s5 / (ms5 * 1e-3), 0), "timing": "events, whole chain"}
            del x5, Wp, W1f, W2f
            torch.cuda.empty_cache()

    # ---- HBM-bound components ---------------------------------------------------------------

    def hbm(name, nbytes, ms, how, shape, traffic):
        gbs = nbytes / (ms * 1e-3) / 1e9
        components[name] = {"shape": shape, "bound": "hbm", "algorithmic_bytes": int(nbytes), "avg_us": round(ms * 1e3, 3),
                            "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                            "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": traffic, "timing": how}
        if traffic is not None:
            components[name]["traffic_source"] = OFFLINE_SOURCE["traffic"]

    if only in ("", "gemv"):
        # config 2: W int8 [10240,4096], 32 vectors; 8 weight copies (336 MB) rotate so every
        # launch streams its matrix from HBM, not from the 256 MB Infinity Cache.  Then the decode shapes of
        # configs 4 and 5 (the FFN's two projections and the attention projections) at 1, 8 and 32 vectors.
        gg = torch.Generator().manual_seed(1002)
        nrot = 8
        for dim_out, dim_in in ((10240, 4096), (4096, 10240), (4096, 4096)):
            mats = [torch.randint(-127, 128, (dim_out, dim_in), generator=gg, dtype=torch.int8).to(dev) for _ in range(nrot * (2 if dim_out * dim_in < (32 << 20) else 1))]
            smat = (torch.rand(dim_out, generator=gg) * 0.009 + 0.001).half().to(dev)
            for nv in (32, 8, 1):
                v = torch.randn(nv, dim_in, generator=gg).half().to(dev)
                sv = torch.empty((nv,), dtype=torch.half, device=dev); qv = torch.empty((nv, dim_in), dtype=torch.int8, device=dev)
                ck.gemv_calc_scale(nv, dim_in, v.data_ptr(), sv.data_ptr(), st())
                ck.gemv_round(nv, dim_in, v.data_ptr(), sv.data_ptr(), qv.data_ptr(), st())
                o = torch.empty((nv, dim_out), dtype=torch.half, device=dev)
                launches = [(lambda m_=m_: ck.gemv_broadcast_mat_int8(nv, dim_out, dim_in, smat.data_ptr(), m_.data_ptr(), sv.data_ptr(),
                                                                       qv.data_ptr(), o.data_ptr(), st())) for m_ in mats]
                ms, how = graph_ms(launches, max(5, reps // nrot))
                headline = (dim_out, dim_in, nv) == (10240, 4096, 32)
                hbm("gemv_broadcast_mat_int8" if headline else "gemv_broadcast_mat_int8 [%d,%d] x %d" % (dim_out, dim_in, nv),
                    dim_out * dim_in + nv * dim_in + 2 * nv * dim_out + 2 * dim_out + 2 * nv, ms, how,
                    "W int8 [%d,%d] x %d vectors" % (dim_out, dim_in, nv), TRAFFIC_BYTES["gemv"] if headline else None)
            del mats

    if only in ("", "ln"):
        gg = torch.Generator().manual_seed(1003)
        nrot = 10    # 10 x 33.5 MB inputs
        xs = [torch.randn(8, 4096, 512, generator=gg).half().to(dev) for _ in range(nrot)]
        y = torch.empty_like(xs[0])
        launches = [(lambda x_=x_: ck.layernorm_forward(8, 4096, 512, x_.data_ptr(), y.data_ptr(), 1e-5, True, st()))
                    for x_ in xs]
        ms, how = graph_ms(launches, max(5, reps // nrot))
        hbm("layernorm_forward", 4 * 8 * 4096 * 512, ms, how, "[8,4096,512] fp16, dim 1", TRAFFIC_BYTES["layernorm"])
        del xs

    if only in ("", "softmax"):
        gg = torch.Generator().manual_seed(1003)
        s = (torch.randn(64, 1024, 1024, generator=gg) * 4).half()
        kk = torch.arange(1024)[:, None]; qq = torch.arange(1024)[None, :]
        s.masked_fill_((kk > qq)[None], float("-inf"))
        sd = s.to(dev).repeat(8, 1, 1).contiguous()          # [512,1024,1024], 1.07 GB
        del s
        so = torch.empty_like(sd)
        launches = [lambda: ck.softmax_forward(512, 1024, 1024, sd.data_ptr(), so.data_ptr(), st())]
        ms, how = graph_ms(launches, max(3, reps // 20))
        hbm("softmax_forward", 4 * 512 * 1024 * 1024, ms, how, "[512,1024,1024] fp16 causal, dim 1", TRAFFIC_BYTES["softmax"])
        del sd, so

    if only in ("", "other"):
        # the other kernels of the path, each at the size its config gives it
        gg = torch.Generator().manual_seed(1004)

        def rot(shape, count, scale=1.0, dtype=torch.half):
            return [(torch.randn(*shape, generator=gg) * scale).to(dtype).to(dev) for _ in range(count)]
        Ws = rot((1, N, K), 3, 0.02)                              # 3 x 84 MB
        sW = torch.empty((1, N), dtype=torch.half, device=dev); qW = torch.empty((1, N, K), dtype=torch.int8, device=dev)
        ms, how = graph_ms([(lambda w=w: ck.gemm_quantize(1, N, K, w.data_ptr(), sW.data_ptr(), qW.data_ptr(), False, st())) for w in Ws], max(3, reps // 12))
        hbm("gemm_quantize (calc_scale+round) W", 3 * N * K + 2 * N, ms, how, "[10240,4096] fp16 -> int8 + row scales", None)
        ms, how = graph_ms([(lambda w=w: ck.gemm_calc_scale(1, N, K, w.data_ptr(), sW.data_ptr(), st())) for w in Ws], max(3, reps // 12))
        hbm("gemm_calc_scale W", 2 * N * K + 2 * N, ms, how, "[10240,4096] fp16", None)
        ms, how = graph_ms([(lambda w=w: ck.gemm_round(1, N, K, w.data_ptr(), sW.data_ptr(), qW.data_ptr(), st())) for w in Ws], max(3, reps // 12))
        hbm("gemm_round W", 3 * N * K + 2 * N, ms, how, "[10240,4096] fp16 -> int8", None)
        del Ws, qW
        accs = [torch.randint(-3000000, 3000000, (1, M, N), generator=gg, dtype=torch.int32).to(dev) for _ in range(2)]
        sA = (torch.rand(M, generator=gg) * 0.03).half().to(dev); sN = (torch.rand(N, generator=gg) * 0.001).half().to(dev)
        o16 = torch.empty((1, M, N), dtype=torch.half, device=dev)
        ms, how = graph_ms([(lambda a_=a_: ck.gemm_scale(1, M, N, a_.data_ptr(), sA.data_ptr(), sN.data_ptr(), o16.data_ptr(), True, True, st())) for a_ in accs], max(3, reps // 8))
        hbm("gemm_scale", 6 * M * N + 2 * (M + N), ms, how, "[4096,10240] int32 -> fp16", None)
        del accs, o16
        xs = rot((8, 4096, 512), 10)                              # C3 / C4 activations, 10 x 33.5 MB
        y = torch.empty_like(xs[0])
        al = (1 + 0.1 * torch.randn(4096, generator=gg)).half().to(dev); be = (0.1 * torch.randn(4096, generator=gg)).half().to(dev)
        ms, how = graph_ms([(lambda x_=x_: ck.layernorm_affine_forward(8, 4096, 512, x_.data_ptr(), al.data_ptr(), be.data_ptr(), y.data_ptr(), 1e-5, True, st())) for x_ in xs], max(5, reps // 10))
        hbm("layernorm + gamma/beta (fused)", 4 * 8 * 4096 * 512, ms, how, "[8,4096,512] fp16", None)
        ms, how = graph_ms([(lambda x_=x_: ck.arith_ln_mul_add(8, 4096, 512, x_.data_ptr(), al.data_ptr(), be.data_ptr(), y.data_ptr(), st())) for x_ in xs], max(5, reps // 10))
        hbm("arith_ln_mul_add", 4 * 8 * 4096 * 512, ms, how, "[8,4096,512] fp16", None)
        ms, how = graph_ms([(lambda i=i: ck.arith_element_add(8, 4096 * 512, xs[i].data_ptr(), xs[(i + 1) % 10].data_ptr(), y.data_ptr(), st())) for i in range(10)], max(5, reps // 10))
        hbm("arith_element_add", 6 * 8 * 4096 * 512, ms, how, "[8, 4096*512] fp16", None)
        mk = (torch.rand(8, 512, generator=gg) > 0.3).to(dev)
        ms, how = graph_ms([(lambda x_=x_: ck.mask(8, 4096, 512, x_.data_ptr(), mk.data_ptr(), float("-inf"), y.data_ptr(), st())) for x_ in xs], max(5, reps // 10))
        hbm("mask", 4 * 8 * 4096 * 512 + 8 * 512, ms, how, "[8,4096,512] fp16", None)
        sX = torch.empty((8, 512), dtype=torch.half, device=dev); qX = torch.empty((8, 512, 4096), dtype=torch.int8, device=dev)
        ms, how = graph_ms([(lambda x_=x_: ck.gemm_quantize_cols(8, 4096, 512, x_.data_ptr(), sX.data_ptr(), qX.data_ptr(), True, st())) for x_ in xs], max(5, reps // 10))
        hbm("gemm_quantize_cols (transposed int8 out)", 3 * 8 * 4096 * 512 + 2 * 8 * 512, ms, how, "[8,4096,512] fp16, per-column scales", None)
        del xs, y, qX
        gs = rot((8, 10240 * 512), 3)                             # C4 gelu input, 3 x 84 MB
        go = torch.empty_like(gs[0])
        ms, how = graph_ms([(lambda x_=x_: ck.gelu_forward(8, 10240 * 512, x_.data_ptr(), go.data_ptr(), st())) for x_ in gs], max(3, reps // 12))
        hbm("gelu_forward", 4 * 8 * 10240 * 512, ms, how, "[8, 10240*512] fp16", None)
        del gs, go
        tbl = torch.empty(128, dtype=torch.int32, device=dev)
        ck.position_embedding_init(32, 128, tbl.data_ptr(), True, st())
        pw = (torch.randn(64, 32, generator=gg) * 0.02).half().to(dev)
        pos = [torch.empty((64, 1024, 1024), dtype=torch.half, device=dev) for _ in range(3)]
        ms, how = graph_ms([(lambda o_=o_: ck.position_embedding_forward(1024, 1024, 32, 128, 64, tbl.data_ptr(), pw.data_ptr(), o_.data_ptr(), True, st())) for o_ in pos], max(3, reps // 12))
        hbm("position_embedding_forward", 2 * 64 * 1024 * 1024 + 2 * 64 * 32 + 4 * 128, ms, how, "64 heads x 1024 x 1024 fp16 written", None)
        del pos
        # fp16 decode-step products: one weight matrix for 32 vectors, and attention over a key / value cache
        # of 32 sequences x 64 heads x 1024 positions x 64 (2 x 268 MB rotate)
        wf = rot((10240, 4096), 4)
        vf = torch.randn(32, 4096, generator=gg).half().to(dev); of = torch.empty((32, 10240), dtype=torch.half, device=dev)
        ms, how = graph_ms([(lambda w_=w_: ck.gemv_broadcast_mat_fp16(32, 10240, 4096, w_.data_ptr(), vf.data_ptr(), of.data_ptr(), st())) for w_ in wf], max(3, reps // 8))
        hbm("gemv_broadcast_mat_fp16", 2 * 10240 * 4096 + 2 * 32 * 4096 + 2 * 32 * 10240, ms, how, "W fp16 [10240,4096] x 32 vectors", None)
        ms, how = graph_ms([(lambda w_=w_: ck.gemv_broadcast_mat_fp16(1, 10240, 4096, w_.data_ptr(), vf.data_ptr(), of.data_ptr(), st())) for w_ in wf], max(3, reps // 8))
        hbm("gemv_broadcast_mat_fp16 x 1", 2 * 10240 * 4096 + 2 * 4096 + 2 * 10240, ms, how, "W fp16 [10240,4096] x 1 vector (row-wise kernel, no matrix cores)", None)
        del wf
        kc = rot((2048, 1024, 64), 2)
        qf = torch.randn(2048, 64, generator=gg).half().to(dev); sc = torch.empty((2048, 1024), dtype=torch.half, device=dev)
        ms, how = graph_ms([(lambda k_=k_: ck.gemv_fp16(2048, 1024, 64, k_.data_ptr(), qf.data_ptr(), sc.data_ptr(), st())) for k_ in kc], max(3, reps // 8))
        hbm("gemv_fp16 (attention scores over a key cache)", 2 * 2048 * 1024 * 64 + 2 * 2048 * 64 + 2 * 2048 * 1024, ms, how, "2048 x [1024,64] fp16", None)
        ov = torch.empty((2048, 64), dtype=torch.half, device=dev)
        ms, how = graph_ms([(lambda k_=k_: ck.gemv_fp16_transpose(2048, 64, 1024, k_.data_ptr(), sc.data_ptr(), ov.data_ptr(), st())) for k_ in kc], max(3, reps // 8))
        hbm("gemv_fp16_transpose (probabilities x value cache)", 2 * 2048 * 1024 * 64 + 2 * 2048 * 1024 + 2 * 2048 * 64, ms, how, "2048 x [1024,64] fp16", None)
        del kc
        # config 4 up-projection in the reference's native layout: bmm(W1[1,10240,4096], x[8,4096,512], int8)
        W1 = (torch.randn(1, 10240, 4096, generator=gg) * 0.02).half().to(dev)
        xa = torch.randn(8, 4096, 512, generator=gg).half().to(dev)
        ms = event_ms(lambda: ct.bmm(W1, False, xa, False, int8=True), 20)
        components["ffn up-projection bmm(int8), native layout"] = {
            "shape": "W1 [1,10240,4096] x act [8,4096,512]", "bound": "mfma", "avg_us": round(ms * 1e3, 2),
            "achieved": round(2.0 * 10240 * 4096 * 4096 / (ms * 1e-3) / 1e12, 1), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
            "frac": round(2.0 * 10240 * 4096 * 4096 / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4), "timing": "events, whole bmm"}
        del W1, xa
        # fp16 product of the north-star shape on the same tile kernel (fp32 accumulation)
        Ah = torch.randn(1, M, K, generator=gg).half().to(dev); Wh = (torch.randn(1, N, K, generator=gg) * 0.02).half().to(dev)
        oh = torch.empty((1, M, N), dtype=torch.half, device=dev)
        ms = event_ms(lambda: ck.gemm_fp16(N, K, M, 1, 1, True, False, Wh.data_ptr(), Ah.data_ptr(), oh.data_ptr(), st()), 20)
        components["gemm_fp16"] = {
            "shape": "M=%d K=%d N=%d fp16, fp32 accumulate" % (M, K, N), "bound": "mfma", "avg_us": round(ms * 1e3, 2),
            "achieved": round(2.0 * M * K * N / (ms * 1e-3) / 1e12, 1), "peak": 2500.0, "unit": "TFLOP/s",
            "frac": round(2.0 * M * K * N / (ms * 1e-3) / 1e12 / 2500.0, 4), "timing": "events"}
        del Ah, Wh, oh


    # ---- what the chip sustains: yardstick kernels and the vendor library on the same shapes ----------
    if only in ("", "ceilings"):
        import ctypes
        from cpm_kernels_amd.build import bench_library_path, build_bench_library
        if not os.path.exists(bench_library_path()):
            build_bench_library(verbose=False)
        cl = ctypes.CDLL(bench_library_path())
        VP, I32, I64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
        cl.ceil_mfma_i8.argtypes = [VP, I32, I32, I32, VP, VP]
        cl.ceil_mfma_i8_16x16x64.argtypes = [VP, I32, I32, I32, VP, VP]
        cl.ceil_read.argtypes = [VP, I64, VP, ctypes.c_int, VP]
        cl.ceil_read_span.argtypes = [VP, I32, VP, VP, VP]
        cl.ceil_empty.argtypes = [I32, I32, VP, VP]
        cl.ceil_xcc_ids.argtypes = [VP, I32, I32, VP]
        cl.ceil_read_gemv_pattern.argtypes = [VP, VP, ctypes.c_int, VP, VP, VP]
        cl.ceil_write.argtypes = [VP, I64, VP]
        cl.ceil_copy.argtypes = [VP, VP, I64, ctypes.c_int, VP]
        cl.ceil_copy_segments.argtypes = [VP, VP, I64, I32, I32, ctypes.c_int, VP]
        cl.ceil_copy_segments_persistent.argtypes = [VP, VP, I64, I32, I32, I32, VP, VP]

        def ok(rc):
            assert rc == 0, "yardstick launch failed: %d" % rc
        ceil = {"note": "kernels of cpm_kernels_amd/bench/ceilings.hip (not part of the library) and, for calibration only, "
                        "the vendor library through torch; same process, same device, HIP events on the launch stream"}
        gg = torch.Generator().manual_seed(11)
        sink = torch.zeros(64, dtype=torch.int32, device=dev)
        cus = props["compute_units"]
        iters = 2048
        for label, opnd in (("zero", torch.zeros(12 * 512 * 16, dtype=torch.int8)),
                            ("random", torch.randint(-127, 128, (12 * 512 * 16,), generator=gg, dtype=torch.int8))):
            od = opnd.to(dev)
            for waves, key in ((8, "mfma_i8_only_%s_operands" % label), (4, "mfma_i8_only_%s_operands_one_wave_per_simd" % label)):
                mfma_ops = float(cus) * waves * iters * 16 * 2 * 32 ** 3
                ms = event_ms(lambda: ok(cl.ceil_mfma_i8(od.data_ptr(), cus, waves, iters, sink.data_ptr(), st())), 10, warmup=3)
                ceil[key] = {"tops": round(mfma_ops / (ms * 1e-3) / 1e12, 1), "us": round(ms * 1e3, 1),
                             "frac_of_published_peak": round(mfma_ops / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)}
            # the same work per wave with the 16x16x64 form of the instruction (the one the 256x256 tile kernel uses)
            mfma_ops = float(cus) * 8 * iters * 32 * 2 * 16 * 16 * 64
            ms = event_ms(lambda: ok(cl.ceil_mfma_i8_16x16x64(od.data_ptr(), cus, 8, iters, sink.data_ptr(), st())), 10, warmup=3)
            ceil["mfma_i8_16x16x64_only_%s_operands" % label] = {"tops": round(mfma_ops / (ms * 1e-3) / 1e12, 1), "us": round(ms * 1e3, 1),
                                                                "frac_of_published_peak": round(mfma_ops / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)}
        # the library's K loop against that loop: one round of 256x256 tiles (4096 x 4096 outputs) at two depths of
        # K; the difference is 64 slabs of 128 bytes per compute unit and nothing else (no launch, prologue or epilogue)
        sweep = {"shape": "M=N=4096 int32 out, K=8192 and K=16384: (t2 - t1) / 64 = time of one 128-byte slab of a 256x256 tile per compute unit"}
        o32 = torch.empty((1, 4096, 4096), dtype=torch.int32, device=dev)
        for label in ("zero", "random"):
            ts = []
            for kk in (8192, 16384):
                if label == "zero":
                    qa = torch.zeros((1, 4096, kk), dtype=torch.int8, device=dev); qw = torch.zeros((1, 4096, kk), dtype=torch.int8, device=dev)
                else:
                    qa = torch.randint(-127, 128, (1, 4096, kk), generator=gg, dtype=torch.int8).to(dev)
                    qw = torch.randint(-127, 128, (1, 4096, kk), generator=gg, dtype=torch.int8).to(dev)
                ts.append(event_ms(lambda: ck.gemm_int8(4096, kk, 4096, 1, 1, True, False, qw.data_ptr(), qa.data_ptr(), o32.data_ptr(), st()), 20, warmup=5))
                del qa, qw
            slab_us = (ts[1] - ts[0]) * 1e3 / 64
            mfma_only_us = 256 * 256 * 128 * 2.0 * cus / (ceil["mfma_i8_16x16x64_only_%s_operands" % label]["tops"] * 1e12) * 1e6
            sweep["%s_operands" % label] = {"k8192_us": round(ts[0] * 1e3, 2), "k16384_us": round(ts[1] * 1e3, 2), "slab_us": round(slab_us, 4),
                                            "mfma_only_slab_us": round(mfma_only_us, 4), "k_loop_frac_of_mfma_only": round(mfma_only_us / slab_us, 4),
                                            "k16384_tops": round(2.0 * 4096 * 4096 * 16384 / (ts[1] * 1e-3) / 1e12, 1)}
        del o32
        ceil["gemm_k_loop (library kernel, K sweep)"] = sweep
        big = torch.randint(-128, 128, (1 << 30,), generator=None, dtype=torch.int8, device=dev)
        big2 = torch.empty_like(big)
        nb = big.numel()

        def gbs(nbytes, ms):
            return {"us": round(ms * 1e3, 2), "gbs": round(nbytes / (ms * 1e-3) / 1e9, 1), "frac_of_published_peak": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
        ceil["read_1GiB"] = gbs(nb, event_ms(lambda: ok(cl.ceil_read(big.data_ptr(), nb, sink.data_ptr(), 0, st())), 10))
        ceil["write_1GiB"] = gbs(nb, event_ms(lambda: ok(cl.ceil_write(big2.data_ptr(), nb, st())), 10))
        ceil["copy_1GiB"] = gbs(2 * nb, event_ms(lambda: ok(cl.ceil_copy(big.data_ptr(), big2.data_ptr(), nb, 0, st())), 10))
        ceil["copy_1GiB_nontemporal"] = gbs(2 * nb, event_ms(lambda: ok(cl.ceil_copy(big.data_ptr(), big2.data_ptr(), nb, 1, st())), 10))
        # calibration only, not this build's code: the runtime's own device-to-device copy (torch's copy_ of a contiguous
        # tensor is hipMemcpyAsync), 1 GiB and the layernorm's 33.5 MB from ten buffers in turn
        ceil["runtime_memcpy_d2d_1GiB"] = gbs(2 * nb, event_ms(lambda: big2.copy_(big), 10))
        ln_bytes = 8 * 4096 * 1024
        srcs = [big[i * (64 << 20): i * (64 << 20) + ln_bytes] for i in range(10)]
        dst_ln = big2[:ln_bytes]
        ms, how = graph_ms([(lambda i=i: dst_ln.copy_(srcs[i])) for i in range(10)], 60)
        ceil["runtime_memcpy_d2d_33.5MB"] = dict(gbs(2 * ln_bytes, ms), timing=how)
        del srcs, dst_ln
        # the premise of the team kernels' layout (a team = workgroups 8s + x of one launch for consecutive s): workgroup i
        # runs on XCD (i + k) % 8 with one k for the whole launch
        ids = torch.full((2048,), -1, dtype=torch.int32, device=dev)
        ok(cl.ceil_xcc_ids(ids.data_ptr(), 2048, 1024, st()))
        torch.cuda.synchronize()
        idl = ids.cpu().tolist()
        off = idl[0] % 8
        ceil["workgroup_to_xcd"] = {"xcds_seen": sorted(set(idl)), "first_workgroups": idl[:16], "k": off,
                                    "workgroup_i_runs_on_xcd_(i+k)_mod_8": all(x == (i + off) % 8 for i, x in enumerate(idl)),
                                    "launch": "2048 workgroups of 1024 threads, XCC_ID read by each"}
        # what one kernel launch costs between two others: a kernel that does nothing, in a graph like the per-kernel legs'
        ms, how = graph_ms([lambda: ok(cl.ceil_empty(256, 512, sink.data_ptr(), st()))], 640)
        ceil["empty_kernel (what a launch costs in the per-kernel legs)"] = {"us": round(ms * 1e3, 2), "timing": how}
        # the GEMV's traffic: a cold 42 MB read, eight different 42 MB pieces of the buffer in turn (336 MB > Infinity Cache)
        piece = 10240 * 4096
        for nt_ in (0, 1):
            ms, how = graph_ms([(lambda i=i: ok(cl.ceil_read(big.data_ptr() + i * (128 << 20), piece, sink.data_ptr(), nt_, st()))) for i in range(8)], 80)
            ceil["cold_read_42MB%s (gemv traffic)" % ("_nontemporal" if nt_ else "")] = dict(gbs(piece, ms), timing=how)
        # the same bytes as one contiguous share per compute unit, every load requested at once (the one-round kernels' shape),
        # timed inside the kernel: last workgroup's end - first workgroup's start, on the device's 100 MHz wall clock
        stamps = torch.zeros(8, 512, dtype=torch.int64, device=dev)
        for _ in range(3):
            for i in range(8):
                ok(cl.ceil_read_span(big.data_ptr() + i * (128 << 20), 256, sink.data_ptr(), stamps[i].data_ptr(), st()))
        torch.cuda.synchronize()
        sp = stamps.cpu().view(8, 256, 2)
        span_us = float(((sp[:, :, 1].max(dim=1).values - sp[:, :, 0].min(dim=1).values).double().mean()) * 0.01)
        ms, how = graph_ms([(lambda i=i: ok(cl.ceil_read_span(big.data_ptr() + i * (128 << 20), 256, sink.data_ptr(), stamps[i].data_ptr(), st()))) for i in range(8)], 80)
        ceil["cold_read_42MB_one_share_per_compute_unit"] = dict(gbs(piece, ms), timing=how, in_kernel_span_us=round(span_us, 2),
                                                               in_kernel_span_frac_of_published_peak=round(piece / (span_us * 1e-6) / 1e9 / PEAK_HBM_GBS, 4),
                                                               note="span = last workgroup's end - first workgroup's start (wall clock stamps inside the kernel); the rest of "
                                                                    "the per-launch time is what a launch costs (see empty_kernel)")
        # what loading a decode GEMV's matrix straight in the MFMA operand layout would cost (an instruction touches 64 bytes of
        # 16 rows; the library's kernel reads 4 rows x 256 bytes per instruction instead and transposes in LDS), alone and with the
        # 128 KB of vectors that every workgroup reads alike; span and per-launch time as above
        vecs = big2[:128 << 10]
        for label, vp_, nt_ in (("matrix_only_nontemporal", None, 1), ("matrix_only_plain_loads", None, 0), ("with_the_vectors_nontemporal", vecs.data_ptr(), 1),
                                ("with_the_vectors_plain_loads", vecs.data_ptr(), 0)):
            for _ in range(3):
                for i in range(8):
                    ok(cl.ceil_read_gemv_pattern(big.data_ptr() + i * (128 << 20), vp_, nt_, sink.data_ptr(), stamps[i].data_ptr(), st()))
            torch.cuda.synchronize()
            sp = stamps.cpu().view(8, 256, 2)
            span_us = float(((sp[:, :, 1].max(dim=1).values - sp[:, :, 0].min(dim=1).values).double().mean()) * 0.01)
            ms, how = graph_ms([(lambda i=i: ok(cl.ceil_read_gemv_pattern(big.data_ptr() + i * (128 << 20), vp_, nt_, sink.data_ptr(), stamps[i].data_ptr(), st())))
                                for i in range(8)], 80)
            ceil["cold_read_42MB_gemv_access_pattern_" + label] = dict(gbs(piece, ms), timing=how, in_kernel_span_us=round(span_us, 2))
        del vecs
        # the layernorm's traffic and pattern: [8*4096 rows, 1024 bytes] in 128-byte (and wider) column segments, ten buffers in turn
        for seg, nt_ in ((128, 0), (128, 1), (256, 1), (1024, 1)):
            ms, how = graph_ms([(lambda i=i: ok(cl.ceil_copy_segments(big.data_ptr() + i * (64 << 20), big2.data_ptr(), 8 * 4096, 1024, seg, nt_, st())))
                                for i in range(10)], 60)
            ceil["tiled_copy_33.5MB_rows_of_1KB_seg%d%s (layernorm traffic)" % (seg, "_nontemporal" if nt_ else "")] = dict(gbs(2 * 8 * 4096 * 1024, ms), timing=how)
        # the softmax's: [512*1024 rows, 2048 bytes], tiles of 1024 x 128 bytes as the kernel holds them, and wider segments
        for seg, nt_ in ((128, 0), (128, 1), (256, 1), (1024, 1)):
            ms = event_ms(lambda: ok(cl.ceil_copy_segments(big.data_ptr(), big2.data_ptr(), 512 * 1024, 2048, seg, nt_, st())), 5)
            ceil["tiled_copy_1GiB_rows_of_2KB_seg%d%s (softmax traffic)" % (seg, "_nontemporal" if nt_ else "")] = gbs(2 * nb, ms)
        # the same tiles through persistent workgroups with the next tile in flight and tiles from a counter (the softmax kernel's structure)
        sched = torch.zeros(2, dtype=torch.int32, device=dev)
        for seg in (128, 256, 512):
            ms = event_ms(lambda: ok(cl.ceil_copy_segments_persistent(big.data_ptr(), big2.data_ptr(), 512 * 1024, 2048, seg, cus, sched.data_ptr(), st())), 5)
            ceil["persistent_tiled_copy_1GiB_rows_of_2KB_seg%d_nontemporal (softmax traffic and structure)" % seg] = gbs(2 * nb, ms)
        del big, big2
        # vendor library, calibration only: torch._int_mm (hipBLASLt) on the north-star and config-1 operands, int32 out
        try:
            qa = torch.randint(-127, 128, (M, K), generator=gg, dtype=torch.int8).to(dev)
            qw = torch.randint(-127, 128, (N, K), generator=gg, dtype=torch.int8).to(dev)
            ms = event_ms(lambda: torch._int_mm(qa, qw.t()), 20, warmup=5)
            ceil["vendor_int_mm_north_star_int32_out"] = {"us": round(ms * 1e3, 1), "tops": round(ops / (ms * 1e-3) / 1e12, 1)}
            o32 = torch.empty((1, M, N), dtype=torch.int32, device=dev)
            ms = event_ms(lambda: ck.gemm_int8(N, K, M, 1, 1, True, False, qw.data_ptr(), qa.data_ptr(), o32.data_ptr(), st()), 20, warmup=5)
            ceil["this_library_gemm_int8_same_operands"] = {"us": round(ms * 1e3, 1), "tops": round(ops / (ms * 1e-3) / 1e12, 1)}
            qa1, qw1 = qa[:512].contiguous(), qw[:4096].contiguous()
            ms = event_ms(lambda: torch._int_mm(qa1, qw1.t()), 50, warmup=5)
            ceil["vendor_int_mm_config_1_int32_out"] = {"us": round(ms * 1e3, 2), "tops": round(2.0 * 512 * 4096 * 4096 / (ms * 1e-3) / 1e12, 1)}
            del qa, qw, o32
            # the GEMV's shape through the vendor's GEMM: 32 vectors x [10240, 4096], eight weight copies in turn (cold), eager launches
            ws = [torch.randint(-127, 128, (10240, 4096), generator=gg, dtype=torch.int8).to(dev) for _ in range(8)]
            v32 = torch.randint(-127, 128, (32, 4096), generator=gg, dtype=torch.int8).to(dev)
            turn = [0]

            def vendor_gemv():
                turn[0] = (turn[0] + 1) % 8
                torch._int_mm(v32, ws[turn[0]].t())
            ms = event_ms(vendor_gemv, 400, warmup=16)
            ceil["vendor_int_mm_gemv_shape_int32_out"] = dict(gbs(10240 * 4096 + 32 * 4096 + 4 * 32 * 10240, ms), timing="events, eager launches")
            del ws, v32
        except Exception as ex:     # pragma: no cover  (calibration only)
            ceil["vendor_int_mm"] = "unavailable: %s" % ex
        # torch's own softmax over dim 1 on config 3's tensor (the same operation, without the -1e6 floor and the 1e-10)
        try:
            xs = torch.randn((512, 1024, 1024), generator=gg, dtype=torch.float16).to(dev)
            ys = torch.empty_like(xs)
            ms = event_ms(lambda: torch.softmax(xs, dim=1, out=ys), 10, warmup=3)
            ceil["torch_softmax_dim1_config_3"] = gbs(2 * xs.numel() * 2, ms)
            del xs, ys
        except Exception as ex:     # pragma: no cover  (calibration only)
            ceil["torch_softmax_dim1_config_3"] = "unavailable: %s" % ex
        result["ceilings"] = ceil

    # ---- the north-star step and its GEMM kernel on the busy device (see the note at leg_pipeline's first call) ----
    if only == "":
        roofline = leg_gemm()
        step_ms, wall_ms = leg_pipeline()
        result["wall_ms_per_step"] = round(wall_ms, 4)
        result["value_protocol"] = ("W warm-up steps, then exactly K timed steps between synchronisations, run right after the roofline loop of "
                                    "this process, i.e. with the device at the clock a sustained load runs at; `from_idle` is the same W + K run "
                                    "first thing in the process, while the clock is still rising (it takes ~30 ms of load)")

    # per-op CPU timings beside the components: the torch formulations the reference's tests compare
    # with (oracle/formulations.py), on all host cores, full shapes (fewer repetitions for the big ones)
    if not args.no_cpu and only == "":
        from oracle import formulations as F
        torch.set_num_threads(os.cpu_count() or 1)

        def cpu_us(fn, n=5, warm=True):
            if warm:
                fn()
            ts = []
            for _ in range(n):
                t0 = time.perf_counter(); fn(); ts.append(time.perf_counter() - t0)
            return round(sorted(ts)[len(ts) // 2] * 1e6, 1)

        def put(name, us, sample):
            if name in components:
                components[name]["cpu_us"] = us
                components[name]["cpu_sample"] = sample
                components[name]["cpu_cores"] = torch.get_num_threads()
        gg = torch.Generator().manual_seed(1002)
        Wq = torch.randint(-127, 128, (10240, 4096), generator=gg, dtype=torch.int8)
        sm_ = (torch.rand(10240, generator=gg) * 0.009 + 0.001).half()
        vv = torch.randn(32, 4096, generator=gg).half()
        Wdeq = (Wq.float() * sm_.float()[:, None]).half()[None]          # the dequantised weight the formulation starts from
        put("gemv_broadcast_mat_int8", cpu_us(lambda: F.quant_bmm_rowwise(vv[None], Wdeq)),
            "fp32 fake-quant of 32 vectors and of the dequantised [10240,4096] weight + fp32 matmul, median of 5")
        del Wq, Wdeq
        gg = torch.Generator().manual_seed(1003)
        xl = torch.randn(8, 4096, 512, generator=gg).half()
        wl = (1 + 0.1 * torch.randn(4096, generator=gg)).half(); bl = (0.1 * torch.randn(4096, generator=gg)).half()
        put("layernorm_forward", cpu_us(lambda: F.layernorm_dim1(xl, wl, bl, 1e-5)), "full [8,4096,512], fp32 formulation with gamma/beta, median of 5")
        del xl
        if "softmax_forward" in components:
            xsm = (torch.randn(64, 1024, 1024, generator=gg) * 4).half()
            kk = torch.arange(1024)[:, None]; qq = torch.arange(1024)[None, :]
            xsm.masked_fill_((kk > qq)[None], float("-inf"))
            xsm = xsm.repeat(8, 1, 1)
            put("softmax_forward", cpu_us(lambda: F.softmax_dim1(xsm), n=1, warm=False), "full [512,1024,1024] causal, torch.softmax on an fp32 copy, one run")
            del xsm
        gg = torch.Generator().manual_seed(1004)
        xg = torch.randn(8, 10240 * 512, generator=gg).half()
        put("gelu_forward", cpu_us(lambda: F.gelu_tanh(xg), n=3), "full [8, 10240*512], tanh form in fp32, median of 3")
        del xg
        pw_ = (torch.randn(64, 32, generator=gg) * 0.02).half()
        put("position_embedding_forward", cpu_us(lambda: F.position_bias(pw_, 1024, 1024, True, 32, 128), n=3),
            "64 heads x 1024 x 1024: T5 bucket formula + gather, median of 3")

    # ---- CPU baseline: torch formulation of the same step on the host cores ------------------
    cpu = None
    if not args.no_cpu and only == "":
        from oracle.formulations import quant_bmm_rowwise
        ncores = os.cpu_count() or 1
        torch.set_num_threads(ncores)
        quant_bmm_rowwise(A_cpu[:, :256], W_cpu[:, :256])      # warm the thread pool
        times = []
        t_begin = time.perf_counter()
        while len(times) < 3 and time.perf_counter() - t_begin < 25.0:
            t0 = time.perf_counter()
            quant_bmm_rowwise(A_cpu, W_cpu)
            times.append(time.perf_counter() - t0)
        best = sorted(times)[len(times) // 2]
        cpu = {"value": round(ops / best / 1e12, 4), "unit": "TOP/s", "cores": torch.get_num_threads(),
               "kind": "port", "seconds_per_step": round(best, 3),
               "sample": "full north-star step (fp32 fake-quant of A and W + fp32 matmul), median of %d runs" % len(times)}

    # The HBM half of the metric inside `roofline`, so that the one object carries all four headline kernels:
    # kernel, average launch time, algorithmic bytes, achieved rate, fraction of the published HBM peak, and
    # the HBM bytes the counters saw per launch (profiles/hbm_traffic_counters.txt).
    hbm_block = {}
    for name, kernel in (("gemv_broadcast_mat_int8", "k_gemv_coalesced<8,3,2>"), ("layernorm_forward", "k_layernorm_team<1024,8,false>"),
                         ("softmax_forward", "k_softmax_stream<1024,8,8>")):
        c = components.get(name)
        if c is not None:
            hbm_block[name] = {"kernel": kernel, "shape": c["shape"], "avg_us": c["avg_us"], "algorithmic_bytes": c["algorithmic_bytes"],
                               "achieved": c["achieved"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": c["frac"], "traffic": c["traffic"],
                               "timing": c["timing"]}
    if hbm_block:
        if roofline is None:
            roofline = {}
        roofline["hbm"] = hbm_block
        roofline["hbm_note"] = ("the metric's HBM-bound kernels: frac = algorithmic_bytes / avg_us / 8 TB/s; inputs rotate through buffers larger "
                                "than the 256 MB Infinity Cache; traffic = HBM bytes per launch from " + OFFLINE_SOURCE["traffic"])

    value = ops / (step_ms * 1e-3) / 1e12 if step_ms else None
    line = {
        "metric": "int8 quant-GEMM TOPS + GEMV/LN/softmax HBM GB/s (frac of peak) at 1 GPU",
        "value": round(value, 2) if value else None, "unit": "TOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_ms, 4) if step_ms else None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 (int32 accumulate, fp16 in/out)", "data": "synthetic",
        "config": {"workload": "north-star int8 quant-GEMM M=4096 K=4096 N=10240: bmm(A[1,4096,4096] fp16, "
                               "W[1,10240,4096] fp16, int8=True) = quantise A and W, int8 MFMA GEMM, fp16 dequant",
                   "seed": 1000},
        "value_cold": result.get("from_idle", {}).get("value"), "ms_per_step_cold": result.get("from_idle", {}).get("ms_per_step"),
        "roofline": roofline, "cpu_baseline": cpu, "components": components,
        "device": torch.cuda.get_device_name(0),
    }
    line.update(result)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
