"""Benchmark of the one-bit 2:4 sparse GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload square:8192]

A step is one product D = A*B (prepared weight, fp16 B resident in HBM, fp32 accumulate, fp16 D). The default
workload is the square 8192^3 problem the headline metric is quoted on; the dense-equivalent FLOP count is
2*M*N*K (the reference's own convention, tests/kernel_test.cu:207-215). The JSON line also carries the
roofline figures of the dominant kernel, the HBM figure of the N=16 decode shape and the CPU baseline.
Other workloads: square:<size>, decode:<m>x<k>x<n>, prefill (4096x2048x4096, alpha=0.5, beta=1).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

CU_COUNT = 256
CLOCK_HZ = 2.4e9
DENSE_F16_PEAK_TFLOPS = CU_COUNT * CLOCK_HZ * 4096 / 1e12        # 2516.6: published dense fp16 MFMA peak
SMFMAC_PEAK_TFLOPS = 2 * DENSE_F16_PEAK_TFLOPS                   # dense-equivalent rate of v_smfmac f16
HBM_PEAK_GBS = 8000.0
# HBM-side bytes per launch of the dominant kernel, from two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE), each
# scaled by what the same counter reads for an elementwise copy kernel over 256 MiB (x2.000 and x1.000): see
# profiles/hbm_traffic_counters.txt. Only the workloads it was measured on have a figure.
MEASURED_TRAFFIC_BYTES = {"square:8192": (229619.5 * 2.000 + 131072.0 * 1.000) * 1024,
                          "prefill": (30840.0 * 2.000 + 16384.0 * 1.000) * 1024,
                          "decode:11008x4096x16": (4709.0 * 2.000 + 344.0 * 1.000) * 1024}


def parse_workload(text):
    if text.startswith("square:"):
        s = int(text.split(":")[1])
        return dict(name=text, m=s, n=s, k=s, alpha=1.0, beta=0.0)
    if text.startswith("decode:"):
        m, k, n = (int(v) for v in text.split(":")[1].split("x"))
        return dict(name=text, m=m, n=n, k=k, alpha=1.0, beta=0.0)
    if text == "prefill":
        return dict(name=text, m=4096, n=2048, k=4096, alpha=0.5, beta=1.0)
    raise SystemExit(f"unknown workload {text!r}")


def algorithmic_bytes(m, n, k, beta):
    # a bits + metadata (= prepared operand, 1.5 bit per weight) + B + D (+ C), each counted once
    return m * k // 16 + m * k // 8 + 2 * k * n + 2 * m * n + (2 * m * n if beta != 0.0 else 0)


def time_launches(fn, steps, warmup):
    """Average duration of one launch: HIP events on the stream the kernels run on (torch's current stream)."""
    import torch
    for _ in range(warmup):
        fn(0)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return start.elapsed_time(stop) / steps * 1e-3, wall / steps


def time_graph(fn, launches, warmup=20, preload_ms=0.0):
    """Average duration of one launch inside a HIP graph of `launches` back-to-back kernel nodes (no host
    launch overhead between them). The graph is replayed once untimed (or, with preload_ms, again and again for at least
    that long, so that the timed replay runs at the clock of a GPU under continuous load) and once timed."""
    import torch
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    # The operands of fn were produced, and blocks of the caching allocator freed, by work queued on the current
    # stream: without this wait the warm-up launches below run concurrently with that work, read operands that are not
    # written yet and write their output into memory that a still-pending kernel of the current stream may own
    # (a freed temporary the allocator handed out again).
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        # warm up on the capture stream: the library keeps its K-split and padded-B buffers per stream and may only
        # allocate them outside a capture
        for i in range(warmup):
            fn(i)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for i in range(launches):
                fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    graph.replay()
    torch.cuda.synchronize()
    # batches of replays that queue up behind one another (no idle gap inside a batch), each batch about 2 ms of GPU time
    per_batch = max(1, int(2e-3 / max(time.perf_counter() - t0, 1e-5)))
    while (time.perf_counter() - t0) * 1e3 < preload_ms:
        for _ in range(per_batch):
            graph.replay()
        torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    graph.replay()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / launches * 1e-3


def make_gemm(w):
    import torch
    from onebitsparsemul_amd import _native, synthetic
    m, n, k = w["m"], w["n"], w["k"]
    a, meta = synthetic.make_weight(m, k, seed=0x0B5A0000, device="cuda")
    b = synthetic.make_b(k, n, seed=1, kind="normal", device="cuda")
    c = synthetic.make_c(m, n, seed=2, device="cuda") if w["beta"] != 0.0 else None
    prep = _native.prepare(a, meta, m, k)
    d = torch.empty((m, n), dtype=torch.float16, device="cuda")
    fn = lambda i: _native.matmul_prepared(prep, b, d, m, n, k, c=c, alpha=w["alpha"], beta=w["beta"])
    return (a, meta, b, d), fn


def run_decode_rotating(m, k, n, launches=2000, copies=None):
    """HBM-bound decode shape: rotate over enough distinct prepared weights (> 256 MiB in total, more than the
    last-level cache) that every launch streams its weight from HBM; also time the same-buffer case. The
    launches are recorded into a HIP graph so that the figure is kernel time, not host launch overhead."""
    import torch
    from onebitsparsemul_amd import _native, synthetic
    a, meta = synthetic.make_weight(m, k, seed=3, device="cuda")
    prep0 = _native.prepare(a, meta, m, k)
    if copies is None:
        copies = max(64, (768 << 20) // prep0.numel() + 1)
    preps = [prep0] + [prep0.clone() for _ in range(copies - 1)]
    b = synthetic.make_b(k, n, seed=4, kind="normal", device="cuda")
    d = torch.empty((m, n), dtype=torch.float16, device="cuda")
    rot = lambda i: _native.matmul_prepared(preps[i % copies], b, d, m, n, k)
    same = lambda i: _native.matmul_prepared(prep0, b, d, m, n, k)
    t_rot = time_graph(rot, launches)
    t_same = time_graph(same, launches)
    nbytes = algorithmic_bytes(m, n, k, 0.0)
    return dict(shape=f"{m}x{k}x{n}", bytes=nbytes, copies=copies, launches=launches,
                us_per_launch_hbm=t_rot * 1e6, gbps_hbm=nbytes / t_rot / 1e9,
                us_per_launch_cache_resident=t_same * 1e6, gbps_cache_resident=nbytes / t_same / 1e9,
                frac_of_hbm_peak=nbytes / t_rot / 1e9 / HBM_PEAK_GBS)


def run_decode_grouped(m, k, tokens, group=8, launches=400):
    """The grouped entry point on decode-sized products: `group` distinct weights of m x k per launch (one launch of the
    split-K kernel for all of them), rotating over enough sets that every launch streams its weights from HBM; next to
    the single-launch figure, never instead of it. Token-major x and y as the layer holds them."""
    import torch
    from onebitsparsemul_amd import _native, synthetic
    a, meta = synthetic.make_weight(m, k, seed=3, device="cuda")
    prep0 = _native.prepare(a, meta, m, k)
    sets = max(4, (768 << 20) // (prep0.numel() * group) + 1)
    x = synthetic.make_b(tokens, k, seed=4, kind="normal", device="cuda")
    problems = []
    for s_ in range(sets):
        problems.append([(prep0 if s_ + g == 0 else prep0.clone(), x, torch.empty((tokens, m), dtype=torch.float16, device="cuda"),
                          m, k, None) for g in range(group)])
    t = time_graph(lambda i: _native.linear_prepared_grouped(problems[i % sets]), launches)
    nbytes = algorithmic_bytes(m, tokens, k, 0.0)
    return dict(shape=f"{group} x ({m}x{k}, {tokens} tokens) per launch", bytes_per_problem=nbytes, sets=sets, launches=launches,
                us_per_launch=t * 1e6, us_per_problem=t * 1e6 / group, gbps_hbm=nbytes * group / t / 1e9,
                frac_of_hbm_peak=nbytes * group / t / 1e9 / HBM_PEAK_GBS)


def run_layer_form(m, k, tokens, launches=1000):
    """The linear layer's call y = x W^T + bias (x and y token-major) three ways, each inside a HIP graph: the
    token-major kernel form, the plain kernel on operands that are already transposed (no bias), and the plain kernel
    with the two transposes and the bias pass around it. The weight is the same every launch (cache-resident)."""
    import torch
    from onebitsparsemul_amd import _native, synthetic
    a, meta = synthetic.make_weight(m, k, seed=5, device="cuda")
    prep = _native.prepare(a, meta, m, k)
    x = synthetic.make_b(tokens, k, seed=6, kind="normal", device="cuda")
    bias = synthetic.make_b(1, m, seed=7, kind="normal", device="cuda").reshape(m)
    b = x.T.contiguous()
    d = torch.empty((m, tokens), dtype=torch.float16, device="cuda")
    y = torch.empty((tokens, m), dtype=torch.float16, device="cuda")

    def around(i):
        _native.matmul_prepared(prep, x.T.contiguous(), d, m, tokens, k)
        return d.T.contiguous() + bias

    t_form = time_graph(lambda i: _native.linear_prepared(prep, x, y, m, k, bias=bias), launches)
    t_plain = time_graph(lambda i: _native.matmul_prepared(prep, b, d, m, tokens, k), launches)
    t_around = time_graph(around, max(50, launches // 4))
    return dict(shape=f"{m}x{k}, {tokens} tokens", us_token_major_form=t_form * 1e6,
                us_plain_kernel_pretransposed=t_plain * 1e6, us_plain_kernel_with_transposes_and_bias=t_around * 1e6)


def cpu_baseline(w, operands, budget_s=12.0, unit="TFLOP/s"):
    """oracle (kind 'port'): decompress + dense fp32 torch.matmul on the host cores, on a row slab sized for
    about budget_s seconds; rate in the workload's unit (dense-equivalent TFLOP/s, or algorithmic GB/s for the
    HBM-bound decode shapes). When the slab is not the whole problem the rate is that of the slab (the rows are
    independent, so it extrapolates linearly) and `extrapolated` says so."""
    import torch
    import oracle
    a, meta, b, d = operands
    m, n, k = w["m"], w["n"], w["k"]
    a_h, e_h, b_h = a.cpu().numpy(), meta.cpu().numpy(), b.cpu().numpy()
    probe_rows = min(m, 256)
    t_probe, _, _ = oracle.cpu_baseline_gemm(a_h, b_h, e_h, m, n, k, 0, probe_rows)
    rate = 2.0 * probe_rows * n * k / max(t_probe, 1e-9)
    rows = int(min(m, max(probe_rows, (budget_s * rate / (2.0 * n * k)) // 64 * 64)))
    # when the whole problem takes less than the budget, repeat it so that about budget_s of CPU work is timed
    once = 2.0 * rows * n * k / rate
    repeats = int(max(1, min(20, budget_s / max(once, 1e-3))))
    t_mm, t_dec, out = oracle.cpu_baseline_gemm(a_h, b_h, e_h, m, n, k, 0, rows, repeats=repeats)
    # the slab doubles as a parity spot check of the timed GPU result
    got = d[:rows].float().cpu().numpy()
    scale = float(abs(out).max())
    rel = float(abs(got - w["alpha"] * out).max() / scale) if w["beta"] == 0.0 else None
    if unit == "GB/s":
        value = algorithmic_bytes(rows, n, k, w["beta"]) / t_mm / 1e9
    else:
        value = 2.0 * rows * n * k / t_mm / 1e12
    return dict(value=value, unit=unit, cores=torch.get_num_threads(), kind="port",
                sample=f"rows 0..{rows} of {m} (all of K={k}, N={n}): decompress {t_dec:.2f}s once + fp32 torch.matmul "
                       f"{t_mm:.4f}s each, {repeats} repetitions",
                extrapolated=rows < m, gpu_vs_oracle_rel_err_on_sample=rel)


def sustained_rate(fn, flops, load_ms=150.0, launches=60):
    """The same launch after at least load_ms of continuous load, timed inside a HIP graph: the rate a long-running job
    sees. The load is the graph itself replayed back to back, so it is continuous for launches of any length."""
    t0 = time.perf_counter()
    t = time_graph(fn, launches, warmup=10, preload_ms=load_ms)
    return dict(ms_per_step=t * 1e3, tflops=flops / t / 1e12, frac=flops / t / 1e12 / SMFMAC_PEAK_TFLOPS,
                preceding_load_ms=(time.perf_counter() - t0) * 1e3, graph_launches=launches,
                note="HIP-graph timing of the same kernel after >= 150 ms of replays of that graph, back to back with no "
                     "host gap (sustained clock)")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # The GPU raises its clock over the first ~50 ms of sustained load (8192^3: 1.77 PF in the first 20 launches,
    # 2.05-2.06 PF from the 80th on), so the default warm-up is long enough to time the sustained rate.
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="square:8192")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-ceiling", action="store_true")
    ap.add_argument("--no-sustained", action="store_true")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one elementwise copy kernel over 256 MiB (reference point for HBM counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")
    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    torch.cuda.set_device(0)
    w = parse_workload(args.workload)
    m, n, k = w["m"], w["n"], w["k"]

    if w["name"].startswith("decode:"):
        dec = run_decode_rotating(m, k, n, launches=max(args.steps, 200))
        line = dict(metric="hbm_gbps_decode", value=dec["gbps_hbm"], unit="GB/s", n_gpus=1, steps=dec["launches"],
                    warmup=20, ms_per_step=dec["us_per_launch_hbm"] * 1e-3, higher_is_better=True, scaling="weak",
                    vs_baseline=None, dtype="f16", data="synthetic", config=dict(workload=w["name"], m=m, n=n, k=k),
                    roofline=dict(bound="hbm", achieved=dec["gbps_hbm"], peak=HBM_PEAK_GBS, unit="GB/s",
                                  frac=dec["frac_of_hbm_peak"], traffic=MEASURED_TRAFFIC_BYTES.get(w["name"])),
                    decode=dec)
        if not args.no_cpu_baseline:
            from onebitsparsemul_amd import _native, synthetic
            a, meta = synthetic.make_weight(m, k, seed=3, device="cuda")
            b = synthetic.make_b(k, n, seed=4, kind="normal", device="cuda")
            d = torch.empty((m, n), dtype=torch.float16, device="cuda")
            _native.matmul_prepared(_native.prepare(a, meta, m, k), b, d, m, n, k)
            torch.cuda.synchronize()
            line["cpu_baseline"] = cpu_baseline(w, (a, meta, b, d), unit="GB/s")
        print(json.dumps(line))
        return

    if args.calibration_copy:
        # a plain elementwise kernel of known size: reads 256 MiB, writes 256 MiB (grid 128 Mi elements / 1024 per block)
        src = torch.randn(128 << 20, dtype=torch.float16, device="cuda")
        dst = torch.empty_like(src)
        torch.neg(src, out=dst)
        torch.cuda.synchronize()
        del src, dst
    operands, fn = make_gemm(w)
    flops = 2.0 * m * n * k
    # Order of the legs. After idle the GPU's power management overshoots: it starts at full clock, throttles below the
    # sustained point within ~3 ms and recovers over the next ~25 ms (8192^3: launches 4-60 after idle run up to 25 %
    # slower than launch 2 and than every launch from the 60th on). A window of 5 warm-ups + 20 launches taken right
    # after idle lies inside that dip and measures the transient, not the kernel. So the sustained leg (>= 150 ms of
    # back-to-back launches, then a HIP-graph timing) runs first and the W warm-ups + K timed launches of the command
    # line follow it without a pause: `value` is the steady-state rate. `after_idle` repeats exactly the same W + K
    # sequence after 3 s of idle, i.e. what `value` would be without the preceding load.
    sustained = None if args.no_sustained else sustained_rate(fn, flops)
    kernel_s, wall_s = time_launches(fn, args.steps, args.warmup)
    # launches shorter than the host's launch interval: also time them inside a HIP graph
    graph_s = time_graph(fn, max(args.steps, 200)) if flops < 2e11 else None
    tflops = flops / kernel_s / 1e12
    line = dict(
        metric="dense_equiv_tflops", value=tflops, unit="TFLOP/s", n_gpus=1, steps=args.steps, warmup=args.warmup,
        ms_per_step=kernel_s * 1e3, higher_is_better=True, scaling="weak", vs_baseline=None, dtype="f16",
        data="synthetic",
        config=dict(workload=w["name"], m=m, n=n, k=k, alpha=w["alpha"], beta=w["beta"], a="1-bit 2:4 prepared",
                    b="fp16 N(0,1)", accumulate="fp32", d="fp16"),
        roofline=dict(bound="mfma", achieved=tflops, peak=SMFMAC_PEAK_TFLOPS, unit="TFLOP/s",
                      frac=tflops / SMFMAC_PEAK_TFLOPS, traffic=MEASURED_TRAFFIC_BYTES.get(w["name"]),
                      note="dense-equivalent FLOPs 2MNK against the fp16 SMFMAC rate (2 x the dense fp16 MFMA peak "
                           f"{DENSE_F16_PEAK_TFLOPS:.1f}); the same fraction as executed FLOPs MNK against the dense peak",
                      hbm_gbps_algorithmic=algorithmic_bytes(m, n, k, w["beta"]) / kernel_s / 1e9),
        wall_ms_per_step=wall_s * 1e3,
        timing="W warm-ups and K timed launches (HIP events on the launch stream) directly after the sustained leg: "
               "steady-state clock" if sustained else "W warm-ups and K timed launches from idle")
    if sustained:
        line["sustained"] = sustained
        time.sleep(3.0)
        idle_s, _ = time_launches(fn, args.steps, args.warmup)
        line["after_idle"] = dict(ms_per_step=idle_s * 1e3, tflops=flops / idle_s / 1e12,
                                  frac=flops / idle_s / 1e12 / SMFMAC_PEAK_TFLOPS,
                                  note="the same W warm-ups + K timed launches after 3 s of idle: the window then lies in "
                                       "the power management's dip that follows the first launches after idle")
    if graph_s is not None:
        line["graph_ms_per_step"] = graph_s * 1e3  # the same launch inside a HIP graph: no host launch interval
        line["graph_tflops"] = flops / graph_s / 1e12
    from onebitsparsemul_amd import _native
    cus, khz = _native.device_info()
    line["device"] = dict(name=torch.cuda.get_device_name(0), compute_units=cus, clock_mhz=khz / 1e3,
                          smfmac_peak_from_device_tflops=2 * cus * khz * 1e3 * 4096 / 1e12,
                          note="peak = CUs x clock x 4096 dense fp16 FLOP/clk/CU x 2 (sparse); roofline.peak uses the "
                               "published 256 CUs x 2.4 GHz")
    if not args.no_ceiling:
        # register-only SMFMAC loops: what the chip sustains under matrix load, which depends on the operand values and
        # on the instruction (m32: v_smfmac_f32_32x32x32_f16, the eight-wavefront tiles; m16: v_smfmac_f32_16x16x64_f16,
        # the default large tile)
        rate = _native.measure_smfmac_rate
        loops = dict(
            m32_benchmark_distribution=max(rate(True, 50000, _native.SMFMAC_32X32X32) for _ in range(4)),
            m32_constant_operands=max(rate(False, 50000, _native.SMFMAC_32X32X32) for _ in range(4)),
            m16_benchmark_distribution=max(rate(True, 100000, _native.SMFMAC_16X16X64) for _ in range(4)),
            m16_constant_operands=max(rate(False, 100000, _native.SMFMAC_16X16X64) for _ in range(4)),
            note="no LDS or global memory in the loop; the gap to the nominal peak is clock throttling under load")
        line["smfmac_register_loop_tflops"] = loops
        tile = _native.describe_launch(m, n, k, compute_units=None).get("tile")
        ceiling = loops["m16_benchmark_distribution"] if tile == 15 else loops["m32_benchmark_distribution"]
        line["roofline"]["frac_of_register_loop"] = tflops / ceiling
        line["roofline"]["register_loop"] = "m16_benchmark_distribution" if tile == 15 else "m32_benchmark_distribution"
    if not args.no_decode:
        line["decode_n16"] = run_decode_rotating(11008, 4096, 16)
        # the same kernel family where the weight is large enough for bandwidth, not latency, to set the time
        line["decode_n16_large"] = run_decode_rotating(28672, 8192, 16, launches=500)
        # several decode-sized products in one launch (the grouped entry point): 8 distinct weights per launch
        line["decode_n16_grouped"] = run_decode_grouped(11008, 4096, 16)
        # the linear layer's token-major form of the same kernels (decode and prefill sized)
        # (8192 tokens on an 8192 x 8192 weight: the token-major form of the 16x16x64 tile the headline figure runs on)
        line["layer_form"] = [run_layer_form(11008, 4096, 16), run_layer_form(4096, 4096, 2048, launches=200),
                              run_layer_form(8192, 8192, 8192, launches=40)]
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(w, operands)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
