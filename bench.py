#!/usr/bin/env python3
"""Benchmark of the block-wise FP8 linear path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--table]

One "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM: act_quant(X) followed by fp8_gemm(Xq, Xs, Wq, Ws) -> bf16,
i.e. the FP8 linear forward with a pre-quantized weight.  The default workload is
the headline shape of the benchmark definition: DeepSeek-V3 dense MLP up/gate,
X[4096, 7168] bf16 ~ N(0,1), W[18432, 7168] e4m3fn with 128x128 fp32 block scales.

Prints ONE JSON line on stdout:
  value        whole-step throughput in TFLOP/s (2*M*N*K / step time, quantizer included)
  roofline     the dominant kernel (fp8_gemm): algorithmic FLOPs per call / its average
               duration, measured with HIP events on the launch stream inside the timed
               region, against the dense FP8 MFMA peak (a call is fp8_gemm() as a user
               makes it: the wrapper passes a scratch buffer, so at this shape the library
               runs a 4 us scale-transposition kernel and two tile launches)
  kernels      the same for act_quant and weight_dequant against the HBM peak
               (algorithmic bytes: 3.03125*M*K and 3*N*K + 4*ceil(N/128)*ceil(K/128)),
               each timed alone, cold cache (a 512 MiB buffer is rewritten before every launch),
               and per launch of several back-to-back launches on uncached buffers (us_streamed)
  cpu_baseline the CPU oracle (dequantize + fp32 matmul, torch CPU ops) on a bounded
               sample of the same workload, on the host cores of this box
Before the W warm-up steps the script runs the same step for 50 ms (set-up, untimed): after an idle period the
GPU needs some 20 ms of work to reach its sustained clock, whatever W is.
With --table a per-kernel table for every benchmark configuration goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0   # MI355X dense FP8 MFMA, published
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E, published

# HBM bytes per fp8_gemm call at the C3 shape (both of its launches), from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (KiB per dispatch, scaled by the same counters read on a plain copy kernel of known size); the runs are
# summarised in profiles/bench_C3_hbm_traffic.txt: FETCH_SIZE (347 857 + 72 233) KiB x 1.9997 (copy-kernel
# calibration) = 860.2 MB read, WRITE_SIZE (134 131 + 16 418) KiB x 1.0 = 154.2 MB written; algorithmic bytes are
# 313 MB (the A and B panels are re-fetched by the eight XCD-local L2s).
GEMM_C3_HBM_TRAFFIC_BYTES = 1014.4e6

WORKLOADS = {
    # name: (activation kind, M, N, K, description)
    "C1": ("normal", 128, 1024, 1024, "CPU reference case: X[128,1024], W[1024,1024]"),
    "C2": ("outliers", 4096, 1536, 7168, "DeepSeek-V3 attention q_a proj: X[4096,7168] (1% outliers x10), W[1536,7168]"),
    "C3": ("normal", 4096, 18432, 7168, "DeepSeek-V3 dense MLP up/gate: X[4096,7168], W[18432,7168] (headline GEMM shape)"),
    "C4": ("heavy", 4096, 7168, 18432, "DeepSeek-V3 dense MLP down: X[4096,18432] heavy-tailed, W[7168,18432]"),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="C3", choices=sorted(WORKLOADS))
    ap.add_argument("--table", action="store_true", help="also print a per-kernel table for all configurations to stderr")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calib-copy", action="store_true",
                    help="first run one plain 256 MiB device-to-device copy kernel (counter calibration for rocprofv3 --pmc)")
    return ap.parse_args()


def make_inputs(torch, kind, M, N, K, seed, dev):
    """Synthetic tensors of the configuration, generated on the device (values follow the
    benchmark definition; the parity tests use CPU-generated seeded inputs instead)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.randn(M, K, generator=g, device=dev)
    if kind == "outliers":
        x = torch.where(torch.rand(M, K, generator=g, device=dev) < 0.01, x * 10, x)
    elif kind == "heavy":
        x = x * torch.randn(M, K, generator=g, device=dev).abs()
    x = x.bfloat16()
    w = (torch.randn(N, K, generator=g, device=dev) * 0.02).bfloat16()
    return x, w


class ColdTimer:
    """HIP-event timing of single launches on the current stream with a cache flush before each."""

    def __init__(self, torch, dev):
        self.torch = torch
        self.flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)

    def run(self, fn, reps, cold=True):
        """cold=True: flush by rewriting 512 MiB, which leaves the caches full of dirty lines (every miss of
        the timed kernel then also pays a write-back: the conservative protocol, used for every headline
        figure); cold="read": flush by reading 512 MiB (clean lines, what a kernel sees when other weights
        were streamed before it); cold=False: back to back."""
        torch = self.torch
        fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(reps):
            if cold == "read":
                self.flush.view(torch.int64).sum()
            elif cold:
                self.flush.add_(1)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3)
        ts.sort()
        return ts[len(ts) // 2], sum(ts) / len(ts)


def streamed_us(torch, timer, fns, reps):
    """Per-launch time of `fns` (the same kernel on different buffers, together larger than the 256 MB
    Infinity Cache) issued back to back inside one event pair after a cache flush: every launch reads and
    writes memory that is not cached, and the ~3 us that an event pair adds to a single launch is spread over
    all of them.  The results are kept alive until the pair is closed so that no output buffer is reused."""
    for f in fns:
        f()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        timer.flush.add_(1)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        keep = [f() for f in fns]
        e1.record()
        torch.cuda.synchronize()
        del keep
        ts.append(e0.elapsed_time(e1) * 1e3 / len(fns))
    ts.sort()
    return ts[len(ts) // 2]


def cpu_baseline(torch, kind, M, N, K, xq, xs, wq, ws):
    """The CPU oracle (dequantize activations + dequantize weights + fp32 matmul -> bf16) on a
    bounded sample: `rows` activation rows (all of them up to 4096) against the full weight,
    one pass.  If rows < M the row-proportional parts are extrapolated linearly."""
    from oracle import oracle as O
    torch.set_num_threads(os.cpu_count() or 1)
    cores = torch.get_num_threads()
    rows = min(M, 4096)
    a = xq[:rows].cpu()
    a_s = xs[:rows].cpu()
    b = wq.cpu()
    b_s = ws.cpu()
    t0 = time.perf_counter()
    bd = O.weight_dequant(b, b_s, dtype=torch.float32)
    t1 = time.perf_counter()
    ad = O.dequant_rows(a, a_s)
    t2 = time.perf_counter()
    c = (ad @ bd.t()).to(torch.bfloat16)
    t3 = time.perf_counter()
    t_w, t_a, t_mm = t1 - t0, t2 - t1, t3 - t2
    full = t_w + (t_a + t_mm) * (M / rows)
    model = ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {
        "value": round(2.0 * M * N * K / full / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": ("%d of %d activation rows x full W[%d,%d]: weight dequant %.2f s (once), act dequant %.3f s, "
                   "fp32 matmul %.2f s; row-proportional parts extrapolated to %d rows -> %.1f s per step; cpu: %s"
                   % (rows, M, N, K, t_w, t_a, t_mm, M, full, model)),
        "checksum": float(c.float().abs().mean()),
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the path shards by N or K "
              "without changing the kernels); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (torch.cuda.is_available() is False)", file=sys.stderr)
        sys.exit(2)
    import mdy_triton_amd as m
    from mdy_triton_amd.fp8 import quant_weight  # noqa: F401  (weight side is prepared once, untimed)
    from oracle import oracle as O

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    kind, M, N, K, desc = WORKLOADS[args.workload]
    x, w = make_inputs(torch, kind, M, N, K, 0, dev)
    # weight: block-quantized once with the official-dialect quantizer (amax/448, no eps)
    wq = torch.empty(N, K, dtype=torch.float8_e4m3fn, device=dev)
    ws = torch.empty((N + 127) // 128, K // 128, dtype=torch.float32, device=dev)
    from mdy_triton_amd import _lib
    _lib.check(_lib.load().mdy_weight_quant(w.data_ptr(), wq.data_ptr(), ws.data_ptr(), None, None, N, K, K, 1,
                                            N, K, 0, None), "weight_quant")
    torch.cuda.synchronize()

    def step():
        xq, xs = m.act_quant(x)
        return xq, xs, m.fp8_gemm(xq, xs, wq, ws, out_dtype=torch.bfloat16)

    if args.calib_copy:
        src = torch.full((64 << 20,), 1.0, dtype=torch.float32, device=dev)   # 256 MiB
        dst = torch.empty_like(src)
        dst.copy_(src)                                                          # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # set-up, not part of the measurement: bring the GPU out of its idle power state (the first ~20 ms of work
    # after an idle period run at a fraction of the sustained clock, whatever --warmup says)
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < 0.05:
        step()
        torch.cuda.synchronize()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # ---- timed region: exactly `steps` steps; HIP events bracket every fp8_gemm launch
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        xq, xs = m.act_quant(x)
        ev[i][0].record()
        out = m.fp8_gemm(xq, xs, wq, ws, out_dtype=torch.bfloat16)
        ev[i][1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    gemm_us = sum(a.elapsed_time(b) for a, b in ev) * 1e3 / args.steps
    flops = 2.0 * M * N * K

    # ---- the two HBM-bound kernels, each alone, cold cache
    timer = ColdTimer(torch, dev)
    aq_us, _ = timer.run(lambda: m.act_quant(x), 30)
    wd_us, _ = timer.run(lambda: m.weight_dequant(wq, ws, out_dtype=torch.bfloat16), 30)
    gemm_cold_us, _ = timer.run(lambda: m.fp8_gemm(xq, xs, wq, ws, out_dtype=torch.bfloat16), 15)
    xs_copies = [x.clone() for _ in range(max(2, int(6e8 // (2 * M * K)) + 1))]
    aq_stream_us = streamed_us(torch, timer, [(lambda xc=xc: m.act_quant(xc)) for xc in xs_copies], 10)
    del xs_copies
    wq_copies = [wq.clone() for _ in range(max(2, int(4e8 // (N * K)) + 1))]
    wd_stream_us = streamed_us(torch, timer, [(lambda wc=wc: m.weight_dequant(wc, ws, out_dtype=torch.bfloat16))
                                              for wc in wq_copies], 10)
    del wq_copies
    aq_bytes = 3.03125 * M * K
    wd_bytes = 3.0 * N * K + 4.0 * ((N + 127) // 128) * (K // 128)

    # ---- parity spot check of this very run against the oracle (a few rows)
    rows = torch.tensor([0, M // 2, M - 1])
    ref = O.fp8_gemm(xq[rows.to(dev)].cpu(), xs[rows.to(dev)].cpu(), wq.cpu(), ws.cpu(), dtype=torch.bfloat16)
    parity_ok = bool(torch.allclose(out[rows.to(dev)].float().cpu(), ref.float(), rtol=1e-2, atol=1e-2))
    yq_ref, s_ref = O.act_quant(x[rows.to(dev)].cpu())
    parity_ok = parity_ok and bool(torch.equal(xq[rows.to(dev)].cpu().view(torch.uint8), yq_ref.view(torch.uint8))) \
        and bool(torch.equal(xs[rows.to(dev)].cpu(), s_ref))

    achieved = flops / (gemm_us * 1e-6) / 1e12
    result = {
        "metric": "fp8_gemm TFLOPS + % FP8 MFMA peak; act_quant/dequant GB/s + % HBM, 1 GPU",
        "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn x fp8_e4m3fn -> fp32 accumulate -> bf16",
        "data": "synthetic",
        "config": {"workload": "%s %s; step = act_quant + fp8_gemm (pre-quantized weight)" % (args.workload, desc),
                   "M": M, "N": N, "K": K},
        "roofline": {"bound": "mfma",
                     "kernel": "fp8_gemm (one call = transpose_scales_kernel + fp8_gemm_mfma_kernel<256,256> on the first 16384 columns + <128,256> on the last 2048)"
                     if args.workload == "C3" else "fp8_gemm",
                     "achieved": round(achieved, 2), "peak": PEAK_FP8_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP8_TFLOPS, 4),
                     "launch_us": round(gemm_us, 2), "flops_per_launch": flops,
                     "traffic": GEMM_C3_HBM_TRAFFIC_BYTES if args.workload == "C3" else None},
        "kernels": {
            "fp8_gemm_cold": {"us": round(gemm_cold_us, 2), "TFLOP/s": round(flops / gemm_cold_us / 1e6, 2),
                              "frac_mfma_peak": round(flops / gemm_cold_us / 1e6 / PEAK_FP8_TFLOPS, 4)},
            # "us": one launch after a cache flush, timed by its own event pair (which adds ~3 us);
            # "us_streamed": per launch, several launches on different uncached buffers inside one event pair
            "act_quant": {"us": round(aq_us, 2), "bytes": aq_bytes, "GB/s": round(aq_bytes / aq_us / 1e3, 1),
                          "frac_hbm_peak": round(aq_bytes / aq_us / 1e3 / PEAK_HBM_GBS, 4),
                          "us_streamed": round(aq_stream_us, 2),
                          "frac_hbm_peak_streamed": round(aq_bytes / aq_stream_us / 1e3 / PEAK_HBM_GBS, 4)},
            "weight_dequant": {"us": round(wd_us, 2), "bytes": wd_bytes, "GB/s": round(wd_bytes / wd_us / 1e3, 1),
                               "frac_hbm_peak": round(wd_bytes / wd_us / 1e3 / PEAK_HBM_GBS, 4),
                               "us_streamed": round(wd_stream_us, 2),
                               "frac_hbm_peak_streamed": round(wd_bytes / wd_stream_us / 1e3 / PEAK_HBM_GBS, 4)},
        },
        "parity_spot_check": parity_ok,
    }
    # the same peak derived from the device the run is on: CUs x 4 SIMDs x 2048 FP8 flop per clock x max clock
    props = torch.cuda.get_device_properties(dev)
    clock_khz = getattr(props, "clock_rate", 0) or 2400000      # MI355X: 2.4 GHz peak engine clock
    result["roofline"]["peak_from_device_props"] = round(props.multi_processor_count * 4 * 2048 * clock_khz * 1e3 / 1e12, 1)
    result["roofline"]["device"] = "%s, %d CUs, %.2f GHz" % (props.name, props.multi_processor_count, clock_khz / 1e6)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, kind, M, N, K, xq, xs, wq, ws)

    if args.table:
        table(torch, m, timer, dev)
    print(json.dumps(result))


def table(torch, m, timer, dev):
    """Per-kernel table for every configuration (stderr)."""
    FP8 = torch.float8_e4m3fn

    def line(name, us, work, unit, peak):
        rate = work / us / (1e6 if unit == "TFLOP/s" else 1e3)
        print("%-46s %9.1f us %10.2f %-8s %5.1f %% of peak" % (name, us, rate, unit, 100 * rate / peak), file=sys.stderr)

    for name, (kind, M, N, K, _) in WORKLOADS.items():
        x, w = make_inputs(torch, kind, M, N, K, 1, dev)
        wq, ws, _, _ = m.quant_weight(w)
        xq, xs = m.act_quant(x)
        line("%s act_quant %dx%d" % (name, M, K), timer.run(lambda: m.act_quant(x), 20)[0], 3.03125 * M * K, "GB/s", PEAK_HBM_GBS)
        line("%s weight_dequant %dx%d" % (name, N, K), timer.run(lambda: m.weight_dequant(wq, ws, out_dtype=torch.bfloat16), 20)[0],
             3.0 * N * K + 4.0 * ((N + 127) // 128) * (K // 128), "GB/s", PEAK_HBM_GBS)
        line("%s fp8_gemm %dx%dx%d" % (name, M, N, K), timer.run(lambda: m.fp8_gemm(xq, xs, wq, ws, out_dtype=torch.bfloat16), 10)[0],
             2.0 * M * N * K, "TFLOP/s", PEAK_FP8_TFLOPS)
    # training-time operators at the C3 shapes (DeepLinear dialect): bytes = 2 in + 1 out + 1 transposed out per element
    kind, M, N, K, _ = WORKLOADS["C3"]
    x, w = make_inputs(torch, kind, M, N, K, 2, dev)
    dy = torch.randn(M, N, device=dev, dtype=torch.bfloat16)
    line("C3 quant_input(train) %dx%d" % (M, K), timer.run(lambda: m.quant_input(x, False), 20)[0], 4.0 * M * K, "GB/s", PEAK_HBM_GBS)
    line("C3 quant_grad_output %dx%d" % (M, N), timer.run(lambda: m.quant_grad_output(dy), 20)[0], 4.0 * M * N, "GB/s", PEAK_HBM_GBS)
    line("C3 quant_weight(train) %dx%d" % (N, K), timer.run(lambda: m.quant_weight(w, False), 20)[0], 4.0 * N * K, "GB/s", PEAK_HBM_GBS)
    lin = m.DeepLinear(K, N, bias=False, dtype=torch.bfloat16, device=dev)
    xg = x.clone().requires_grad_(True)

    def train_step():
        lin.zero_grad(set_to_none=True)
        xg.grad = None
        lin(xg).backward(dy)
    def three_steps():      # the GPU idles ~70 us while the host prepares the first launch after a flush: spread it
        for _ in range(3):
            train_step()
    line("C3 DeepLinear fwd+bwd (3 GEMMs + quantizers), per step of 3", timer.run(three_steps, 6)[0] / 3, 6.0 * M * N * K, "TFLOP/s", PEAK_FP8_TFLOPS)
    del lin, xg, dy, x, w
    # SwiGLU in front of the MLP-down quantizer (C4's activation): fused vs the reference's two passes
    Ms, Ns = 4096, 18432
    ug = (torch.randn(Ms, 2 * Ns, device=dev) * 1.5).to(torch.bfloat16)
    line("C4 silu_act_quant fused %dx%d" % (Ms, Ns), timer.run(lambda: m.silu_act_quant(ug), 20)[0], 5.03125 * Ms * Ns, "GB/s", PEAK_HBM_GBS)

    def unfused():
        m.act_quant(m.silu_fwd(ug))
    line("C4 silu_fwd + act_quant (2 passes) %dx%d" % (Ms, Ns), timer.run(unfused, 20)[0], 9.03125 * Ms * Ns, "GB/s", PEAK_HBM_GBS)
    line("C4 silu_fwd %dx%d" % (Ms, Ns), timer.run(lambda: m.silu_fwd(ug), 20)[0], 6.0 * Ms * Ns, "GB/s", PEAK_HBM_GBS)
    dact = (torch.randn(Ms, Ns, device=dev)).to(torch.bfloat16)
    # backward: reads up, gate and dy, writes d_up and d_gate: 10 bytes per activation element
    line("C4 silu_bwd %dx%d" % (Ms, Ns), timer.run(lambda: m.silu_bwd(dact, ug), 20)[0], 10.0 * Ms * Ns, "GB/s", PEAK_HBM_GBS)
    del ug, dact
    # grouped (MoE) GEMM: 32 routed experts of the up/gate projection (N = 2 x 2048, K = 7168)
    G, Ng, Kg = 32, 4096, 7168
    bq = torch.randint(0, 120, (G, Ng, Kg), dtype=torch.uint8, device=dev).view(FP8)
    bsg = torch.rand(G, Ng // 128, Kg // 128, device=dev)
    for mg in (512, 16):
        Mt = G * mg
        aq = torch.randint(0, 120, (Mt, Kg), dtype=torch.uint8, device=dev).view(FP8)
        asg = torch.rand(Kg // 128, Mt, device=dev).t()     # logical [Mt, K/128], strides (1, Mt): what
        #                                                       group_per_token_cast_to_fp8 returns
        us = timer.run(lambda: m.fp8_grouped_matmul(aq, asg, bq, bsg, [mg] * G), 10)[0]
        if mg >= 256:
            line("grouped fp8_gemm %d experts x %d rows, N=%d K=%d" % (G, mg, Ng, Kg), us, 2.0 * Mt * Ng * Kg, "TFLOP/s", PEAK_FP8_TFLOPS)
        else:
            line("grouped fp8_gemm %d experts x %d rows, N=%d K=%d" % (G, mg, Ng, Kg), us,
                 Mt * Kg + G * Ng * Kg + 2.0 * Mt * Ng + 4.0 * Mt * Kg / 128, "GB/s", PEAK_HBM_GBS)
            us = timer.run(lambda: m.fp8_grouped_matmul(aq, asg, bq, bsg, [mg] * G), 10, cold="read")[0]
            line("   the same after a read-only cache flush", us,
                 Mt * Kg + G * Ng * Kg + 2.0 * Mt * Ng + 4.0 * Mt * Kg / 128, "GB/s", PEAK_HBM_GBS)
    # ragged experts (8 x 1000 rows): 256-row tiles plus one 128-row tile per expert in the same launch
    Gr, mr = 8, 1000
    aq = torch.randint(0, 120, (Gr * mr, Kg), dtype=torch.uint8, device=dev).view(FP8)
    asg = torch.rand(Kg // 128, Gr * mr, device=dev).t()
    us = timer.run(lambda: m.fp8_grouped_matmul(aq, asg, bq[:Gr], bsg[:Gr], [mr] * Gr), 10)[0]
    line("grouped fp8_gemm %d experts x %d rows, N=%d K=%d" % (Gr, mr, Ng, Kg), us, 2.0 * Gr * mr * Ng * Kg, "TFLOP/s", PEAK_FP8_TFLOPS)
    del bq, bsg, aq, asg
    for M in (1, 16, 64):
        for (N, K) in ((7168, 2048), (2048, 7168)):
            a = torch.randint(0, 120, (M, K), dtype=torch.uint8, device=dev).view(FP8)
            b = torch.randint(0, 120, (N, K), dtype=torch.uint8, device=dev).view(FP8)
            a_s = torch.rand(M, K // 128, device=dev)
            b_s = torch.rand(N // 128, K // 128, device=dev)
            byts = M * K + N * K + 4 * M * K / 128 + 4 * (N // 128) * (K // 128) + 2 * M * N

            def many():
                for _ in range(20):
                    m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.bfloat16)
            us = timer.run(many, 10, cold=False)[0] / 20
            line("C5 fp8_gemm M=%d N=%d K=%d (warm, back-to-back)" % (M, N, K), us, byts, "GB/s", PEAK_HBM_GBS)
    # few rows against a long K (small-batch prefill / large-batch decode): tiles do not fill the GPU, the
    # wrapper hands the library a workspace and the shape is split along K; weight bytes bound these
    for (M, N, K) in ((128, 7168, 16384), (128, 2112, 7168), (256, 7168, 18432), (512, 4096, 7168)):
        a = torch.randint(0, 120, (M, K), dtype=torch.uint8, device=dev).view(FP8)
        b = torch.randint(0, 120, (N, K), dtype=torch.uint8, device=dev).view(FP8)
        a_s = torch.rand(M, K // 128, device=dev)
        b_s = torch.rand((N + 127) // 128, K // 128, device=dev)
        byts = M * K + N * K + 4 * M * K / 128 + 4 * ((N + 127) // 128) * (K // 128) + 2 * M * N
        us = timer.run(lambda: m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.bfloat16), 10)[0]
        line("fp8_gemm M=%d N=%d K=%d (split along K)" % (M, N, K), us, byts, "GB/s", PEAK_HBM_GBS)
        us = timer.run(lambda: m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.bfloat16), 10, cold="read")[0]
        line("   the same after a read-only cache flush", us, byts, "GB/s", PEAK_HBM_GBS)


if __name__ == "__main__":
    main()
