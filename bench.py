#!/usr/bin/env python3
"""Benchmark of the block-wise FP8 linear path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--table] [--ablation] [--ceilings] [--energy]

One "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM: act_quant(X) followed by fp8_gemm(Xq, Xs, Wq, Ws) -> bf16,
i.e. the FP8 linear forward with a pre-quantized weight.  The default workload is
the headline shape of the benchmark definition: DeepSeek-V3 dense MLP up/gate,
X[4096, 7168] bf16 ~ N(0,1), W[18432, 7168] e4m3fn with 128x128 fp32 block scales.
Inputs are generated on the CPU from torch.Generator().manual_seed(config index)
and copied to the device, so that the CPU oracle and the device see the same bits.

Prints ONE JSON line on stdout:
  value        whole-step throughput in TFLOP/s (2*M*N*K / step time, quantizer included)
  roofline     the dominant kernel (fp8_gemm): algorithmic FLOPs per call / its average
               duration, measured with HIP events on the launch stream inside the timed
               region, against the dense FP8 MFMA peak (a call is fp8_gemm() as a user
               makes it: the wrapper passes a scratch buffer, so at this shape the library
               runs a 4 us scale-transposition kernel and two tile launches); `traffic` is
               read from the tracked rocprofv3 summary profiles/bench_C3_hbm_traffic.txt
  kernels      act_quant and weight_dequant of the workload against the HBM peak
               (algorithmic bytes: 3.03125*M*K and 3*N*K + 4*ceil(N/128)*ceil(K/128)),
               each timed alone, cold cache (a 512 MiB buffer is rewritten before every launch),
               and per launch of several back-to-back launches on uncached buffers (us_streamed);
               the same three kernels at the other large configurations (C2, C4; cold, one
               event pair per launch; the GEMM also as the headline GEMM is timed: bracketed by
               events inside a loop of act_quant + fp8_gemm, `us_in_loop`); the six decode shapes (C5) as the per-call time of a
               replayed HIP graph of 20 calls (the Python call is not in the number)
  power        socket power and shader clock while the GEMM runs back to back for about a
               second (amd-smi readings), next to the board's power cap
  cpu_baseline the CPU oracle (dequantize + fp32 matmul, torch CPU ops) on a bounded
               sample of the same workload, on the host cores of this box
Before the W warm-up steps the script runs the same step for 50 ms (set-up, untimed): after an idle period the
GPU needs some 20 ms of work to reach its sustained clock, whatever W is.
With --table a per-kernel table for every benchmark configuration and for the shapes the reference
publishes numbers for goes to stderr; with --ablation the tile kernel is timed with parts of its K loop
switched off (mdy_fp8_gemm_probe of libmdyfp8_probe.so), power and clock beside each line (stdout, no JSON); with
--ceilings the copy-only twins of the quantizers, a register-resident MFMA loop and the launch floor (same library).
"""
import argparse
import json
import os
import re
import subprocess
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0   # MI355X dense FP8 MFMA, published
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E, published
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bench_C3_hbm_traffic.txt")

WORKLOADS = {
    # name: (seed, activation kind, M, N, K, description)
    "C1": (1, "normal", 128, 1024, 1024, "CPU reference case: X[128,1024], W[1024,1024]"),
    "C2": (2, "outliers", 4096, 1536, 7168, "DeepSeek-V3 attention q_a proj: X[4096,7168] (1% outliers x10), W[1536,7168]"),
    "C3": (3, "normal", 4096, 18432, 7168, "DeepSeek-V3 dense MLP up/gate: X[4096,7168], W[18432,7168] (headline GEMM shape)"),
    "C4": (4, "heavy", 4096, 7168, 18432, "DeepSeek-V3 dense MLP down: X[4096,18432] heavy-tailed, W[7168,18432]"),
}
DECODE_SHAPES = [(M, N, K) for M in (1, 16, 64) for (N, K) in ((7168, 2048), (2048, 7168))]


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="C3", choices=sorted(WORKLOADS))
    ap.add_argument("--table", action="store_true", help="also print a per-kernel table for all configurations to stderr")
    ap.add_argument("--ablation", action="store_true",
                    help="time the tile kernel with parts of its K loop switched off, with power and clock (no JSON)")
    ap.add_argument("--energy", action="store_true",
                    help="energy per call of the headline GEMM's main launch for other XCD tile-block shapes (no JSON)")
    ap.add_argument("--energy-launches", type=int, default=0,
                    help="with --energy: launch every variant only this many times (for a rocprofv3 --pmc run)")
    ap.add_argument("--ceilings", action="store_true",
                    help="copy-only twins of the quantizers, the MFMA-only register loop and the launch floor (no JSON)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload (skip C2, C4, C5 and the power loop)")
    ap.add_argument("--only-decode", action="store_true",
                    help="only the six decode shapes (C5): 200 eager calls each, then the graph replays; prints their JSON entries")
    ap.add_argument("--calib-copy", action="store_true",
                    help="first run one plain 256 MiB device-to-device copy kernel (counter calibration for rocprofv3 --pmc)")
    return ap.parse_args()


def make_inputs(torch, kind, M, N, K, seed, dev):
    """Synthetic tensors of a configuration: generated on the CPU from a seeded generator (values follow the
    benchmark definition), then copied to the device."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    if kind == "outliers":
        x = torch.where(torch.rand(M, K, generator=g) < 0.01, x * 10, x)
    elif kind == "heavy":
        x = x * torch.randn(M, K, generator=g).abs()
    x = x.bfloat16()
    w = torch.randn(N, K, generator=g).mul_(0.02).bfloat16()
    return x.to(dev), w.to(dev)


def quantize_weight(torch, w, dev):
    """Block-quantize a bf16 weight once with the official-dialect quantizer (amax/448, no eps): set-up, untimed."""
    from mdy_triton_amd import _lib
    N, K = w.shape
    wq = torch.empty(N, K, dtype=torch.float8_e4m3fn, device=dev)
    ws = torch.empty((N + 127) // 128, K // 128, dtype=torch.float32, device=dev)
    PN = (N + 127) // 128 * 128
    if PN != N:
        wq_p = torch.empty(PN, K, dtype=torch.float8_e4m3fn, device=dev)
        _lib.check(_lib.load().mdy_weight_quant(w.data_ptr(), wq_p.data_ptr(), ws.data_ptr(), None, None, N, K, K, 1,
                                                PN, K, 0, None), "weight_quant")
        wq.copy_(wq_p[:N])
    else:
        _lib.check(_lib.load().mdy_weight_quant(w.data_ptr(), wq.data_ptr(), ws.data_ptr(), None, None, N, K, K, 1,
                                                N, K, 0, None), "weight_quant")
    torch.cuda.synchronize()
    return wq, ws


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


def graph_replay_us(torch, fn, calls=20, reps=7):
    """Per-call time of `fn` inside a replayed HIP graph of `calls` calls (the median of `reps` replays): kernel
    durations plus the gaps between dependent kernels, no host launch cost."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for _ in range(calls):
            out = fn()
    graph.replay()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        ts.append(e0.elapsed_time(e1) * 1e3 / calls)
    del out, graph
    ts.sort()
    return ts[len(ts) // 2]


class SmiSampler(threading.Thread):
    """Socket power (W) and the mean shader clock of the XCDs (MHz) from `amd-smi metric --clock --power --json`,
    sampled in the background while a loop runs on the GPU.  Readings are best effort: no amd-smi, no samples."""

    def __init__(self, period=0.1):
        super().__init__(daemon=True)
        self.period = period
        self.halt = False
        self.samples = []

    @staticmethod
    def read():
        try:
            r = subprocess.run(["amd-smi", "metric", "--clock", "--power", "--json"], stdout=subprocess.PIPE,
                               stderr=subprocess.DEVNULL, text=True, timeout=5)
            d = json.loads(r.stdout)
            g = (d["gpu_data"] if isinstance(d, dict) else d)[0]
            power = g["power"]["socket_power"]["value"]
            clks = [v["clk"]["value"] for k, v in g["clock"].items() if k.startswith("gfx_") and isinstance(v, dict)
                    and isinstance(v.get("clk"), dict) and isinstance(v["clk"].get("value"), (int, float))]
            return float(power), (sum(clks) / len(clks) if clks else None)
        except Exception:
            return None

    def run(self):
        while not self.halt:
            s = self.read()
            if s is not None:
                self.samples.append((time.perf_counter(),) + s)
            time.sleep(self.period)

    def summary(self, t_from):
        rows = [s for s in self.samples if s[0] >= t_from]
        if not rows:
            return None
        ps = [s[1] for s in rows]
        cs = [s[2] for s in rows if s[2] is not None]
        return {"socket_power_w": round(sum(ps) / len(ps), 1), "socket_power_max_w": round(max(ps), 1),
                "gfx_clock_mhz": round(sum(cs) / len(cs), 0) if cs else None, "samples": len(rows)}


def power_cap_w():
    import glob
    for f in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap"):
        try:
            return float(open(f).read()) / 1e6
        except (OSError, ValueError):
            pass
    return None


def sustained(torch, fn, seconds=2.0, batch=10):
    """Runs fn back to back for `seconds`; returns (us per call over the second half, amd-smi summary of the same half)."""
    sampler = SmiSampler()
    sampler.start()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    half = None
    n_half = 0
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    while True:
        now = time.perf_counter()
        if half is None and now - t0 >= seconds / 2:
            half = now
            e0.record()
        if now - t0 >= seconds:
            break
        for _ in range(batch):
            fn()
        if half is not None:
            n_half += batch
        torch.cuda.synchronize()
    e1.record()
    torch.cuda.synchronize()
    sampler.halt = True
    sampler.join()
    us = e0.elapsed_time(e1) * 1e3 / max(n_half, 1)
    return us, sampler.summary(half)


def cpu_baseline(torch, kind, M, N, K, xq, xs, wq, ws, x=None):
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
    # the two HBM-bound operators on the same host cores, each alone: the oracle's act_quant on the workload's
    # activations, and its weight_dequant to bf16 (what the GPU kernel writes)
    extra = {}
    if x is not None:
        xc = x[:rows].cpu()
        t4 = time.perf_counter()
        O.act_quant(xc)
        t5 = time.perf_counter()
        extra["act_quant"] = {"GB/s": round(3.03125 * rows * K / (t5 - t4) / 1e9, 2), "s": round(t5 - t4, 3), "rows": rows}
    t6 = time.perf_counter()
    O.weight_dequant(b, b_s, dtype=torch.bfloat16)
    t7 = time.perf_counter()
    extra["weight_dequant"] = {"GB/s": round((3.0 * N * K + 4.0 * b_s.numel()) / (t7 - t6) / 1e9, 2), "s": round(t7 - t6, 3)}
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
        "kernels": extra,
    }, c


def traffic_from_profile():
    """HBM-side bytes of one fp8_gemm call at the C3 shape, from the line `fp8_gemm_call_traffic_bytes <n>` of the
    tracked rocprofv3 summary (FETCH_SIZE + WRITE_SIZE of the call's launches, calibrated on a copy kernel)."""
    try:
        m = re.search(r"^fp8_gemm_call_traffic_bytes\s+([0-9.eE+]+)", open(TRAFFIC_PROFILE).read(), re.M)
        return float(m.group(1)) if m else None
    except OSError:
        return None


def gemm_bytes(M, N, K):
    return M * K + N * K + 4 * M * (K // 128) + 4 * ((N + 127) // 128) * (K // 128) + 2 * M * N


def kernel_entries(torch, m, timer, x, wq, ws, reps=12):
    """act_quant / weight_dequant / fp8_gemm of one configuration, cold cache, one event pair per launch."""
    M, K = x.shape
    N = wq.size(0)
    xq, xs = m.act_quant(x)
    aq_us, _ = timer.run(lambda: m.act_quant(x), reps)
    wd_us, _ = timer.run(lambda: m.weight_dequant(wq, ws, out_dtype=torch.bfloat16), reps)
    g_us, _ = timer.run(lambda: m.fp8_gemm(xq, xs, wq, ws, out_dtype=torch.bfloat16), reps)
    # the same GEMM in the loop the headline value is measured in: act_quant + fp8_gemm back to back, the GEMM bracketed by
    # events (its operands come from the caches the way they do between the layers of a model)
    for _ in range(5):
        a_, s_ = m.act_quant(x)
        m.fp8_gemm(a_, s_, wq, ws, out_dtype=torch.bfloat16)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(20)]
    for e0, e1 in ev:
        a_, s_ = m.act_quant(x)
        e0.record()
        m.fp8_gemm(a_, s_, wq, ws, out_dtype=torch.bfloat16)
        e1.record()
    torch.cuda.synchronize()
    loop_us = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in ev)[len(ev) // 2]
    aq_b = 3.03125 * M * K
    wd_b = 3.0 * N * K + 4.0 * ((N + 127) // 128) * (K // 128)
    fl = 2.0 * M * N * K
    return {
        "act_quant": {"us": round(aq_us, 2), "GB/s": round(aq_b / aq_us / 1e3, 1),
                      "frac_hbm_peak": round(aq_b / aq_us / 1e3 / PEAK_HBM_GBS, 4)},
        "weight_dequant": {"us": round(wd_us, 2), "GB/s": round(wd_b / wd_us / 1e3, 1),
                           "frac_hbm_peak": round(wd_b / wd_us / 1e3 / PEAK_HBM_GBS, 4)},
        "fp8_gemm": {"us": round(g_us, 2), "TFLOP/s": round(fl / g_us / 1e6, 1),
                     "frac_mfma_peak": round(fl / g_us / 1e6 / PEAK_FP8_TFLOPS, 4),
                     "us_in_loop": round(loop_us, 2), "frac_mfma_peak_in_loop": round(fl / loop_us / 1e6 / PEAK_FP8_TFLOPS, 4)},
    }


def decode_entries(torch, m, dev, eager_calls=0):
    """The six decode / routed-expert shapes: per-call time inside a replayed HIP graph, against the HBM peak on the
    algorithmic bytes (weights + activations + scales + output).  The weights (14.7 MB) stay in the caches between
    the calls of a graph, so this is the kernel's speed, not a cold-memory figure."""
    out = {}
    for i, (M, N, K) in enumerate(DECODE_SHAPES):
        g = torch.Generator().manual_seed(50 + i)
        x = torch.randn(M, K, generator=g).bfloat16().to(dev)
        w = torch.randn(N, K, generator=g).mul_(0.02).bfloat16().to(dev)
        wq, ws = quantize_weight(torch, w, dev)
        xq, xs = m.act_quant(x)
        for _ in range(eager_calls):        # for a kernel trace: plain launches, one kernel record each
            m.fp8_gemm(xq, xs, wq, ws, out_dtype=torch.bfloat16)
        us = graph_replay_us(torch, lambda: m.fp8_gemm(xq, xs, wq, ws, out_dtype=torch.bfloat16))
        aq_us = graph_replay_us(torch, lambda: m.act_quant(x))
        b = gemm_bytes(M, N, K)
        out["M=%d,N=%d,K=%d" % (M, N, K)] = {"fp8_gemm_us": round(us, 2), "GB/s": round(b / us / 1e3, 1),
                                              "frac_hbm_peak": round(b / us / 1e3 / PEAK_HBM_GBS, 4),
                                              "act_quant_us": round(aq_us, 2)}
    return out


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
    from oracle import oracle as O

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.ablation:
        ablation(torch, m, dev)
        return
    if args.ceilings:
        ceilings(torch, m, ColdTimer(torch, dev), dev)
        return
    if args.energy:
        energy(torch, m, dev, args.energy_launches)
        return
    if args.only_decode:
        print(json.dumps({"C5_graph_replay": decode_entries(torch, m, dev, eager_calls=200)}))
        return
    seed, kind, M, N, K, desc = WORKLOADS[args.workload]
    x, w = make_inputs(torch, kind, M, N, K, seed, dev)
    wq, ws = quantize_weight(torch, w, dev)
    del w

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
        "data": "synthetic (CPU-seeded, copied to the device)",
        "config": {"workload": "%s %s; step = act_quant + fp8_gemm (pre-quantized weight)" % (args.workload, desc),
                   "M": M, "N": N, "K": K},
        "roofline": {"bound": "mfma",
                     "kernel": "fp8_gemm (one call = transpose_scales_kernel + fp8_gemm_mfma_kernel<256,256> on the first 16384 columns + <128,256> on the last 2048)"
                     if args.workload == "C3" else "fp8_gemm",
                     "achieved": round(achieved, 2), "peak": PEAK_FP8_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP8_TFLOPS, 4),
                     "launch_us": round(gemm_us, 2), "flops_per_launch": flops,
                     "traffic": traffic_from_profile() if args.workload == "C3" else None},
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
    }
    # the same peak derived from the device the run is on: CUs x 4 SIMDs x 2048 FP8 flop per clock x max clock
    props = torch.cuda.get_device_properties(dev)
    clock_khz = getattr(props, "clock_rate", 0) or 2400000      # MI355X: 2.4 GHz peak engine clock
    result["roofline"]["peak_from_device_props"] = round(props.multi_processor_count * 4 * 2048 * clock_khz * 1e3 / 1e12, 1)
    result["roofline"]["device"] = "%s, %d CUs, %.2f GHz" % (props.name, props.multi_processor_count, clock_khz / 1e6)

    if not args.no_extra:
        # power and clock while the dominant kernel runs back to back (what bounds it: see the power cap beside it)
        us, smi = sustained(torch, lambda: m.fp8_gemm(xq, xs, wq, ws, out_dtype=torch.bfloat16))
        result["power"] = {"loop": "fp8_gemm %s back to back for 2 s, second half" % args.workload,
                           "gemm_us": round(us, 1), "power_cap_w": power_cap_w()}
        if smi:
            result["power"].update(smi)

    # ---- parity of this very run against the oracle: act_quant bit-exact on sampled rows, GEMM on the CPU leg's rows
    rows = torch.tensor([0, M // 2, M - 1])
    yq_ref, s_ref = O.act_quant(x[rows.to(dev)].cpu())
    parity_ok = bool(torch.equal(xq[rows.to(dev)].cpu().view(torch.uint8), yq_ref.view(torch.uint8))) \
        and bool(torch.equal(xs[rows.to(dev)].cpu(), s_ref))
    if not args.no_cpu:
        result["cpu_baseline"], c_ref = cpu_baseline(torch, kind, M, N, K, xq, xs, wq, ws, x)
        got = out[:c_ref.size(0)].float().cpu()
        parity_ok = parity_ok and bool(torch.allclose(got, c_ref.float(), rtol=1e-2, atol=1e-2))
        result["parity_rows_checked"] = int(c_ref.size(0))
        del c_ref, got
    else:
        ref = O.fp8_gemm(xq[rows.to(dev)].cpu(), xs[rows.to(dev)].cpu(), wq.cpu(), ws.cpu(), dtype=torch.bfloat16)
        parity_ok = parity_ok and bool(torch.allclose(out[rows.to(dev)].float().cpu(), ref.float(), rtol=1e-2, atol=1e-2))
        result["parity_rows_checked"] = 3
    result["parity_spot_check"] = parity_ok

    if not args.no_extra:
        del out, xq, xs
        for name in ("C2", "C3", "C4"):
            if name == args.workload:
                continue
            s2, k2, M2, N2, K2, _ = WORKLOADS[name]
            x2, w2 = make_inputs(torch, k2, M2, N2, K2, s2, dev)
            wq2, ws2 = quantize_weight(torch, w2, dev)
            del w2
            result["kernels"][name] = kernel_entries(torch, m, timer, x2, wq2, ws2)
            result["kernels"][name]["shape"] = {"M": M2, "N": N2, "K": K2}
            del x2, wq2, ws2
        result["kernels"]["C5_graph_replay"] = decode_entries(torch, m, dev)

    if args.table:
        table(torch, m, timer, dev)
    print(json.dumps(result))


def load_probe_lib():
    """libmdyfp8_probe.so: the timing probes (ablated tile kernels, copy-only and MFMA-only ceilings).  Not part of the
    product library; only the diagnostic modes of this script load it."""
    import ctypes
    path = os.path.join(ROOT, "mdy_triton_amd", "csrc", "libmdyfp8_probe.so")
    if not os.path.exists(path):
        raise SystemExit("%s not found: build it with `python -m mdy_triton_amd.csrc.build`" % path)
    L = ctypes.CDLL(path)
    i64, p, i = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
    L.mdy_fp8_gemm_probe.argtypes = [i, i, p, p, i64, i64, p, p, p, i64, i64, i64, p]
    L.mdy_fp8_gemm_order_probe.argtypes = [i, i, p, p, i64, i64, p, p, p, i64, i64, i64, p]
    L.mdy_fp8_gemm_order_probe.restype = i
    L.mdy_probe_copy_aq.argtypes = [p, p, p, i64, i64, p]
    L.mdy_probe_copy_wd.argtypes = [p, p, p, i64, i64, p]
    L.mdy_probe_mfma_loop.argtypes = [i, p, p, i, i, p]
    L.mdy_probe_empty.argtypes = [p]
    L.mdy_probe_load_pattern.argtypes = [i, p, p, p, i64, i64, p]
    L.mdy_probe_load_pattern.restype = i
    for f in (L.mdy_fp8_gemm_probe, L.mdy_probe_copy_aq, L.mdy_probe_copy_wd, L.mdy_probe_mfma_loop, L.mdy_probe_empty):
        f.restype = i
    return L


def energy(torch, m, dev, launches=0):
    """Energy per call of the headline GEMM's main launch (1024 tiles of 256x256: C3's first 16384 columns) for the shapes
    of the block of tiles that an XCD runs at a time (2x16, 4x8 = product, 8x4) with the pre-touches on and off: each
    variant relaunched for ~1.5 s, time per launch x socket power.  With launches > 0 every variant is only launched that
    many times (the run that rocprofv3 --pmc FETCH_SIZE counts)."""
    L = load_probe_lib()
    seed, kind, M, N, K, _ = WORKLOADS["C3"]
    N = 16384
    x, w = make_inputs(torch, kind, M, N, K, seed, dev)
    wq, ws = quantize_weight(torch, w, dev)
    xq, xs = m.act_quant(x)
    xst = xs.t().contiguous()
    c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    ref = None
    idle = SmiSampler.read()
    print("M=%d N=%d K=%d, 1024 tiles of 256x256; power cap %s W; idle reading %s" % (M, N, K, power_cap_w(), idle))
    print("%-34s %9s %8s %7s %9s %s" % ("tiles per XCD at a time / touches", "us", "W", "MHz", "mJ/call", "same bits"))
    for gm in (4, 2, 8):
        for touch in (1, 0):
            def fn(gm=gm, touch=touch):
                rc = L.mdy_fp8_gemm_order_probe(gm, touch, xq.data_ptr(), xst.data_ptr(), 1, M, wq.data_ptr(), ws.data_ptr(), c.data_ptr(),
                                                M, N, K, None)
                if rc != 0:
                    raise RuntimeError("mdy_fp8_gemm_order_probe(%d, %d) returned %d" % (gm, touch, rc))
            fn()
            torch.cuda.synchronize()
            if ref is None:
                ref = c.clone()
            same = bool(torch.equal(c, ref))
            if launches > 0:
                for _ in range(launches):
                    fn()
                torch.cuda.synchronize()
                print("%-34s launched %d times, same bits %s" % ("%dx%d, pre-touches %s" % (gm, 32 // gm, "on" if touch else "off"), launches, same))
                continue
            us, smi = sustained(torch, fn, seconds=1.5)
            smi = smi or {}
            pw = smi.get("socket_power_w")
            print("%-34s %9.1f %8s %7s %9s %s" % ("%dx%d, pre-touches %s" % (gm, 32 // gm, "on" if touch else "off"), us, pw,
                                                 smi.get("gfx_clock_mhz"), "%.1f" % (us * pw * 1e-3) if pw else "-", same), flush=True)


def ceilings(torch, m, timer, dev):
    """What the memory system and the matrix cores give this library's access patterns with the arithmetic taken out
    (libmdyfp8_probe.so), next to the product kernels under the same timing protocols (stdout, no JSON):
    copy-only twins of act_quant and weight_dequant; a register-resident MFMA loop with and without the fp32 fold of the
    block-scaled GEMM, on hashed and on constant operand bytes, with socket power and shader clock; an empty kernel
    and the M = 1 GEMM in a replayed graph."""
    L = load_probe_lib()
    from mdy_triton_amd._torch_glue import stream_ptr

    def ok(rc, what):
        if rc != 0:
            raise RuntimeError("%s returned %d" % (what, rc))

    print("== HBM streams: copy-only twin against the product kernel (us; cold = one launch after a 512 MiB flush incl. ~3 us "
          "of event overhead; streamed = per launch of back-to-back launches on uncached buffers)")
    for M, K in ((4096, 7168), (4096, 18432), (16384, 4096)):
        n = max(2, int(6e8 // (2 * M * K)) + 1)
        xs = [torch.randn(M, K, device=dev).bfloat16() for _ in range(n)]
        ys = [torch.empty(M, K, dtype=torch.uint8, device=dev) for _ in range(n)]
        ss = [torch.empty(M, K // 128, device=dev) for _ in range(n)]
        twin = [(lambda i=i: ok(L.mdy_probe_copy_aq(xs[i].data_ptr(), ys[i].data_ptr(), ss[i].data_ptr(), M, K, stream_ptr(dev)), "copy_aq"))
                for i in range(n)]
        prod = [(lambda i=i: m.act_quant(xs[i])) for i in range(n)]
        b = 3.03125 * M * K
        tc, _ = timer.run(twin[0], 20)
        pc, _ = timer.run(prod[0], 20)
        ts, ps = streamed_us(torch, timer, twin, 10), streamed_us(torch, timer, prod, 10)
        print("act_quant %5dx%-5d  copy-only cold %6.2f streamed %6.2f (%4.1f %% of 8 TB/s) | product cold %6.2f streamed %6.2f (%4.1f %%) "
              "| product / copy-only %5.3f" % (M, K, tc, ts, b / ts / 1e3 / 80, pc, ps, b / ps / 1e3 / 80, ts / ps), flush=True)
        del xs, ys, ss
    for N, K in ((18432, 7168), (7168, 18432)):
        n = max(2, int(4e8 // (N * K)) + 1)
        ws = torch.rand((N + 127) // 128, K // 128, device=dev) + 0.5
        xq = [torch.randint(0, 120, (N, K), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn) for _ in range(n)]
        ys = [torch.empty(N, K, dtype=torch.bfloat16, device=dev) for _ in range(n)]
        twin = [(lambda i=i: ok(L.mdy_probe_copy_wd(xq[i].data_ptr(), ws.data_ptr(), ys[i].data_ptr(), N, K, stream_ptr(dev)), "copy_wd"))
                for i in range(n)]
        prod = [(lambda i=i: m.weight_dequant(xq[i], ws, out_dtype=torch.bfloat16)) for i in range(n)]
        b = 3.0 * N * K + 4.0 * ws.numel()
        tc, _ = timer.run(twin[0], 20)
        pc, _ = timer.run(prod[0], 20)
        ts, ps = streamed_us(torch, timer, twin, 10), streamed_us(torch, timer, prod, 10)
        print("weight_dequant %5dx%-5d  copy-only cold %6.2f streamed %6.2f (%4.1f %% of 8 TB/s) | product cold %6.2f streamed %6.2f "
              "(%4.1f %%) | product / copy-only %5.3f" % (N, K, tc, ts, b / ts / 1e3 / 80, pc, ps, b / ps / 1e3 / 80, ts / ps), flush=True)
        del xq, ys

    print("== matrix cores alone: 8 waves per CU, 32 v_mfma_f32_16x16x128_f8f6f4 per iteration from registers, relaunched for "
          "~1.5 s; power cap %s W" % power_cap_w())
    out = torch.empty(256 * 512, device=dev)
    g = torch.Generator().manual_seed(7)
    seeds = {"hashed operand bytes": torch.randint(1, 2 ** 31 - 1, (64,), generator=g, dtype=torch.int64).to(torch.int32).to(dev),
             "constant operand bytes (0x38)": torch.zeros(64, dtype=torch.int32, device=dev)}
    iters = 1000
    flop = 256.0 * 8 * iters * 32 * 65536
    for fold, label in ((0, "MFMA only, accumulating in place"), (1, "each MFMA from zero + 4 v_fma_f32 (the block-scale fold)"),
                        (2, "32x32x64 MFMAs, accumulating in place"), (3, "32x32x64 MFMAs in pairs from zero + 16 v_fma_f32 a pair")):
        for sname, seed in seeds.items():
            def fn(fold=fold, seed=seed):
                ok(L.mdy_probe_mfma_loop(fold, seed.data_ptr(), out.data_ptr(), 256, iters, stream_ptr(dev)), "mfma_loop")
            us, smi = sustained(torch, fn, seconds=1.5)
            smi = smi or {}
            print("  %-58s %-30s %8.1f us  %6.2f PFLOP/s (%4.1f %% of 5.0)  %6s W  %5s MHz" % (
                label, sname, us, flop / us / 1e9, flop / us / 1e9 / 5.0 * 100, smi.get("socket_power_w"), smi.get("gfx_clock_mhz")), flush=True)

    print("== operand loads of a small-M GEMM alone (16 weight rows + 16 re-read activation rows per workgroup of 8 waves, every load "
          "of a wave up front): per call inside a replayed HIP graph of 20 calls")
    act = torch.randint(0, 255, (16, 8192), dtype=torch.uint8, device=dev)
    sink = torch.zeros(1 << 16, dtype=torch.int32, device=dev)
    for (N, K) in ((2048, 7168), (7168, 2048)):
        wbytes = torch.randint(0, 255, (N, K), dtype=torch.uint8, device=dev)
        row = []
        for pat, label in ((0, "MFMA fragments from memory (16 lines x 64 B per instruction)"), (1, "whole lines (8 rows x 128 B)"),
                           (2, "whole rows (1 KB per instruction)")):
            us = graph_replay_us(torch, lambda pat=pat: ok(L.mdy_probe_load_pattern(pat, wbytes.data_ptr(), act.data_ptr(), sink.data_ptr(),
                                                                                    N, K, stream_ptr(dev)), "load_pattern"))
            row.append("%s %5.2f us" % (label, us))
        print("  N=%d K=%d (%d workgroups): %s" % (N, K, N // 16, " | ".join(row)), flush=True)

    print("== launch floor: per call inside a replayed HIP graph of 20 calls")
    e_us = graph_replay_us(torch, lambda: ok(L.mdy_probe_empty(stream_ptr(dev)), "empty"))
    print("  empty kernel                         %5.2f us" % e_us)
    for (M, N, K) in ((1, 7168, 2048), (1, 2048, 7168)):
        x = torch.randn(M, K, device=dev).bfloat16()
        w = torch.randn(N, K, device=dev).mul_(0.02).bfloat16()
        wq, wsc = quantize_weight(torch, w, dev)
        xq, xsc = m.act_quant(x)
        us = graph_replay_us(torch, lambda: m.fp8_gemm(xq, xsc, wq, wsc, out_dtype=torch.bfloat16))
        print("  fp8_gemm M=%d N=%d K=%d              %5.2f us  (%.1f MB of weights: %.2f TB/s over the empty kernel's time)" % (
            M, N, K, us, N * K / 1e6, N * K / (us - e_us) / 1e6))


def ablation(torch, m, dev):
    """The tile kernel with parts of its K loop switched off, each variant run back to back for ~1.5 s on the
    product's own operands; per launch: time, the rate the same FLOPs would mean, socket power, shader clock."""
    L = load_probe_lib()
    names = {0: "full kernel, pre-touches on", 8: "full kernel, no pre-touches", 4: "no FMA fold (MFMAs accumulate in place)",
             2: "no LDS fragment reads", 1: "no global->LDS copies (ring replayed)", 5: "no copies, no fold",
             3: "no copies, no LDS reads", 7: "MFMA only (no copies, no LDS reads, no fold)"}
    cap = power_cap_w()
    print("power cap %s W; idle reading: %s" % (cap, SmiSampler.read()))
    for tile, (label, wl, N_use) in enumerate((("256x256 tiles", "C3", 16384), ("128x256 tiles", "C2", 2048))):
        seed, kind, M, N, K, _ = WORKLOADS[wl]
        N = N_use
        x, w = make_inputs(torch, kind, M, N, K, seed, dev)
        wq, ws = quantize_weight(torch, w, dev)
        xq, xs = m.act_quant(x)
        xst = xs.t().contiguous()              # [K/128, M]: the layout the tile kernel is given by fp8_gemm
        c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        for const in (False, True):
            a_op, b_op = xq, wq
            if const:       # every operand byte 0x38 (= 1.0): no data toggling in the matrix cores
                a_op = torch.full_like(xq.view(torch.uint8), 0x38).view(torch.float8_e4m3fn)
                b_op = torch.full_like(wq.view(torch.uint8), 0x38).view(torch.float8_e4m3fn)
            bm = 256 if tile == 0 else 128
            print("%s, M=%d N=%d K=%d (%d tiles), %s operands" % (label, M, N, K, ((M + bm - 1) // bm) * ((N + 255) // 256),
                                                               "constant" if const else "quantized N(0,1) x N(0,0.02)"))
            for abl in ((0, 8, 4, 2, 1, 5, 3, 7) if not const else (0, 7)):
                def fn(abl=abl):
                    rc = L.mdy_fp8_gemm_probe(tile, abl, a_op.data_ptr(), xst.data_ptr(), 1, M, b_op.data_ptr(), ws.data_ptr(),
                                              c.data_ptr(), M, N, K, None)
                    if rc != 0:
                        raise RuntimeError("mdy_fp8_gemm_probe(tile=%d, ablation=%d) returned %d" % (tile, abl, rc))
                us, smi = sustained(torch, fn, seconds=1.5)
                smi = smi or {}
                print("  %-46s %8.1f us  %7.1f TFLOP/s-equivalent (%4.1f %% of peak)   %6s W   %5s MHz" % (
                    names[abl], us, 2.0 * M * N * K / us / 1e6, 2.0 * M * N * K / us / 1e6 / PEAK_FP8_TFLOPS * 100,
                    smi.get("socket_power_w"), smi.get("gfx_clock_mhz")), flush=True)
        del x, w, wq, ws, xq, xs, xst, c


def table(torch, m, timer, dev):
    """Per-kernel table for every configuration (stderr)."""
    FP8 = torch.float8_e4m3fn

    def line(name, us, work, unit, peak):
        rate = work / us / (1e6 if unit == "TFLOP/s" else 1e3)
        print("%-46s %9.1f us %10.2f %-8s %5.1f %% of peak" % (name, us, rate, unit, 100 * rate / peak), file=sys.stderr)

    for name, (seed, kind, M, N, K, _) in WORKLOADS.items():
        x, w = make_inputs(torch, kind, M, N, K, seed, dev)
        wq, ws, _, _ = m.quant_weight(w)
        xq, xs = m.act_quant(x)
        line("%s act_quant %dx%d" % (name, M, K), timer.run(lambda: m.act_quant(x), 20)[0], 3.03125 * M * K, "GB/s", PEAK_HBM_GBS)
        line("%s weight_dequant %dx%d" % (name, N, K), timer.run(lambda: m.weight_dequant(wq, ws, out_dtype=torch.bfloat16), 20)[0],
             3.0 * N * K + 4.0 * ((N + 127) // 128) * (K // 128), "GB/s", PEAK_HBM_GBS)
        line("%s fp8_gemm %dx%dx%d" % (name, M, N, K), timer.run(lambda: m.fp8_gemm(xq, xs, wq, ws, out_dtype=torch.bfloat16), 10)[0],
             2.0 * M * N * K, "TFLOP/s", PEAK_FP8_TFLOPS)
    # ---- the shapes the reference publishes numbers for (H800 there; same shapes, this GPU, same cold-cache protocol)
    xr = torch.randn(16384, 4096, device=dev).bfloat16()
    line("ref act_quant 16384x4096 (fp8-benchmark.ipynb:141)", timer.run(lambda: m.act_quant(xr), 20)[0], 3.03125 * 16384 * 4096, "GB/s", PEAK_HBM_GBS)
    del xr
    for (Mr, Nr, Kr) in ((8192, 8192, 8192), (16384, 4096, 1024), (16384, 16384, 4096), (16384, 28672, 7168), (16384, 32768, 8192)):   # test_fp8.ipynb:212-221: M = 16384, N = 4 K
        lin = m.DeepLinear(Kr, Nr, bias=False, dtype=torch.bfloat16, device=dev)
        lin.cache_weight = True
        xg = torch.randn(Mr, Kr, device=dev).bfloat16().requires_grad_(True)
        dy = torch.randn(Mr, Nr, device=dev).bfloat16()
        with torch.no_grad():
            line("ref DeepLinear fwd %dx%dx%d (test_fp8.ipynb:169)" % (Mr, Nr, Kr), timer.run(lambda: lin(xg), 8)[0],
                 2.0 * Mr * Nr * Kr, "TFLOP/s", PEAK_FP8_TFLOPS)

        def fwd_bwd():
            lin.zero_grad(set_to_none=True)
            xg.grad = None
            lin(xg).backward(dy)
        line("ref DeepLinear fwd+bwd %dx%dx%d (test_fp8.ipynb:172)" % (Mr, Nr, Kr), timer.run(fwd_bwd, 6)[0],
             6.0 * Mr * Nr * Kr, "TFLOP/s", PEAK_FP8_TFLOPS)
        del lin, xg, dy
    for d in (4096, 7168, 8192):          # fp8-benchmark.ipynb:351-359 (fwd), :456-464 (bwd): x = [8192, d], W = [d, d]
        lin = m.Fp8Linear(d, d, bias=False, dtype=torch.bfloat16, device=dev, fp8_dtype=torch.float8_e4m3fn)
        xg = torch.randn(8192, d, device=dev).bfloat16().requires_grad_(True)
        dy = torch.randn(8192, d, device=dev).bfloat16()
        with torch.no_grad():
            fwd_us = timer.run(lambda: lin(xg), 8)[0]
        line("ref Fp8Linear fwd 8192x%dx%d (fp8-benchmark.ipynb:351)" % (d, d), fwd_us, 2.0 * 8192 * d * d, "TFLOP/s", PEAK_FP8_TFLOPS)

        def fwd_bwd():
            lin.zero_grad(set_to_none=True)
            xg.grad = None
            lin(xg).backward(dy)
        both_us = timer.run(fwd_bwd, 6)[0]
        line("ref Fp8Linear bwd 8192x%dx%d = fwd+bwd - fwd (:456)" % (d, d), both_us - fwd_us, 4.0 * 8192 * d * d, "TFLOP/s", PEAK_FP8_TFLOPS)
        del lin, xg, dy
    # training-time operators at the C3 shapes (DeepLinear dialect): bytes = 2 in + 1 out + 1 transposed out per element
    seed, kind, M, N, K, _ = WORKLOADS["C3"]
    x, w = make_inputs(torch, kind, M, N, K, seed, dev)
    dy = torch.randn(M, N, device=dev, dtype=torch.bfloat16)
    line("C3 quant_input(train) %dx%d" % (M, K), timer.run(lambda: m.quant_input(x, False), 20)[0], 4.0 * M * K, "GB/s", PEAK_HBM_GBS)
    line("C3 quant_grad_output %dx%d" % (M, N), timer.run(lambda: m.quant_grad_output(dy), 20)[0], 4.0 * M * N, "GB/s", PEAK_HBM_GBS)
    line("C3 quant_weight(train) %dx%d" % (N, K), timer.run(lambda: m.quant_weight(w, False), 20)[0], 4.0 * N * K, "GB/s", PEAK_HBM_GBS)
    lin = m.DeepLinear(K, N, bias=False, dtype=torch.bfloat16, device=dev)
    lin.cache_weight = True
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
    for (M, N, K) in DECODE_SHAPES:
        a = torch.randint(0, 120, (M, K), dtype=torch.uint8, device=dev).view(FP8)
        b = torch.randint(0, 120, (N, K), dtype=torch.uint8, device=dev).view(FP8)
        a_s = torch.rand(M, K // 128, device=dev)
        b_s = torch.rand(N // 128, K // 128, device=dev)

        def many():
            for _ in range(20):
                m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.bfloat16)
        us = timer.run(many, 10, cold=False)[0] / 20
        line("C5 fp8_gemm M=%d N=%d K=%d (warm, back-to-back, Python calls)" % (M, N, K), us, gemm_bytes(M, N, K), "GB/s", PEAK_HBM_GBS)
        us = graph_replay_us(torch, lambda: m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.bfloat16))
        line("   the same inside a replayed HIP graph", us, gemm_bytes(M, N, K), "GB/s", PEAK_HBM_GBS)
    # few rows against a long K (small-batch prefill / large-batch decode): tiles do not fill the GPU, the
    # wrapper hands the library a workspace and the shape is split along K; weight bytes bound these
    for (M, N, K) in ((128, 7168, 16384), (128, 2112, 7168), (256, 7168, 18432), (512, 4096, 7168)):
        a = torch.randint(0, 120, (M, K), dtype=torch.uint8, device=dev).view(FP8)
        b = torch.randint(0, 120, (N, K), dtype=torch.uint8, device=dev).view(FP8)
        a_s = torch.rand(M, K // 128, device=dev)
        b_s = torch.rand((N + 127) // 128, K // 128, device=dev)
        byts = gemm_bytes(M, N, K)
        us = timer.run(lambda: m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.bfloat16), 10)[0]
        line("fp8_gemm M=%d N=%d K=%d (split along K)" % (M, N, K), us, byts, "GB/s", PEAK_HBM_GBS)
        us = timer.run(lambda: m.fp8_gemm(a, a_s, b, b_s, out_dtype=torch.bfloat16), 10, cold="read")[0]
        line("   the same after a read-only cache flush", us, byts, "GB/s", PEAK_HBM_GBS)


if __name__ == "__main__":
    main()
