#!/usr/bin/env python3
"""Benchmark of the transformer-block hot path on one MI355X.

A "step" is one pass of the Flux.1-dev-shape double-stream joint attention block's hot path
(512 text + 4096 image tokens, 24 heads x 128, q6p weights): the six fused-QKV palettized Dense projections
(text M=512, image M=4096; three 3072->3072 weights each) as one grouped launch whose epilogue applies the per-head
QK RMSNorm and RoPE, joint ScaledDotProductAttention over 4608 tokens, and the two palettized output projections as
one grouped launch.  All inputs are resident in HBM before the timed region.  Prints ONE JSON line.

The timed region launches the three kernels one by one with an event before and after each, so the line's
per-kernel times ('kernels_in_step', and 'roofline') are means over the very steps that 'value' is computed from;
'breakdown_consistent' says whether they add up to the step.  The single-kernel legs that follow
('kernels_standalone_loops') repeat one launch back to back and are checked to run on the step's own data.  The CPU
baseline leg runs the oracle on the step's own inputs and compares every output element ('step_checked').
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_F16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0
# HBM-side bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this script, scaled by what the same
# counters read for a 256 MiB device copy (x2.00 and x1.00); the summary is profiles/bench_flux_block_counters.txt
MEASURED_TRAFFIC_BYTES = {"dense_qkv": 3.742e8, "sdpa": 1.327e8}
TRAFFIC_SOURCE = "profiles/bench_flux_block_counters.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script; not measured by this run)"
SDPA_NAME = "sdpa_kernel<128> S=4608 H=24"
QKV_NAME = "dense_qx_kernel<6,256,256> M=4096+512 N=3x3072 K=3072 (fused norm/RoPE epilogue)"
OUT_NAME = "dense_qx_kernel<6,256,256> M=4096+512 N=3072 K=3072 (out projections)"


def other_configs(pkg, torch, np):
    """Single operators of the benchmark configurations other than the Flux 1024 x 1024 block, at their full shapes:
    events around ~100 ms of back-to-back launches each, after ~50 ms of warm-up (weights stay hot in the
    memory-side cache), TFLOP/s from 2 M N K and 4 B H Sq Skv D."""
    dev = "cuda"
    rng = np.random.default_rng(1)

    def timed(fn, n):
        # at least ~50 ms of warm-up and ~100 ms of timed work, so that short kernels are measured at the
        # sustained clock like the step above
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        fn()
        torch.cuda.synchronize()
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        once = max(e0.elapsed_time(e1), 1e-3)
        for _ in range(min(2000, int(50.0 / once))):
            fn()
        n = max(n, min(4000, int(100.0 / once)))
        torch.cuda.synchronize()
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    def synth(N, K, q, nib):
        count = N * K
        pal = (rng.standard_normal(((count + nib - 1) // nib, 1 << q)) * 0.02).astype(np.float16)
        idx = rng.integers(0, 1 << q, size=count, dtype=np.uint8)
        return pkg.QxTensor.from_packed(pkg.pack_qx(q, nib, pal, idx), q, nib, (N, K))

    out = {}

    def record(name, flop, ms):
        out[name] = {"ms": round(ms, 4), "tflops": round(flop / ms / 1e9, 1),
                     "frac_f16_peak": round(flop / ms / 1e9 / PEAK_F16_TFLOPS, 4)}

    def sdpa(name, B, Sq, Skv, H, D, n):
        q = torch.randn(B, Sq, H, D, device=dev).half()
        k = torch.randn(B, Skv, H, D, device=dev).half()
        v = torch.randn_like(k)
        o = torch.empty_like(q)
        record(name, 4.0 * B * H * Sq * Skv * D, timed(lambda: pkg.sdpa_segments([q], [k], [v], 1 / np.sqrt(D), out=o), n))

    def dense(name, M, K, Ns, codec, n):
        qb, nb = pkg.CODEC[codec]
        x = torch.randn(M, K, device=dev).half()
        ws = [synth(N, K, qb, nb) for N in Ns]
        outs = [torch.empty(M, N, device=dev, dtype=torch.float16) for N in Ns]
        record(name, 2.0 * M * K * sum(Ns), timed(lambda: pkg.dense_multi(x, ws, [None] * len(ws), outs=outs), n))

    sdpa("cfg1 SD1.5 self-attention B2 H8 D40 S4096", 2, 4096, 4096, 8, 40, 10)
    sdpa("cfg1 SD1.5 cross-attention B2 H8 D40 Sq4096 Skv77", 2, 4096, 77, 8, 40, 10)
    dense("cfg1 Dense q6p M8192 320->320", 8192, 320, [320], "q6p", 10)
    dense("cfg2 Dense q8p M4608 3072->3x3072", 4608, 3072, [3072] * 3, "q8p", 10)
    dense("cfg2 Dense q8p M4608 3072->3072", 4608, 3072, [3072], "q8p", 10)
    # sensitivity to the palette block size (the per-codec constants are inferred from file sizes, not read from
    # the codec's source): q6p and q8p at every candidate, same shape
    for codec in ("q6p", "q8p"):
        qb = pkg.CODEC[codec][0]
        for nb in (512, 1024, 4096, 16384):
            x = torch.randn(4608, 3072, device=dev).half()
            ws = [synth(3072, 3072, qb, nb) for _ in range(3)]
            outs = [torch.empty(4608, 3072, device=dev, dtype=torch.float16) for _ in range(3)]
            record(f"cfg2 nib sweep Dense {codec} nib{nb} M4608 3072->3x3072", 2.0 * 4608 * 3072 * 9216,
                   timed(lambda: pkg.dense_multi(x, ws, [None] * 3, outs=outs), 10))
    sdpa("cfg4 Flux 2048^2 attention H24 D128 S16896", 1, 16896, 16896, 24, 128, 3)
    dense("cfg4 Dense q4p M16896 3072->3x3072", 16896, 3072, [3072] * 3, "q4p", 3)
    sdpa("cfg5 Wan self-attention H40 D128 S32760", 1, 32760, 32760, 40, 128, 2)
    sdpa("cfg5 Wan cross-attention H40 D128 Sq32760 Skv512", 1, 32760, 512, 40, 128, 3)
    dense("cfg5 Dense q5p M32760 5120->5120", 32760, 5120, [5120], "q5p", 2)
    return out


def occupancy_sweep(pkg, torch, np, sampler_cls):
    """What the card delivers as a function of how many of its compute units a launch keeps busy: attention launches
    of ONE round of workgroups (18 x heads workgroups of 72 key tiles each, 4608 tokens, head size 128) for a growing
    number of heads, the two-round Flux launch, Dense launches of one, one and a half, two and three rounds of
    256 x 256 tiles, and the key-split form of the attention kernel against the unsplit one -- each in a sustained
    loop with the shader clock sampled from sysfs.  Answers whether the idle compute units of a launch's last round
    are throughput lost (they are not, for attention: per-workgroup time grows by a third from half to full
    occupancy while the clock falls by a fifth)."""
    dev = "cuda"
    out = {}

    def timed(fn, flop, name, extra=None):
        fn()
        torch.cuda.synchronize()
        t = time.perf_counter()
        while time.perf_counter() - t < 0.15:
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
        sampler = sampler_cls(torch)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n = 300
        sampler.start()
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        clk = sampler.stop()
        ms = e0.elapsed_time(e1) / n
        out[name] = {"us": round(ms * 1e3, 1), "tflops": round(flop / ms / 1e9, 1),
                     "sclk_mhz_median": None if clk is None else clk["median"]}
        if extra:
            out[name].update(extra)

    S, D = 4608, 128
    saved = os.environ.get("DT_SDPA_KEY_SPLIT")
    for H in (2, 4, 7, 10, 12, 14, 24):
        q, k, v = (torch.randn((1, S, H, D), device=dev).half() for _ in range(3))
        o = torch.empty_like(q)
        os.environ["DT_SDPA_KEY_SPLIT"] = "never"
        timed(lambda: pkg.sdpa_segments([q], [k], [v], 1 / np.sqrt(D), out=o), 4.0 * H * S * S * D,
              f"sdpa {H} heads x 4608 tokens, unsplit", {"workgroups": 18 * H, "key_tiles_each": 72})
        if H in (4, 24):
            os.environ["DT_SDPA_KEY_SPLIT"] = "always"
            timed(lambda: pkg.sdpa_segments([q], [k], [v], 1 / np.sqrt(D), out=o), 4.0 * H * S * S * D,
                  f"sdpa {H} heads x 4608 tokens, key-split into one equal run per compute unit",
                  {"workgroups": 256, "key_tiles_each": round(18 * H * 72 / 256, 1)})
    if saved is None:
        os.environ.pop("DT_SDPA_KEY_SPLIT", None)
    else:
        os.environ["DT_SDPA_KEY_SPLIT"] = saved
    rng = np.random.default_rng(0)

    def synth(N, K, q, nib):
        count = N * K
        pal = (rng.standard_normal(((count + nib - 1) // nib, 1 << q)) * 0.02).astype(np.float16)
        idx = rng.integers(0, 1 << q, size=count, dtype=np.uint8)
        return pkg.QxTensor.from_packed(pkg.pack_qx(q, nib, pal, idx), q, nib, (N, K))

    x = torch.randn(4096, 3072, device=dev).half()
    for kind in ("q6p", "f16"):
        for nt in (12, 16, 24, 32, 48):
            N = 256 * nt
            w = synth(N, 3072, 6, 4096) if kind == "q6p" else pkg.QxTensor.from_f16((torch.randn(N, 3072, device=dev) * 0.02).half())
            y = torch.empty(4096, N, device=dev, dtype=torch.float16)
            timed(lambda: pkg.dense_multi(x, [w], [None], outs=[y]), 2.0 * 4096 * 3072 * N,
                  f"dense {kind} M4096 K3072 N{N}", {"tiles_256x256": 16 * nt, "rounds_of_256": round(16 * nt / 256, 2)})
    return out


def clock_probe(torch, legs, zero_inputs):
    """What the card's clock does under the step's two kernels, and under the vendor library's plain fp16 GEMM of the
    QKV shape for comparison: each leg (name, launch, flop) runs back to back for ~2.5 s on its normal (random)
    inputs and again with all activations zero, while `rocm-smi --showclocks` is sampled from a second thread.
    Same instruction stream both times; the difference is what the data does to the card's power draw."""
    import subprocess
    import threading

    def sclk():
        try:
            out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
            for line in out.splitlines():
                if "sclk" in line and "(" in line:
                    return int(line.split("(")[1].split("Mhz")[0])
        except Exception:
            return None
        return None

    res = {}
    for kname, fn, flop in legs:
        for data in ("random", "zero"):
            if data == "zero":
                zero_inputs(True)
            stop, count = [False], [0]

            def spin():
                while not stop[0]:
                    for _ in range(50):
                        fn()
                    torch.cuda.synchronize()
                    count[0] += 50

            th = threading.Thread(target=spin)
            th.start()
            time.sleep(1.0)
            c0, t0 = count[0], time.perf_counter()
            clocks = []
            for _ in range(3):
                time.sleep(0.4)
                clocks.append(sclk())
            c1, t1 = count[0], time.perf_counter()
            stop[0] = True
            th.join()
            if data == "zero":
                zero_inputs(False)
            ms = (t1 - t0) * 1e3 / max(c1 - c0, 1)
            res[f"{kname}_{data}"] = {"sclk_mhz": clocks, "ms": round(ms, 4), "tflops": round(flop / ms / 1e9, 1)}
    return res


class SclkSampler:
    """Samples the card's shader clock from sysfs (pp_dpm_sclk of the PCI device torch reports for cuda:0; the
    starred level is the current one) every few milliseconds on a thread of its own, between start() and stop()."""

    def __init__(self, torch):
        self.path = None
        self.samples = []
        self._stop = False
        self._thread = None
        try:
            p = torch.cuda.get_device_properties(0)
            bdf = f"{p.pci_domain_id:04x}:{p.pci_bus_id:02x}:{p.pci_device_id:02x}.0"
            cand = f"/sys/bus/pci/devices/{bdf}/pp_dpm_sclk"
            if os.path.exists(cand) and self._read(cand) is not None:
                self.path = cand
        except Exception:
            self.path = None

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                for line in f:
                    if "*" in line:
                        return int(line.split(":")[1].lower().split("mhz")[0])
        except Exception:
            return None
        return None

    def start(self):
        if self.path is None:
            return
        import threading

        self._stop = False

        def run():
            while not self._stop:
                v = self._read(self.path)
                if v is not None:
                    self.samples.append(v)
                time.sleep(0.004)

        self._thread = threading.Thread(target=run, daemon=True)
        self._thread.start()

    def stop(self):
        self._stop = True
        if self._thread is not None:
            self._thread.join()
        if not self.samples:
            return None
        xs = sorted(self.samples)
        return {"source": self.path, "n": len(xs), "min": xs[0], "median": xs[len(xs) // 2], "max": xs[-1]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # One step is ~0.7 ms.  The clock settling is taken care of by --prewarm-ms, not by these two.
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--prewarm-ms", type=float, default=150.0,
                    help="wall time of untimed steps before the counted warm-up, so that the clock has settled "
                         "however few warm-up steps are asked for")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--graph", action="store_true",
                    help="replay the step's three kernels as a HIP graph in the timed region (default: eager launches "
                         "with an event between them, which is no slower on this driver stack and yields the "
                         "per-kernel times from the timed region itself)")
    ap.add_argument("--kernel-iters", type=int, default=100, help="launches per kernel for the per-kernel timings")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--clock-probe", action="store_true",
                    help="also run the two kernels of the step, the plain fp16 Dense and the vendor library's fp16 GEMM of the QKV shape for a few seconds each on random and on all-zero "
                         "activations while sampling the card's clock with rocm-smi (adds 'clock_probe' to the line)")
    ap.add_argument("--occupancy-sweep", action="store_true",
                    help="also time attention and Dense launches that keep a quarter ... all of the compute units busy, "
                         "and the key-split attention kernel against the unsplit one (adds 'occupancy_sweep' to the line)")
    ap.add_argument("--other-configs", action="store_true",
                    help="also time the operators of the other benchmark configurations (SD 1.5, q8p Dense alone, "
                         "Flux at 2048 x 2048 with q4p, Wan 14B with q5p) and add them to the JSON line as 'other_configs'")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    pkg = importlib.import_module("draw-things-community_amd")
    L = pkg.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    assert L.dt_init(0) == 0, "device 0 is not gfx950"
    dev = torch.device("cuda:0")

    # ---------------- workload: Flux joint block, q6p -----------------
    T, HW, H, D = 512, 4096, 24, 128
    S, C = T + HW, H * D
    qbits, nib = pkg.CODEC["q6p"]
    rng = np.random.default_rng(0)

    def synth_weight():
        count = C * C
        nblocks = (count + nib - 1) // nib
        pal = (rng.standard_normal((nblocks, 1 << qbits)) * 0.02).astype(np.float16)
        idx = rng.integers(0, 1 << qbits, size=count, dtype=np.uint8)
        packed = pkg.pack_qx(qbits, nib, pal, idx)
        return pkg.QxTensor.from_packed(packed, qbits, nib, (C, C)), packed

    def f16(shape, std=1.0):
        return torch.from_numpy((rng.standard_normal(shape) * std).astype(np.float16)).to(dev)

    w, packed_host, bias = {}, {}, {}
    for name in ("c_q", "c_k", "c_v", "x_q", "x_k", "x_v", "c_o", "x_o"):
        w[name], packed_host[name] = synth_weight()
        bias[name] = f16((C,), 0.02)
    gamma = {n: (1 + 0.02 * torch.randn(D, device=dev)).half() for n in ("c_q", "c_k", "x_q", "x_k")}
    rot = torch.from_numpy(pkg.Flux1RotaryPositionEmbedding(64, 64, T, channels=D).astype(np.float16)).to(dev)
    ctx = f16((T, C))
    img = f16((HW, C))
    # fused QKV outputs land in one [S, 3, H, D] buffer: text rows first, then image rows
    qkv = torch.empty((S, 3, H, D), dtype=torch.float16, device=dev)
    att = torch.empty((1, S, H, D), dtype=torch.float16, device=dev)
    out_c = torch.empty((T, C), dtype=torch.float16, device=dev)
    out_x = torch.empty((HW, C), dtype=torch.float16, device=dev)
    scale = 1.0 / float(np.sqrt(D))
    qkv2 = qkv.view(S, 3 * C)
    views = lambda lo, hi: [qkv2[lo:hi, i * C:(i + 1) * C] for i in range(3)]
    q4 = qkv[:, 0].unsqueeze(0)
    k4 = qkv[:, 1].unsqueeze(0)
    v4 = qkv[:, 2].unsqueeze(0)
    att2 = att.view(S, C)

    # Q and K leave the projection already RMS-normalised per head and rotated (fused GEMM epilogue)
    epi_c = [pkg.HeadEpilogue(gamma["c_q"], rot, 0, 1e-6, D), pkg.HeadEpilogue(gamma["c_k"], rot, 0, 1e-6, D), None]
    epi_x = [pkg.HeadEpilogue(gamma["x_q"], rot, T, 1e-6, D), pkg.HeadEpilogue(gamma["x_k"], rot, T, 1e-6, D), None]

    def k_qkv_text():
        pkg.dense_multi(ctx, [w["c_q"], w["c_k"], w["c_v"]], [bias["c_q"], bias["c_k"], bias["c_v"]], outs=views(0, T),
                        epilogues=epi_c)

    def k_qkv_image():
        pkg.dense_multi(img, [w["x_q"], w["x_k"], w["x_v"]], [bias["x_q"], bias["x_k"], bias["x_v"]], outs=views(T, S),
                        epilogues=epi_x)

    # the context and image projections are independent Dense ops: enqueued together they share one launch
    def k_qkv():
        pkg.dense_grouped([
            dict(x=img, weights=[w["x_q"], w["x_k"], w["x_v"]], biases=[bias["x_q"], bias["x_k"], bias["x_v"]],
                 outs=views(T, S), epilogues=epi_x),
            dict(x=ctx, weights=[w["c_q"], w["c_k"], w["c_v"]], biases=[bias["c_q"], bias["c_k"], bias["c_v"]],
                 outs=views(0, T), epilogues=epi_c)])

    def k_sdpa():
        pkg.sdpa_segments([q4], [k4], [v4], scale, out=att)

    def k_out():
        pkg.dense_grouped([dict(x=att2[T:], weights=[w["x_o"]], biases=[bias["x_o"]], outs=[out_x]),
                           dict(x=att2[:T], weights=[w["c_o"]], biases=[bias["c_o"]], outs=[out_c])])

    def step():
        k_qkv()
        k_sdpa()
        k_out()

    # inputs of the per-kernel legs, made here so that no host work (and no idle GPU) sits between the timed loops
    x_all = f16((S, C))
    y3 = [torch.empty((S, C), dtype=torch.float16, device=dev) for _ in range(3)]
    wf16 = pkg.QxTensor.from_f16(w["x_q"].dequantize())
    x32 = torch.randn((S, C), dtype=torch.float32, device=dev)
    ln_out = torch.empty((S, C), dtype=torch.float16, device=dev)
    ln_scale, ln_shift = f16((C,), 0.2), f16((C,), 0.2)

    flop_dense = 2.0 * S * C * C * 4          # 6 QKV + 2 out projections, per-stream rows
    flop_sdpa = 4.0 * H * S * S * D
    flop_block = flop_dense + flop_sdpa

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # What the step leaves in its buffers, for the checks below: every single-kernel leg must run on the step's own
    # data (a kernel timed on operands that another leg has degraded -- e.g. Q / K after thousands of in-place
    # normalisation passes -- draws less power, clocks higher and reads faster than it runs in the step).
    step()
    torch.cuda.synchronize()
    sig_ref = {"qkv": float(qkv.float().abs().mean()), "att": float(att.float().abs().mean())}

    def check_step_inputs(leg):
        torch.cuda.synchronize()
        for name, t in (("qkv", qkv), ("att", att)):
            got = float(t.float().abs().mean())
            assert abs(got - sig_ref[name]) <= 0.1 * sig_ref[name], \
                f"{leg}: {name} no longer holds the step's data (mean |x| {got:.4f}, after the step {sig_ref[name]:.4f})"

    # The step is three dependent launches.  By default they go out one by one, with an event between them, so that
    # the timed region itself yields the per-kernel times; --graph replays them as a HIP graph instead (then the
    # per-kernel times come from a second, eager region of the same length right after the timed one).
    run_step, launch_mode, graph = step, "eager (3 launches, events between them)", None
    if args.graph:
        try:
            want = (out_x.clone(), out_c.clone(), att.clone())
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            ok = True
            for _ in range(3):
                out_x.zero_(); out_c.zero_(); att.zero_()
                graph.replay()
                torch.cuda.synchronize()
                ok = ok and all(torch.equal(a_, b_) for a_, b_ in zip((out_x, out_c, att), want))
                step()  # eager work between replays
                torch.cuda.synchronize()
            if ok:
                run_step, launch_mode = graph.replay, "hip graph (3 kernels)"
            else:
                print("graph replays do not reproduce the eager outputs: running eagerly", file=sys.stderr)
        except Exception as e:  # capture not possible: stay eager
            print(f"graph capture failed, running eagerly: {e}", file=sys.stderr)
            torch.cuda.synchronize()

    names3 = ("dense_qkv", "sdpa", "dense_out")

    def step_with_events(ev):
        ev[0].record()
        k_qkv()
        ev[1].record()
        k_sdpa()
        ev[2].record()
        k_out()
        ev[3].record()

    def in_step_times(events):
        """Per-kernel means over a region of eager steps with an event before and after each launch (events on the
        launch stream), and the region's length per step from its first to its last event."""
        acc = [0.0, 0.0, 0.0]
        for ev in events:
            for i in range(3):
                acc[i] += ev[i].elapsed_time(ev[i + 1])
        n = max(len(events), 1)
        per = {names3[i]: acc[i] / n for i in range(3)}
        span = events[0][0].elapsed_time(events[-1][3]) / n if events else 0.0
        return per, span

    def make_events(n):
        return [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(n)]

    # The card needs tens of milliseconds of continuous work before its clock settles (a cold card runs the first
    # launches faster or slower than the sustained rate, depending on where the governor starts): run the step for
    # --prewarm-ms of wall time first, whatever --warmup says.  The counted warm-up and the timed region follow
    # without a gap, and the timed region is exactly --steps steps.
    warm_events = make_events(1)
    step_with_events(warm_events[0])  # first use of timing events: not measured
    torch.cuda.synchronize()
    events = make_events(args.steps)
    sampler = SclkSampler(torch)
    t_pre = time.perf_counter()
    while (time.perf_counter() - t_pre) * 1e3 < args.prewarm_ms:
        for _ in range(20):
            run_step()
        torch.cuda.synchronize()
    prewarm_ms = (time.perf_counter() - t_pre) * 1e3
    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()
    sampler.start()
    t0 = time.perf_counter()
    if graph is None or run_step is step:
        for ev in events:
            step_with_events(ev)
    else:
        for _ in range(args.steps):
            run_step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / max(args.steps, 1)
    if run_step is not step:
        # the graph's replays carry no events: the breakdown comes from an eager region right behind the timed one
        for ev in events:
            step_with_events(ev)
        torch.cuda.synchronize()
    sclk = sampler.stop()
    value = flop_block / (ms_per_step * 1e-3) / 1e12
    in_step, span_ms = in_step_times(events)
    in_step_sum = sum(in_step.values())
    check_step_inputs("after the timed region")

    # ---------------- single-kernel legs (events on the launch stream, back-to-back launches) ----------------
    def time_kernel(fn, iters):
        # ~120 ms of the same kernel first: the clock the card sustains depends on the kernel, and after a lighter
        # kernel (or an idle gap) it takes the power controller tens of milliseconds to come down to it
        fn()
        torch.cuda.synchronize()
        t_w = time.perf_counter()
        while time.perf_counter() - t_w < 0.12:
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters

    # the standalone norm / RoPE pass works in place: it gets a copy of Q and K of its own, never the step's buffer
    qkv_prep = qkv.float().half()  # (elementwise kernels, not a device copy: --copy-calibration counts those)
    qp4, kp4 = qkv_prep[:, 0].unsqueeze(0), qkv_prep[:, 1].unsqueeze(0)

    def k_prep():
        for t4, gc, gx in ((qp4, gamma["c_q"], gamma["x_q"]), (kp4, gamma["c_k"], gamma["x_k"])):
            pkg.qk_norm_rope_(t4[:, :T], gc, 1e-6, True, rot=rot, rot_pos0=0)
            pkg.qk_norm_rope_(t4[:, T:], gx, 1e-6, True, rot=rot, rot_pos0=T)

    it = args.kernel_iters
    ms = {}
    ms["dense_qkv_grouped"] = time_kernel(k_qkv, it)
    ms["dense_qkv_image_M4096"] = time_kernel(k_qkv_image, it)
    ms["dense_qkv_text_M512"] = time_kernel(k_qkv_text, it)
    check_step_inputs("before the attention leg")  # the three legs above rewrite qkv with the step's own values
    ms["sdpa_S4608"] = time_kernel(k_sdpa, it)
    check_step_inputs("before the out-projection leg")
    ms["dense_out_2x"] = time_kernel(k_out, it)
    ms["qk_norm_rope"] = time_kernel(k_prep, it)  # the standalone pass; not part of the step (fused into the QKV epilogue)
    # the "palettized Dense alone" shape of the headline benchmark: M = 4608, 3072 -> 9216 (three weights) and 3072 -> 3072
    ms["dense_qkv_M4608_N9216"] = time_kernel(
        lambda: pkg.dense_multi(x_all, [w["x_q"], w["x_k"], w["x_v"]], [bias["x_q"], bias["x_k"], bias["x_v"]], outs=y3), it)
    ms["dense_out_M4608_N3072"] = time_kernel(
        lambda: pkg.dense_multi(x_all, [w["x_o"]], [bias["x_o"]], outs=[y3[0]]), it)
    ms["dense_plainf16_M4608_N3072"] = time_kernel(
        lambda: pkg.dense_multi(x_all, [wf16], [bias["x_o"]], outs=[y3[0]]), it)

    # the op in front of the block's Dense layers: LayerNorm + adaLN modulation of the fp32 stream (HBM-bound)
    ms["layernorm_modulate"] = time_kernel(lambda: pkg.layernorm_modulate(x32, ln_scale, ln_shift, 1e-6, out=ln_out), max(it, 10))

    # the palettized format on its own: one 3072 x 3072 q6p weight to fp16 (HBM-bound byte work)
    deq_out = torch.empty((C, C), dtype=torch.float16, device=dev)
    ms["depalettize"] = time_kernel(lambda: w["x_o"].dequantize(out=deq_out), max(it, 10))
    deq_bytes = len(packed_host["x_o"]) + 2 * C * C
    check_step_inputs("after the single-kernel legs")

    tf = lambda flop, t_ms: flop / (t_ms * 1e-3) / 1e12
    flop_qkv, flop_out = 2.0 * S * C * 3 * C, 2.0 * S * C * C
    # in-step figures: what each of the step's three launches took inside the timed region
    kernels_in_step = {
        "dense_qkv (context + image in one launch, norm / RoPE epilogue)": {"ms": in_step["dense_qkv"], "tflops": tf(flop_qkv, in_step["dense_qkv"])},
        "sdpa_S4608": {"ms": in_step["sdpa"], "tflops": tf(flop_sdpa, in_step["sdpa"]),
                       "ref_units_G": pkg.ScaledDotProductAttentionInstructionCount(1, H, D, S, S) / 1e9},
        "dense_out (context + image in one launch)": {"ms": in_step["dense_out"], "tflops": tf(flop_out, in_step["dense_out"])},
    }
    # single-kernel legs: the same launch repeated back to back (a different clock and cache state than in the step)
    kernels = {
        "sdpa_S4608": {"ms": ms["sdpa_S4608"], "tflops": tf(flop_sdpa, ms["sdpa_S4608"])},
        "dense_qkv_M4608_N9216_q6p": {"ms": ms["dense_qkv_M4608_N9216"], "tflops": tf(flop_qkv, ms["dense_qkv_M4608_N9216"])},
        "dense_out_M4608_N3072_q6p": {"ms": ms["dense_out_M4608_N3072"], "tflops": tf(flop_out, ms["dense_out_M4608_N3072"])},
        "dense_plainf16_M4608_N3072": {"ms": ms["dense_plainf16_M4608_N3072"], "tflops": tf(flop_out, ms["dense_plainf16_M4608_N3072"])},
        "dense_qkv_image_M4096": {"ms": ms["dense_qkv_image_M4096"], "tflops": tf(2.0 * HW * C * 3 * C, ms["dense_qkv_image_M4096"])},
        "dense_qkv_text_M512": {"ms": ms["dense_qkv_text_M512"], "tflops": tf(2.0 * T * C * 3 * C, ms["dense_qkv_text_M512"])},
        "dense_qkv_text+image_one_launch": {"ms": ms["dense_qkv_grouped"], "tflops": tf(flop_qkv, ms["dense_qkv_grouped"])},
        "dense_out_text+image_one_launch": {"ms": ms["dense_out_2x"], "tflops": tf(flop_out, ms["dense_out_2x"])},
        "qk_norm_rope": {"ms": ms["qk_norm_rope"], "gbs": 2 * 2 * S * C * 2 / (ms["qk_norm_rope"] * 1e-3) / 1e9},
        "layernorm_modulate_M4608_C3072": {"ms": ms["layernorm_modulate"], "gbs": 6 * S * C / (ms["layernorm_modulate"] * 1e-3) / 1e9,
                                           "frac_hbm_peak": 6 * S * C / (ms["layernorm_modulate"] * 1e-3) / 8e12},
    }
    kernels["depalettize_q6p_3072x3072"] = {"ms": ms["depalettize"], "gbs": deq_bytes / (ms["depalettize"] * 1e-3) / 1e9,
                                            "frac_hbm_peak": deq_bytes / (ms["depalettize"] * 1e-3) / 8e12}
    for grp in (kernels, kernels_in_step):
        for k in grp.values():
            if "tflops" in k:
                k["frac_f16_peak"] = round(k["tflops"] / PEAK_F16_TFLOPS, 4)
                k["tflops"] = round(k["tflops"], 2)
            k["ms"] = round(k["ms"], 4)

    # dominant kernel of the step (the longest of its three launches, by the in-step times): roofline against the
    # fp16 MFMA peak, algorithmic FLOPs / mean launch duration inside the timed region
    if in_step["sdpa"] >= in_step["dense_qkv"]:
        dom, dom_flop, dom_ms, dom_tr = SDPA_NAME, flop_sdpa, in_step["sdpa"], "sdpa"
    else:
        dom, dom_flop, dom_ms, dom_tr = QKV_NAME, flop_qkv, in_step["dense_qkv"], "dense_qkv"
    roofline = {
        "kernel": dom, "bound": "mfma", "achieved": round(tf(dom_flop, dom_ms), 2), "peak": PEAK_F16_TFLOPS,
        "unit": "TFLOP/s", "frac": round(tf(dom_flop, dom_ms) / PEAK_F16_TFLOPS, 4),
        "traffic": MEASURED_TRAFFIC_BYTES[dom_tr], "traffic_source": TRAFFIC_SOURCE,
        "flop_per_launch": dom_flop, "avg_launch_ms": round(dom_ms, 4),
        "timing": "mean over the timed region's steps of the time between the events before and after the launch",
        "others": {
            SDPA_NAME: {"achieved": round(tf(flop_sdpa, in_step["sdpa"]), 2),
                        "frac": round(tf(flop_sdpa, in_step["sdpa"]) / PEAK_F16_TFLOPS, 4),
                        "avg_launch_ms": round(in_step["sdpa"], 4), "traffic": MEASURED_TRAFFIC_BYTES["sdpa"]},
            QKV_NAME: {"achieved": round(tf(flop_qkv, in_step["dense_qkv"]), 2),
                       "frac": round(tf(flop_qkv, in_step["dense_qkv"]) / PEAK_F16_TFLOPS, 4),
                       "avg_launch_ms": round(in_step["dense_qkv"], 4), "traffic": MEASURED_TRAFFIC_BYTES["dense_qkv"]},
            OUT_NAME: {"achieved": round(tf(flop_out, in_step["dense_out"]), 2),
                       "frac": round(tf(flop_out, in_step["dense_out"]) / PEAK_F16_TFLOPS, 4),
                       "avg_launch_ms": round(in_step["dense_out"], 4), "traffic": None},
        },
    }

    # ---------------- CPU baseline: the oracle on the step's own inputs, which also checks the step ----------------
    cpu = None
    step_checked = None
    if not args.no_cpu:
        from oracle import oracle

        oracle.build()
        ncores = oracle.C.lib.dto_num_threads()
        # the GPU's outputs for these inputs, from a fresh pass
        step()
        torch.cuda.synchronize()
        got = {"x": out_x.cpu().numpy(), "c": out_c.cpu().numpy()}
        host = lambda t: t.cpu().numpy()
        xs = {"c": host(ctx), "x": host(img)}
        bias_h = {n: host(b) for n, b in bias.items()}
        gam_h = {n: host(g) for n, g in gamma.items()}
        rot_h = host(rot)
        # the whole block at full size: 8 Dense (6 QKV + 2 out, per-stream rows) + attention over all heads; the
        # first pass keeps its outputs and is compared with the GPU's, further passes (until ~12 s of CPU work) only
        # add to the timing
        t_dense = t_sdpa = 0.0
        passes = 0
        while passes < 8 and t_dense + t_sdpa < 12.0:
            t0 = time.perf_counter()
            proj = {s_ + n: oracle.C.dense_qx(xs[s_], packed_host[f"{s_}_{n}"], qbits, nib, C, bias_h[f"{s_}_{n}"])
                    for s_ in "cx" for n in "qkv"}
            t1 = time.perf_counter()
            heads = lambda a: a.reshape(-1, H, D)
            rq = oracle.C.cmul(np.concatenate([oracle.C.rmsnorm(heads(proj["cq"]), gam_h["c_q"], 1e-6),
                                               oracle.C.rmsnorm(heads(proj["xq"]), gam_h["x_q"], 1e-6)]), rot_h)
            rk = oracle.C.cmul(np.concatenate([oracle.C.rmsnorm(heads(proj["ck"]), gam_h["c_k"], 1e-6),
                                               oracle.C.rmsnorm(heads(proj["xk"]), gam_h["x_k"], 1e-6)]), rot_h)
            rv = np.concatenate([heads(proj["cv"]), heads(proj["xv"])])
            t2 = time.perf_counter()
            ratt = oracle.C.sdpa(rq[None], rk[None], rv[None], scale).reshape(S, C)
            t3 = time.perf_counter()
            want_c = oracle.C.dense_qx(np.ascontiguousarray(ratt[:T]), packed_host["c_o"], qbits, nib, C, bias_h["c_o"])
            want_x = oracle.C.dense_qx(np.ascontiguousarray(ratt[T:]), packed_host["x_o"], qbits, nib, C, bias_h["x_o"])
            t4 = time.perf_counter()
            t_dense += (t1 - t0) + (t4 - t3)
            t_sdpa += t3 - t2
            if passes == 0:
                mx_c, rr_c = oracle.err_stats(got["c"], want_c)
                mx_x, rr_x = oracle.err_stats(got["x"], want_x)
                step_checked = {"max_abs": round(float(max(mx_c, mx_x)), 6), "rel_rms": round(float(max(rr_c, rr_x)), 7),
                                "bar": {"max_abs": 2e-2, "rel_rms": 2e-3},
                                "what": "out_x [4096, 3072] and out_c [512, 3072] of the step, every element, against the "
                                        "oracle's op-by-op pass over the same inputs and weights (Dense -> per-head "
                                        "RMSNorm -> cmul -> two-pass softmax attention -> Dense)"}
                step_checked["ok"] = bool(step_checked["max_abs"] <= 2e-2 and step_checked["rel_rms"] <= 2e-3)
            passes += 1
        t_dense /= passes
        t_sdpa /= passes
        t_block = t_dense + t_sdpa
        cpu = {
            "value": round(flop_block / t_block / 1e12, 5), "unit": "TFLOP/s", "cores": int(ncores), "kind": "port",
            "sample": f"oracle (C, OpenMP, {ncores} threads), the whole block at full size on the step's own inputs, mean of "
                      f"{passes} passes: 8 q6p Dense 3072->3072 (512 / 4096 rows, depalettize included, {t_dense:.2f} s) + "
                      f"attention 24 heads x 4608 x 4608 ({t_sdpa:.2f} s); RMSNorm/RoPE run but not timed",
            "ms_per_block": round(t_block * 1e3, 1),
            "dense_gflops": round(flop_dense / t_dense / 1e9, 1), "sdpa_gflops": round(flop_sdpa / t_sdpa / 1e9, 1),
        }

    other = other_configs(pkg, torch, np) if args.other_configs else None
    sweep = occupancy_sweep(pkg, torch, np, SclkSampler) if args.occupancy_sweep else None
    probe = None
    if args.clock_probe:
        saved = {}

        # the library's GEMM (torch.matmul) and this library's plain fp16 Dense on the QKV shape, one problem
        xm = torch.randn(S, C, device=dev).half()
        wm = (torch.randn(3 * C, C, device=dev) * 0.02).half()
        om = torch.empty(S, 3 * C, device=dev, dtype=torch.float16)
        wq16 = [pkg.QxTensor.from_f16(wm[i * C:(i + 1) * C].contiguous()) for i in range(3)]
        om3 = [torch.empty(S, C, device=dev, dtype=torch.float16) for _ in range(3)]

        def zero_inputs(on):
            for name, t in (("img", img), ("ctx", ctx), ("qkv", qkv), ("xm", xm)):
                if on:
                    saved[name] = t.clone()
                    t.zero_()
                else:
                    t.copy_(saved[name])
            torch.cuda.synchronize()

        k_qkv()  # fills qkv for the attention leg
        torch.cuda.synchronize()
        flop_qkv = 2.0 * S * C * 3 * C
        probe = clock_probe(torch, (
            ("dense_qkv", k_qkv, flop_qkv), ("sdpa", k_sdpa, flop_sdpa),
            ("dense_plain_f16_qkv_shape", lambda: pkg.dense_multi(xm, wq16, [None] * 3, outs=om3), flop_qkv),
            ("library_matmul_f16_qkv_shape", lambda: torch.matmul(xm, wm.t(), out=om), flop_qkv)), zero_inputs)

    consistent = abs(in_step_sum - ms_per_step) <= 0.03 * ms_per_step
    line = {
        "metric": "SDPA + palettized-GEMM TFLOP/s (% fp16 peak); ms/block, Flux 4608 tok q6p",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "prewarm_ms": round(prewarm_ms, 1),
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic", "launch": launch_mode,
        "config": {"workload": "Flux.1-dev joint attention block hot path: 512 text + 4096 image tokens, 24x128 heads, "
                               "q6p (nib 4096) weights; 6 QKV Dense (QK RMSNorm/RoPE fused in the epilogue) + SDPA + 2 out-proj Dense",
                   "flop_per_block": flop_block, "frac_f16_peak": round(value / PEAK_F16_TFLOPS, 4)},
        "roofline": roofline, "cpu_baseline": cpu,
        "kernels_in_step": kernels_in_step,
        "in_step_ms_sum": round(in_step_sum, 4), "in_step_ms_first_to_last_event": round(span_ms, 4),
        "breakdown_consistent": bool(consistent),
        "breakdown_rule": "|sum of the three in-step kernel times - ms_per_step| <= 3 % of ms_per_step",
        "sclk_mhz_during_timed_region": sclk,
        "step_checked": step_checked,
        "kernels_standalone_loops": kernels,
    }
    if other is not None:
        line["other_configs"] = other
    if sweep is not None:
        line["occupancy_sweep"] = sweep
    if probe is not None:
        line["clock_probe"] = probe
    print(json.dumps(line))


if __name__ == "__main__":
    main()
