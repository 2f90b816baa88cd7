#!/usr/bin/env python3
"""Benchmark of the FP8 grouped-linear MoE expert path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c3|c4|c5|c1]

One "step" is one pass of the hot path over one synthetic routed batch, inputs already
resident in HBM (quantised operands for the GEMM workloads, bf16 tokens for c5):

  c2 (default)  Mixtral-8x7B-like expert FFN, 8 experts, hidden 4096, gate_up 2x14336 and
                down 14336->4096, 16384 tokens top-2: the six grouped GEMMs of forward, dgrad
                and wgrad of both layers.  metric = fp8 grouped-GEMM TFLOP/s.
  c3            DeepSeek-V3-like, 64 experts, Zipf(1.2) ragged routing with empty groups: forward.
  c4            Qwen-MoE-like, 60 experts, fwd + dgrad + wgrad.
  c5            permute + 1x128 quant and unpermute + combine of 65536 x 7168 tokens (GB/s).
  c1            the small CPU-runnable case.

Prints one JSON line.  ``roofline`` prices the dominant kernel against the published MI355X
peaks (dense fp8 MFMA 5.0 PFLOP/s, HBM 8 TB/s) from HIP-event timings taken on the launch
stream; ``cpu_baseline`` is the reference's PyTorch CPU path (dequantise + per-expert matmul,
or the torch quantise / permute restatement) timed on this host on a bounded sample.
"""
import argparse
import hashlib
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0  # MI355X dense fp8 MFMA, published
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E, published
TILE = 128
# HBM bytes per launch of the dominant kernel come from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this file
# (with --copy-probe: a plain 1 GiB copy reads FETCH_SIZE*2.0 KiB, WRITE_SIZE*1.0 KiB), averaged over that kernel's
# launches of one step.  Counters cannot be read from inside the process, so the figures are recorded in
# profiles/hbm_traffic.json beside the profile summaries they come from, each with the SHA-256 of the kernel sources
# it was measured on: a figure whose sources have changed since is not reported.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
CSRC = os.path.join(ROOT, "atorch_amd", "csrc")


def source_hash(files):
    h = hashlib.sha256()
    for f in files:
        with open(os.path.join(CSRC, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def measured_traffic(key):
    """Bytes per launch recorded for `key`, or None (with the reason) when there is no record for these sources."""
    try:
        rec = json.load(open(TRAFFIC_FILE))[key]
    except (OSError, KeyError, ValueError):
        return None, "no record in profiles/hbm_traffic.json"
    if rec.get("source_sha256") != source_hash(rec["sources"]):
        return None, f"stale: {', '.join(rec['sources'])} changed since {rec.get('profile')} was taken"
    return rec["bytes_per_launch"], rec.get("profile")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3", "c4", "c5", "quant", "module"],
                    help="c1-c5: the configurations of the benchmark; quant: every quantisation kernel of the path at "
                         "the c2 shapes, each beside the streaming probe of its read:write mix")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--operands", default="random", choices=["random", "zeros"],
                    help="GEMM workloads: 'zeros' clears the fp8 codes of the activations and weights after set-up; "
                         "the same launches then draw far less power (not a result, a measurement of the power limit)")
    ap.add_argument("--no-extras", action="store_true",
                    help="default workload only: skip the c5 quant/permute kernels, the clock and the matrix-pipe probe")
    ap.add_argument("--mix-probe", default=None, metavar="R:W[,R:W...]",
                    help="instead of a workload: GB/s of a pure streaming kernel that reads R and writes W 16-byte "
                         "words per unit of work (the ceiling of this GPU for a kernel with that mix of bytes); "
                         "'all' runs every built mix")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch one plain 1 GiB device-to-device copy before the timed region: under "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE its known size calibrates the counters")
    return ap.parse_args()


def copy_probe(dev):
    """A plain copy of known size (1 GiB read + 1 GiB written) for counter calibration."""
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    dst.copy_(src)
    torch.cuda.synchronize()


# ------------------------------------------------------------------------------------------
# probes: shader clock under load, matrix pipes from registers
# ------------------------------------------------------------------------------------------
def clock_under(fn, dev, cycles=5_000_000):
    """Shader clock (GHz) read by a one-wave kernel on a second stream while fn()'s kernels run."""
    from atorch_amd._probes import check, lib

    out = torch.zeros(2, dtype=torch.int64, device=dev)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    fn()
    fn()
    with torch.cuda.stream(side):
        check(lib().aamd_clock_probe(out.data_ptr(), cycles, side.cuda_stream))
    fn()
    fn()
    torch.cuda.synchronize()
    c, r = out.cpu().tolist()
    return round(c / max(r, 1) * 0.1, 3)


MIXES = ["1:0", "0:1", "1:1", "2:1", "1:2", "1:4", "4:1", "8:1", "3:2", "2:2"]


def mix_probe(dev, mixes, stream_mib=512, iters=5):
    """GB/s of the streaming probe for each 'R:W' in mixes: R + W streams of stream_mib MiB each."""
    from atorch_amd._probes import check, lib

    res = {}
    # streams one after the other, the stride kept off the powers of two: words of equal index in
    # different streams would otherwise share their DRAM channel and bank
    stride = (stream_mib << 20) + int(os.environ.get("AAMD_MIX_SKEW", 0x11100))
    for m in mixes:
        r, w = (int(v) for v in m.split(":"))
        src = torch.empty(max(r, 1) * stride, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty(max(w, 1) * stride, dtype=torch.uint8, device=dev)
        units = (stream_mib << 20) // 16
        st = torch.cuda.current_stream().cuda_stream
        call = lambda: check(lib().aamd_stream_probe(src.data_ptr(), dst.data_ptr(), r, w, stride, units, st))  # noqa: E731
        call()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            call()
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / iters
        nbytes = (r + w) * units * 16
        gbs = nbytes / ms / 1e6
        res[m] = {"GB/s": round(gbs, 1), "frac_of_8TBs": round(gbs / PEAK_HBM_GBS, 4), "bytes": nbytes}
        del src, dst
        torch.cuda.empty_cache()
    return res


def mfma_probe(kernels, dev, iters=3000):
    """TFLOP/s of the GEMM's MFMA sequence issued from registers only, for three operand sets."""
    from atorch_amd._probes import check, lib

    nbytes = 64 * 512 * 12 * 32
    g = torch.Generator(device=dev).manual_seed(7)
    q, _ = kernels.tile_quant(torch.randn((nbytes // 128, 128), generator=g, device=dev).to(torch.bfloat16))
    rnd = torch.randint(0, 255, (nbytes,), generator=g, device=dev, dtype=torch.uint8)
    rnd = torch.where((rnd & 0x7F) == 0x7F, rnd ^ 1, rnd)  # no NaN codes
    sets = {"zeros": torch.zeros(nbytes, dtype=torch.uint8, device=dev), "uniform_random_codes": rnd,
            "quantised_normal": q.view(torch.uint8).reshape(-1).contiguous()}  # fmt: skip
    wgs = 1024
    out = torch.empty(wgs * 512, dtype=torch.float32, device=dev)
    cyc = torch.zeros(1, dtype=torch.int64, device=dev)
    res = {}
    for name, ops in sets.items():
        # 1: the block-scale fold (forward, dgrad); 2: per-row scales on both operands (wgrad); 3: the accumulator
        # rescaled instead of a raw product folded (a measured and rejected form of 1)
        for fold in (0, 1, 2, 3):
            st = torch.cuda.current_stream().cuda_stream
            check(lib().aamd_mfma_probe(ops.data_ptr(), fold, iters, wgs, out.data_ptr(), cyc.data_ptr(), st))
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            check(lib().aamd_mfma_probe(ops.data_ptr(), fold, iters, wgs, out.data_ptr(), cyc.data_ptr(), st))
            b.record()
            torch.cuda.synchronize()
            ms = a.elapsed_time(b)
            fl = wgs * 8 * iters * 16 * 131072.0
            key = name + ("", "+fold", "+fold_per_row", "+rescaled_accumulator")[fold]
            res[key] = {"TFLOP/s": round(fl / ms / 1e9, 1)}
            if fold in (1, 2):
                # with the fold the two waves of a SIMD alternate on its pipe, so the probed wave runs for the
                # whole of its round (one of wgs/256): its cycle count over that time is the shader clock
                res[key]["sclk_ghz"] = round(int(cyc.item()) / (ms * 1e6 / (wgs / 256)), 3)
            if fold == 1:
                res[key]["board_power"] = power_under(
                    lambda: check(lib().aamd_mfma_probe(ops.data_ptr(), 1, iters, wgs, out.data_ptr(), cyc.data_ptr(), st)), 1.0)
    return res


def loop_probe(dev, iters=2000):
    """One step of the 256 x 256 GEMM loop as an instruction sequence on private data (zero codes): shader
    cycles per step as one wave sees them (2048 of them are MFMA work) and TFLOP/s by the clock, with
    cache-resident loads, with loads that stream shared panels, and with the GEMM's barriers and waits."""
    from atorch_amd._probes import check, lib

    panels = torch.zeros(16 * (96 << 20), dtype=torch.uint8, device=dev)  # 1.5 GiB: more than the last-level cache
    out = torch.empty(256 * 512, dtype=torch.float32, device=dev)
    cyc = torch.zeros(1, dtype=torch.int64, device=dev)
    res = {}
    for name, stream_panels, nbytes in (("resident_loads", 0, 96 << 20), ("streaming_panels_96MiB", 1, 96 << 20),
                                        ("streaming_panels_1.5GiB", 1, panels.numel()),
                                        ("streaming_panels_1.5GiB_barriers_and_waits", 2, panels.numel())):
        st = torch.cuda.current_stream().cuda_stream
        call = lambda: check(lib().aamd_loop_probe(panels.data_ptr(), nbytes, stream_panels, iters,  # noqa: E731
                                                   out.data_ptr(), cyc.data_ptr(), st))
        call()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        call()
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b)
        c = int(cyc.item()) / iters
        res[name] = {"cycles_per_step": round(c, 1), "mfma_share_of_cycles": round(2048.0 / c, 4),
                     "TFLOP/s": round(256 * 8 * iters * 16 * 131072.0 / ms / 1e9, 1)}  # fmt: skip
    return res


# ------------------------------------------------------------------------------------------
# synthetic routed batches (seeds fixed; generated on the device, nothing is read from disk)
# ------------------------------------------------------------------------------------------
def routing(T, E, k, dev, zipf_s=None, seed=2):
    g = torch.Generator(device=dev).manual_seed(seed)
    if zipf_s is None:
        logits = torch.randn(T, E, generator=g, device=dev)
    else:
        p = torch.arange(1, E + 1, dtype=torch.float32, device=dev).pow(-zipf_s)
        u = torch.rand(T, E, generator=g, device=dev).clamp_min(1e-30)
        logits = p.log() - torch.log(-torch.log(u))  # Gumbel top-k = sampling without replacement
    vals, idx = torch.topk(logits, k, dim=1)
    return idx, torch.softmax(vals, dim=1).to(torch.bfloat16)


def randn(shape, dev, std, seed, dtype=torch.bfloat16):
    g = torch.Generator(device=dev).manual_seed(seed)
    out = torch.empty(shape, dtype=dtype, device=dev)
    # fill in row chunks to bound the fp32 temporary
    rows = shape[0]
    step = max(1, (1 << 28) // max(1, out[0].numel()))
    for r in range(0, rows, step):
        n = min(step, rows - r)
        out[r : r + n] = (torch.randn((n, *shape[1:]), generator=g, device=dev) * std).to(dtype)
    return out


def student_t(shape, dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    out = torch.empty(shape, dtype=torch.bfloat16, device=dev)
    step = max(1, (1 << 26) // shape[1])
    for r in range(0, shape[0], step):
        n = min(step, shape[0] - r)
        z = torch.randn((n, shape[1]), generator=g, device=dev)
        chi = torch.randn((n, shape[1], 3), generator=g, device=dev).pow(2).sum(-1)
        out[r : r + n] = (z / torch.sqrt(chi / 3)).to(torch.bfloat16)
    return out


def host_threads():
    """Threads for the CPU baseline: the box's CPU share (OMP_NUM_THREADS when set, else at most 16)."""
    n = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or min(os.cpu_count() or 1, 16)
    torch.set_num_threads(n)
    return n


class PowerSampler:
    """Board power (W) while a region runs, read from the amdgpu hwmon file every 25 ms by a thread of this
    process; the package power cap is read beside it.  The grouped GEMMs of the benchmark run at that cap:
    their clock, and with it their throughput, is what the power management leaves them."""

    def __init__(self):
        import glob

        hw = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))
        self.file = next((os.path.join(h, n) for h in hw for n in ("power1_input", "power1_average")
                          if os.path.exists(os.path.join(h, n))), None)  # fmt: skip
        self.cap = None
        for h in hw:
            try:
                self.cap = int(open(os.path.join(h, "power1_cap")).read()) / 1e6
                break
            except (OSError, ValueError):
                pass
        self.vals = []

    def __enter__(self):
        import threading

        self._stop = False

        def poll():
            while not self._stop and self.file:
                try:
                    self.vals.append(int(open(self.file).read()) / 1e6)
                except (OSError, ValueError):
                    return
                time.sleep(0.025)

        self._t = threading.Thread(target=poll, daemon=True)
        self._t.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        self._t.join()
        return False

    def summary(self):
        if not self.vals:
            return None
        v = self.vals[len(self.vals) // 4 :] or self.vals  # the first samples still see the ramp
        return {"mean_W": round(sum(v) / len(v), 1), "max_W": round(max(v), 1), "cap_W": self.cap, "samples": len(v)}


def power_under(fn, seconds=1.5):
    """Board power while fn() is launched back to back for `seconds`."""
    ps = PowerSampler()
    if ps.file is None:
        return None
    fn()
    torch.cuda.synchronize()
    with ps:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
    return ps.summary()


class Timer:
    """HIP events on torch's current stream, which is the stream every kernel here is launched on."""

    def __init__(self):
        self.pairs = []

    def region(self):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        self.pairs.append((a, b))
        return a, b

    def ms(self):
        return [a.elapsed_time(b) for a, b in self.pairs]

    def mean(self):
        ms = self.ms()
        return sum(ms) / len(ms)

    def median(self):
        return statistics.median(self.ms())


# ------------------------------------------------------------------------------------------
# GEMM workloads
# ------------------------------------------------------------------------------------------
class Layer:
    """One grouped linear's resident operands: fp8 codes and scales of x, w, dy (+ transposes)."""

    def __init__(self, kernels, M, K, N, E, goff, dev, seed, backward):
        x = randn((M, K), dev, 1.0, seed)
        w = randn((E, N, K), dev, 0.02, seed + 1)
        self.M, self.K, self.N, self.E = M, K, N, E
        self.goff = goff
        if backward:
            self.qx, self.sx, self.qx_t, self.sx_t = kernels.tile_quant_dual_grouped(x, goff, E, blocked=True)
            dy = randn((M, N), dev, 1e-2, seed + 2)
            self.qdy, self.sdy, self.qdy_t, self.sdy_t = kernels.tile_quant_dual_grouped(dy, goff, E, blocked=True)
            del dy
            self.qw, self.sw, self.qw_t, self.sw_t = kernels.block_quant_batched(w, return_transpose=True)
            self.dx = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
            self.dw = torch.empty((E, N, K), dtype=torch.float32, device=dev)
        else:
            self.qx, self.sx = kernels.tile_quant(x)
            self.qw, self.sw, _, _ = kernels.block_quant_batched(w)
        del x, w
        self.y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        self.flops = 2.0 * M * N * K

    def fwd(self, kernels):
        kernels.grouped_gemm_nt(self.qx, self.sx, self.qw, self.sw, self.goff, out=self.y)

    def dgrad(self, kernels):
        kernels.grouped_gemm_nt(self.qdy, self.sdy, self.qw_t, self.sw_t, self.goff, out=self.dx)

    def wgrad(self, kernels):
        kernels.grouped_gemm_wgrad(self.qdy_t, self.sdy_t, self.qx_t, self.sx_t, self.goff, out=self.dw)


GEMM_WORKLOADS = {
    # name: (E, T, topk, zipf, [(K, N), ...], backward, description)
    "c1": (4, 2048, 1, None, [(512, 1024)], False, "4 experts, 512->1024, 2048 tokens top-1, forward"),
    "c2": (8, 16384, 2, None, [(4096, 28672), (14336, 4096)], True,
           "Mixtral-8x7B-like expert FFN: 8 experts, 4096->2x14336 and 14336->4096, 16384 tokens top-2, "
           "fwd+dgrad+wgrad"),
    "c3": (64, 8192, 8, 1.2, [(7168, 4096), (2048, 7168)], False,
           "DeepSeek-V3-like: 64 experts, 7168->4096 and 2048->7168, 8192 tokens top-8 Zipf(1.2), forward"),
    "c4": (60, 32768, 4, None, [(2048, 2816), (1408, 2048)], True,
           "Qwen-MoE-like: 60 experts, 2048->2816 and 1408->2048, 32768 tokens top-4, fwd+dgrad+wgrad"),
}  # fmt: skip


def run_gemm(args, kernels, dev, workload=None, steps=None, warmup=None, cpu_baseline=True, probes=True):
    workload = workload or args.workload
    steps = steps or args.steps
    warmup = args.warmup if warmup is None else warmup
    E, T, k, zipf, shapes, backward, desc = GEMM_WORKLOADS[workload]
    idx, _ = routing(T, E, k, dev, zipf_s=zipf)
    if zipf is not None:
        # the ragged configuration asks for empty groups: when the draw has none, the rarest expert's
        # few tokens go to expert 0
        cnt = torch.bincount(idx.view(-1), minlength=E)
        if int((cnt == 0).sum()) == 0:
            idx = torch.where(idx == cnt.argmin(), torch.zeros_like(idx), idx)
    _, _, goff = kernels.moe_preprocess(idx, E, want_sorted=False)
    M = T * k
    layers = [Layer(kernels, M, K, N, E, goff, dev, 10 * i, backward) for i, (K, N) in enumerate(shapes)]
    counts = (goff[1:] - goff[:-1]).cpu()
    if args.operands == "zeros":
        for L in layers:
            for name in ("qx", "qw", "qx_t", "qw_t", "qdy", "qdy_t"):
                t = getattr(L, name, None)
                if t is not None:
                    t.view(torch.uint8).zero_()
    torch.cuda.synchronize()

    nt_timer, wg_timer = Timer(), Timer()

    def step(timed):
        for L in layers:
            if timed:
                a, b = nt_timer.region()
                a.record()
            L.fwd(kernels)
            if timed:
                b.record()
        if backward:
            for L in layers:
                if timed:
                    a, b = nt_timer.region()
                    a.record()
                L.dgrad(kernels)
                if timed:
                    b.record()
                    a, b = wg_timer.region()
                    a.record()
                L.wgrad(kernels)
                if timed:
                    b.record()

    for _ in range(warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step(True)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0

    passes = 3 if backward else 1
    flops_step = passes * sum(L.flops for L in layers)
    ms_step = dt * 1e3 / steps
    tflops = flops_step / (ms_step * 1e-3) / 1e12

    # dominant kernel: the forward / dgrad grouped GEMM (4 of the 6 launches of a step)
    n_nt = len(layers) * (2 if backward else 1)
    nt_flops = sum(L.flops for L in layers) * (2 if backward else 1) / n_nt  # per launch, averaged
    nt_avg_ms = nt_timer.mean()
    nt_tflops = nt_flops / (nt_avg_ms * 1e-3) / 1e12
    # per-launch times of one step's launches differ by shape: the median is taken over steps of the per-step mean
    per_step = [sum(nt_timer.ms()[i * n_nt : (i + 1) * n_nt]) / n_nt for i in range(steps)]
    nt_med_ms = statistics.median(per_step)
    traffic, traffic_src = measured_traffic("grouped_gemm_" + workload)
    roofline = {
        "kernel": "grouped_gemm_kernel<kRaggedRows> (forward and dgrad)",
        "bound": "mfma",
        "achieved": round(nt_tflops, 2),
        "peak": PEAK_FP8_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(nt_tflops / PEAK_FP8_TFLOPS, 4),
        "traffic": traffic,
        "traffic_source": traffic_src,
        "avg_launch_ms": round(nt_avg_ms, 4),
        "median_launch_ms": round(nt_med_ms, 4),
        "achieved_by_median": round(nt_flops / (nt_med_ms * 1e-3) / 1e12, 2),
        "flop_per_launch": nt_flops,
    }
    extras = {"tokens_per_expert_min_max": [int(counts.min()), int(counts.max())],
              "empty_groups": int((counts == 0).sum()), "operands": args.operands}
    if probes:
        extras["sclk_ghz_under_forward_gemm"] = clock_under(lambda: layers[0].fwd(kernels), dev)
        if not args.no_extras:
            extras["board_power_under_forward_gemm"] = power_under(lambda: layers[0].fwd(kernels))
            if backward:
                extras["board_power_under_wgrad_gemm"] = power_under(lambda: layers[0].wgrad(kernels))
    if backward:
        wg_avg = wg_timer.mean()
        wg_flops = sum(L.flops for L in layers) / len(layers)
        n_wg = len(layers)
        wg_med = statistics.median([sum(wg_timer.ms()[i * n_wg : (i + 1) * n_wg]) / n_wg for i in range(steps)])
        extras["wgrad_kernel"] = {"avg_launch_ms": round(wg_avg, 4), "median_launch_ms": round(wg_med, 4),
                                  "achieved_tflops": round(wg_flops / (wg_avg * 1e-3) / 1e12, 2),
                                  "frac": round(wg_flops / (wg_avg * 1e-3) / 1e12 / PEAK_FP8_TFLOPS, 4),
                                  "output": "fp32 (a main_grad buffer)"}
        if not args.no_extras:
            # the same launches writing bf16, the dtype of the parameters, beside fp32: each launch repeated back to
            # back (five timed after two untimed), which at the power cap runs a few per cent slower than inside
            # the step, where the launches around it draw less
            b2b = {}
            for name, dt in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
                t = Timer()
                for L in layers:
                    dw = torch.empty((L.E, L.N, L.K), dtype=dt, device=dev)
                    for i in range(7):
                        a, b = t.region() if i >= 2 else (None, None)
                        if a is not None:
                            a.record()
                        kernels.grouped_gemm_wgrad(L.qdy_t, L.sdy_t, L.qx_t, L.sx_t, L.goff, out=dw)
                        if b is not None:
                            b.record()
                    del dw
                torch.cuda.synchronize()
                b2b[name] = {"avg_launch_ms": round(t.mean(), 4),
                             "frac": round(wg_flops / (t.mean() * 1e-3) / 1e12 / PEAK_FP8_TFLOPS, 4)}
            extras["wgrad_kernel"]["back_to_back_by_output_dtype"] = b2b

    if workload == "c2" and probes and not args.no_extras and args.operands == "random":
        extras["forward_gemm_by_operand_data"] = operand_data_probe(kernels, layers[0], dev)

    cpu = None
    if cpu_baseline and not args.no_cpu_baseline and args.operands == "random":
        cpu = cpu_gemm_baseline(layers[0], counts)
    return {
        "metric": "fp8 grouped-GEMM TFLOPS (fwd+bwd)" if backward else "fp8 grouped-GEMM TFLOPS (fwd)",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "ms_per_step": round(ms_step, 4),
        "dtype": "fp8",
        "config": {"workload": f"{workload}: {desc}", "rows": M, "experts": E,
                   "flop_per_step": flops_step, "frac_of_fp8_peak": round(tflops / PEAK_FP8_TFLOPS, 4)},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "extras": extras,
    }  # fmt: skip


def module_step(kernels, dev, steps=5):
    """Forward + backward of the c2 expert MLP through the Python mirror (grouped_mlp_swiglu: quantisers, the fused
    SwiGLU kernels and the six grouped GEMMs, host code included), the weights' codes cached as between the
    microbatches of a step (quantized_grouped_linear.py:103-134)."""
    from atorch_amd.expert_mlp import grouped_mlp_swiglu
    from atorch_amd.quantization import WeightCodeCache

    E, T, k, H, F = 8, 16384, 2, 4096, 14336
    idx, _ = routing(T, E, k, dev)
    _, _, goff = kernels.moe_preprocess(idx, E, want_sorted=False)
    counts = goff[1:] - goff[:-1]
    M = T * k
    x = randn((M, H), dev, 1.0, 1).requires_grad_(True)
    w1 = randn((E, 2 * F, H), dev, 0.02, 2).requires_grad_(True)
    w2 = randn((E, F, H), dev, 0.02, 3).requires_grad_(True)
    dy = randn((M, H), dev, 1e-2, 4)
    cache = WeightCodeCache()

    def one(first):
        out = grouped_mlp_swiglu(x, w1, w2, counts, is_first_microbatch=first, weight_cache=cache)
        out.backward(dy)
        x.grad = w1.grad = w2.grad = None

    one(True)
    one(False)
    torch.cuda.synchronize()
    res = {}
    for name, first in (("cached_weight_codes", False), ("weights_quantised_every_call", None)):
        t = Timer()
        for _ in range(steps):
            a, b = t.region()
            a.record()
            one(first)
            b.record()
        torch.cuda.synchronize()
        fl = 3 * 2.0 * M * (2 * F * H + F * H)
        res[name] = {"ms_per_step": round(t.mean(), 3), "median_ms": round(t.median(), 3),
                     "TFLOP/s": round(fl / t.mean() / 1e9, 1), "frac_of_fp8_peak": round(fl / t.mean() / 1e9 / PEAK_FP8_TFLOPS, 4)}  # fmt: skip
    res["what"] = "grouped_mlp_swiglu forward + backward at the c2 shapes: 2 + 3 quantiser launches and 6 grouped GEMMs"
    del x, w1, w2, dy, cache
    torch.cuda.empty_cache()
    return res


def operand_data_probe(kernels, layer, dev, iters=5):
    """The first layer's forward launch with its own codes and with all-zero codes (same scales, sizes and
    addresses pattern): the instruction stream is the same, what differs is the switching activity of the
    matrix pipes, which the GPU's power management answers with the shader clock."""
    res = {}
    zx, zw = torch.zeros_like(layer.qx.view(torch.uint8)), torch.zeros_like(layer.qw.view(torch.uint8))
    out = torch.empty_like(layer.y)  # the layer's own output stays as the timed steps left it
    for name, qx, qw in (("benchmark_codes", layer.qx, layer.qw), ("zero_codes", zx.view(layer.qx.dtype), zw.view(layer.qw.dtype))):
        fn = lambda: kernels.grouped_gemm_nt(qx, layer.sx, qw, layer.sw, layer.goff, out=out)  # noqa: E731
        fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / iters
        tf = layer.flops / ms / 1e9
        res[name] = {"TFLOP/s": round(tf, 1), "frac": round(tf / PEAK_FP8_TFLOPS, 4), "avg_launch_ms": round(ms, 4),
                     "sclk_ghz": clock_under(fn, dev), "board_power": power_under(fn, 1.0)}  # fmt: skip
    del zx, zw, out
    return res


def cpu_gemm_baseline(layer, counts):
    """The reference's PyTorch CPU path (dequantise + per-expert matmul) on a bounded sample of
    the first layer's forward: as many leading experts as about 1.6e13 FLOP cover (about 10 s
    of host time; all of them at the default workload)."""
    from oracle import oracle as O

    K, N = layer.K, layer.N
    budget, rows, ne = 1.6e13, 0, 0
    for c in counts.tolist():
        if ne > 0 and 2.0 * (rows + c) * N * K > budget:
            break
        rows += c
        ne += 1
    if rows == 0:
        return None
    qx = layer.qx[:rows].view(torch.uint8).cpu()
    sx = layer.sx[:rows].cpu()
    qw = layer.qw[:ne].view(torch.uint8).cpu()
    sw = layer.sw[:ne].cpu()
    splits = counts[:ne].tolist()
    cores = host_threads()
    t0 = time.perf_counter()
    ref = O.torch_grouped_gemm_dequant(qx, sx, qw, sw, splits)
    dt = time.perf_counter() - t0
    # the sample doubles as an end-to-end check of the GPU result
    got = layer.y[:rows].float().cpu()
    err = float(((got - ref.float()).abs().max()) / ref.float().abs().max().clamp_min(1e-30))
    fl = 2.0 * rows * N * K
    return {"value": round(fl / dt / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"forward of layer 0, first {ne} experts ({rows} rows, {fl:.3e} FLOP, {dt:.1f} s): "
                      "torch CPU dequantise + per-expert fp32 matmul",
            "max_err_vs_gpu_over_max": round(err, 5)}  # fmt: skip


# ------------------------------------------------------------------------------------------
# c5: quant / permute kernels
# ------------------------------------------------------------------------------------------
def run_c5(args, kernels, dev, cpu_baseline=True, mixes_too=None):
    T, H, E, k = 65536, 7168, 64, 8
    x = student_t((T, H), dev, seed=0)
    idx, probs = routing(T, E, k, dev)
    sorted_idx, row_map, goff = kernels.moe_preprocess(idx, E)
    M = T * k
    y = randn((M, H), dev, 1.0, seed=5)
    torch.cuda.synchronize()
    q1 = 1 + 4 / TILE
    pq_bytes = T * H * 2 + M * H + M * (H // TILE) * 4 + M * 4
    uc_bytes = M * H * 2 + T * k * 2 + M * 4 + T * H * 2
    tq_bytes = M * H * 2 + M * H + M * (H // TILE) * 4
    t_pq, t_uc, t_tq, t_pre = Timer(), Timer(), Timer(), Timer()

    def step(timed):
        for timer, fn in (
            (t_pre, lambda: kernels.moe_preprocess(idx, E, want_sorted=False)),
            (t_pq, lambda: kernels.permute_tile_quant(x, row_map, k, M)),
            (t_uc, lambda: kernels.unpermute_combine(y, row_map, probs, T, k)),
            (t_tq, lambda: kernels.tile_quant(y)),
        ):
            if timed:
                a, b = timer.region()
                a.record()
            fn()
            if timed:
                b.record()

    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(True)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_step = dt * 1e3 / args.steps

    def entry(nbytes, timer):
        ms, med = timer.mean(), timer.median()
        return {"GB/s": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                "avg_launch_ms": round(ms, 4), "median_launch_ms": round(med, 4), "bytes_per_launch": nbytes}  # fmt: skip

    pq, uc, tq = entry(pq_bytes, t_pq), entry(uc_bytes, t_uc), entry(tq_bytes, t_tq)
    total_gbs = (pq_bytes + uc_bytes) / ((t_pq.mean() + t_uc.mean()) * 1e-3) / 1e9

    # the training form: row-wise and transposed codes of the permuted rows.  Separate kernels write the permuted
    # bf16 rows and read them back; the fused kernel quantises each permuted row straight from its token's row.
    del y
    torch.cuda.empty_cache()
    t_sep, t_fused = Timer(), Timer()
    for i in range(2 + 5):
        for timer, fn in (
            (t_sep, lambda: kernels.tile_quant_dual_grouped(kernels.permute_rows(x, row_map, k, M), goff, E, blocked=True)),
            (t_fused, lambda: kernels.permute_tile_quant_dual_grouped(x, sorted_idx, k, goff, E, blocked=True)),
        ):
            a, b = timer.region() if i >= 2 else (None, None)
            if a is not None:
                a.record()
            out = fn()
            if b is not None:
                b.record()
            del out
    torch.cuda.synchronize()
    out_bytes = int(2 * M * H * q1)
    dual = {
        "permute_rows + quant_dual_grouped": {
            "ms": round(t_sep.mean(), 4), "bytes_moved": T * H * 2 + 2 * M * H * 2 + out_bytes},
        "permute_quant_dual_grouped (fused)": {
            "ms": round(t_fused.mean(), 4), "bytes_moved": M * H * 2 + out_bytes,
            "bytes_saved": T * H * 2 + M * H * 2,
            "GB/s_of_bytes_moved": round((M * H * 2 + out_bytes) / t_fused.mean() / 1e6, 1),
            "frac_of_bytes_moved": round((M * H * 2 + out_bytes) / t_fused.mean() / 1e6 / PEAK_HBM_GBS, 4)},
        "note": "bytes_moved counts every token row once per top-k copy (the gather re-reads a token for each of its "
                "experts' tiles; 0.94 GB of tokens do not stay in the 256 MB last-level cache between them)",
    }  # fmt: skip

    cpu = None
    if cpu_baseline and not args.no_cpu_baseline:
        cpu = cpu_quant_baseline(x, idx)
    mixes = None
    want_mixes = (args.workload == "c5" and not args.no_extras) if mixes_too is None else mixes_too
    if want_mixes:
        # what plain streaming kernels reach with each kernel's ratio of bytes read to bytes written
        torch.cuda.empty_cache()
        pr = mix_probe(dev, ["1:4", "8:1", "2:1"])
        mixes = {"permute_quant (1:4)": pr["1:4"]["GB/s"], "unpermute_combine (8:1)": pr["8:1"]["GB/s"],
                 "tile_quant_plain (2:1)": pr["2:1"]["GB/s"]}  # fmt: skip
    traffic, traffic_src = measured_traffic("permute_quant_c5")
    return {
        "metric": "quant/permute HBM GB/s (permute+1x128 quant and unpermute+combine)",
        "value": round(total_gbs, 1),
        "unit": "GB/s",
        "ms_per_step": round(ms_step, 4),
        "dtype": "fp8",
        "config": {"workload": "c5: 65536 tokens x 7168 bf16 Student-t(3), top-8 into 64 experts; "
                               "fused permute + 1x128 quant, and unpermute + weighted combine",
                   "rows": M, "experts": E},
        "roofline": {"kernel": "quant_1x128_kernel<bf16, scatter> (permute + quant)", "bound": "hbm",
                     "achieved": pq["GB/s"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": pq["frac"], "traffic": traffic, "traffic_source": traffic_src,
                     "avg_launch_ms": pq["avg_launch_ms"], "median_launch_ms": pq["median_launch_ms"],
                     "bytes_per_launch": pq_bytes},
        "cpu_baseline": cpu,
        "extras": {
            "unpermute_combine": uc,
            "tile_quant_plain": tq,
            "permute_quant_dual (training form)": dual,
            "moe_preprocess_ms": round(t_pre.mean(), 4),
            "mix_probe_GB/s": mixes,
        },
    }  # fmt: skip


def cpu_quant_baseline(x, idx):
    """torch CPU restatement of permute + per-row quantise on the first 32768 tokens (half the
    batch), in chunks of 4096 tokens to bound the fp32 temporaries."""
    from oracle import oracle as O

    n, chunk = 32768, 4096
    xs = x[:n].cpu()
    ids = idx[:n].cpu()
    cores = host_threads()
    t0 = time.perf_counter()
    for lo in range(0, n, chunk):
        p, _ = O.torch_permute(xs[lo : lo + chunk], ids[lo : lo + chunk])
        q, s = O.torch_tile_quant(p)
    dt = time.perf_counter() - t0
    k = ids.shape[1]
    H = xs.shape[1]
    nbytes = n * H * 2 + n * k * H + n * k * (H // TILE) * 4 + n * k * 4
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"first {n} tokens: torch CPU permute (argsort + index_select) then amax/448, divide, "
                      f"cast ({dt:.2f} s)"}  # fmt: skip


# ------------------------------------------------------------------------------------------
# quant: the quantisation kernels of the expert MLP at the c2 shapes
# ------------------------------------------------------------------------------------------
def run_quant(args, kernels, dev, steps=None, with_probe=True):
    steps = steps or args.steps
    E, T, k, F = 8, 16384, 2, 14336
    idx, _ = routing(T, E, k, dev)
    _, _, goff = kernels.moe_preprocess(idx, E, want_sorted=False)
    M = T * k
    q1 = 1 + 4 / TILE  # bytes written per element by one 1x128 quantisation (code + its share of the scale)
    x = randn((M, F), dev, 1.0, 1)
    fc1 = randn((M, 2 * F), dev, 1.0, 2)
    dh = randn((M, F), dev, 1e-2, 3)
    w = randn((E, 2 * F, 4096), dev, 0.02, 4)
    # name: (call, algorithmic bytes, read:write mix of the streaming probe in equal-sized streams)
    cases = {
        "quant_1x128": (lambda: kernels.tile_quant(x), M * F * (2 + q1), "2:1"),
        "quant_1x128_dual_grouped": (lambda: kernels.tile_quant_dual_grouped(x, goff, E, blocked=True), M * F * (2 + 2 * q1), "1:1"),
        "swiglu_quant_1x128": (lambda: kernels.swiglu_tile_quant(fc1), M * F * (4 + q1), "4:1"),
        "swiglu_quant_1x128_dual_grouped": (lambda: kernels.swiglu_tile_quant_dual_grouped(fc1, goff, E, blocked=True),
                                            M * F * (4 + 2 * q1), "2:1"),
        "swiglu_bwd_quant_1x128_dual_grouped": (lambda: kernels.swiglu_bwd_tile_quant_dual_grouped(dh, fc1, goff, E, blocked=True),
                                                M * F * (6 + 4 * q1), "3:2"),
        "gelu_quant_1x128_dual_grouped": (lambda: kernels.gelu_tile_quant_dual_grouped(x, goff, E, blocked=True),
                                          M * F * (2 + 2 * q1), "1:1"),
        "gelu_bwd_quant_1x128_dual_grouped": (lambda: kernels.gelu_tile_quant_dual_grouped(x, goff, E, dh=dh, blocked=True),
                                              M * F * (4 + 2 * q1), "2:1"),
        "quant_128x128": (lambda: kernels.block_quant_batched(w), w.numel() * 3, "2:1"),
        "quant_128x128_with_transpose": (lambda: kernels.block_quant_batched(w, return_transpose=True),
                                         w.numel() * 4, "1:1"),
    }  # fmt: skip
    res, tot_b, tot_ms = {}, 0.0, 0.0
    for name, (fn, nbytes, mix) in cases.items():
        for _ in range(max(args.warmup, 1)):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / steps
        gbs = nbytes / ms / 1e6
        res[name] = {"GB/s": round(gbs, 1), "frac": round(gbs / PEAK_HBM_GBS, 4), "avg_launch_ms": round(ms, 4),
                     "bytes_per_launch": int(nbytes), "mix": mix}  # fmt: skip
        tot_b += nbytes
        tot_ms += ms
    del x, fc1, dh, w
    torch.cuda.empty_cache()
    if with_probe:
        probe = mix_probe(dev, sorted({v[2] for v in cases.values()}))
        for name, (_, _, mix) in cases.items():
            res[name]["mix_probe_GB/s"] = probe[mix]["GB/s"]
            res[name]["frac_of_mix_probe"] = round(res[name]["GB/s"] / probe[mix]["GB/s"], 4)
    worst = min(res, key=lambda n: res[n]["frac"])
    total = tot_b / tot_ms / 1e6
    return {
        "metric": "quantisation kernels HBM GB/s (c2 shapes, all kernels one after the other)",
        "value": round(total, 1), "unit": "GB/s", "ms_per_step": round(tot_ms, 4), "dtype": "fp8",
        "config": {"workload": "quant: 32768 routed rows of 14336 features in 8 groups, weights 8 x 28672 x 4096, bf16 in"},
        "roofline": {"kernel": worst, "bound": "hbm", "achieved": res[worst]["GB/s"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": res[worst]["frac"], "traffic": None},
        "cpu_baseline": None,
        "extras": {"kernels": res},
    }  # fmt: skip


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(3)
    from atorch_amd import kernels

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.copy_probe:
        copy_probe(dev)
    if args.mix_probe:
        mixes = MIXES if args.mix_probe == "all" else args.mix_probe.split(",")
        print(json.dumps({"metric": "streaming probe GB/s by read:write mix", "unit": "GB/s", "n_gpus": 1,
                          "mixes": mix_probe(dev, mixes)}))  # fmt: skip
        return
    if args.workload == "module":
        # the expert MLP through the Python mirror alone (what extras.module_step of the default run reports): the
        # run a kernel trace of the whole forward + backward is taken from
        ms = module_step(kernels, dev, steps=args.steps)
        c = ms["cached_weight_codes"]
        print(json.dumps({"metric": "fp8 expert MLP forward + backward TFLOPS (module level)", "value": c["TFLOP/s"],
                          "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": 2, "ms_per_step": c["ms_per_step"],
                          "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8",
                          "data": "synthetic", "config": {"workload": ms["what"]}, "extras": ms}))  # fmt: skip
        return
    if args.workload == "quant":
        res = run_quant(args, kernels, dev)
    else:
        res = run_c5(args, kernels, dev) if args.workload == "c5" else run_gemm(args, kernels, dev)
    if args.workload == "c2" and not args.no_extras and args.operands == "random":
        # the other half of the metric (quant / permute GB/s), the other GEMM configurations, the module-level step and
        # the probes ride along in extras; each is a short run of its own with the same timers
        torch.cuda.empty_cache()
        r5 = run_c5(args, kernels, dev, cpu_baseline=False, mixes_too=False)
        pq = r5["roofline"]
        res["extras"]["c5"] = {
            "permute_quant": {k: pq[k] for k in ("achieved", "frac", "avg_launch_ms", "median_launch_ms", "bytes_per_launch",
                                                 "traffic")},
            "unpermute_combine": r5["extras"]["unpermute_combine"],
            "tile_quant_plain": r5["extras"]["tile_quant_plain"],
            "permute_quant_dual (training form)": r5["extras"]["permute_quant_dual (training form)"],
        }  # fmt: skip
        del r5
        torch.cuda.empty_cache()
        rq = run_quant(args, kernels, dev, steps=10, with_probe=False)
        res["extras"]["quant_kernels_c2_shapes"] = {
            name: {k: v[k] for k in ("GB/s", "frac", "avg_launch_ms")} for name, v in rq["extras"]["kernels"].items()}
        del rq
        torch.cuda.empty_cache()
        for wl in ("c3", "c4"):
            r = run_gemm(args, kernels, dev, workload=wl, steps=10, warmup=3, cpu_baseline=False, probes=False)
            res["extras"][wl] = {
                "value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"],
                "frac_of_fp8_peak": r["config"]["frac_of_fp8_peak"],
                "forward_dgrad_kernel_frac": r["roofline"]["frac"],
                "empty_groups": r["extras"]["empty_groups"],
                "tokens_per_expert_min_max": r["extras"]["tokens_per_expert_min_max"],
                "wgrad_kernel": r["extras"].get("wgrad_kernel"),
                "workload": r["config"]["workload"]}  # fmt: skip
            del r
            torch.cuda.empty_cache()
        res["extras"]["module_step"] = module_step(kernels, dev)
        res["extras"]["mfma_probe"] = mfma_probe(kernels, dev)
        # what the matrix pipes deliver on this operand data from registers alone, fold included: the ceiling the
        # power limit leaves the kernel (the fraction above stays priced against the published 5.0 PFLOP/s)
        lim = res["extras"]["mfma_probe"]["quantised_normal+fold"]["TFLOP/s"]
        res["roofline"]["data_limited_ceiling_tflops"] = lim
        res["roofline"]["frac_of_data_limited_ceiling"] = round(res["roofline"]["achieved"] / lim, 4)
        res["extras"]["loop_probe"] = loop_probe(dev)
    out = {
        "metric": res["metric"],
        "value": res["value"],
        "unit": res["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": res["dtype"],
        "data": "synthetic",
        "config": res["config"],
        "roofline": res["roofline"],
        "cpu_baseline": res["cpu_baseline"],
        "extras": res["extras"],
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
