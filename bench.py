#!/usr/bin/env python3
"""Benchmark of the FP8 block-scale path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload quant|prefill|decode|decode9|sweep|moe|fused|norm|stream|ceiling]
                    [--no-also] [--no-cpu]

A step is one pass of the hot path over one batch of synthetic input that is already resident
in HBM.  The primary workload (default ``quant``) fills ``value``; the other workloads of the
path are timed briefly as well and reported under ``also`` in the same JSON line.

Workloads (the benchmark configurations):
  quant    config 2  x bf16 [16384,7168] (1 % channels x50) -> fp8 + fp32 scales, HBM-bound
  prefill  config 4  blockscale GEMM M=8192 N=36864 K=7168, MFMA-bound
  decode   config 3  blockscale GEMM M=64 N=24576 K=1536 (the largest decode shape)
  decode9  config 3  all nine: M in {1,16,64} x (N,K) in {(7168,2048),(24576,1536),(2112,7168)};
                     weights rotate through 640 MB so that every call reads them from HBM
  sweep    (beyond the configs) M in {128..4096} x four projection shapes, each beside the
                     duration the reference's tuner recorded for it
  moe      (beyond the configs) block-scale expert layer of DeepSeek-V3, 1..1024 tokens
  fused    config 5  RMSNorm + 1x128 quant on [2048,7168], then GEMM N=4096
  stream   (calibration) read-only / write-only / 2:1 mixed streaming rates of the quant kernel's
                     access pattern without its arithmetic, on config 2's byte counts
  ceiling  (calibration) the prefill GEMM's arithmetic (fp8 MFMA + four scale FMAs per MFMA) on
                     register-resident operands -- no LDS, no global memory -- run for seconds with
                     the shader clock and socket power sampled beside it, then the prefill kernel
                     itself under the same sampling
The two calibration workloads use kernels of their own (bench_probes.hip -> libbench_probes.so,
built by __graft_entry__.build()); they are not part of the product library.

Timing uses HIP events recorded on the stream the kernels are launched on (torch's current
stream) around exactly K launches-worth of steps, bracketed by device synchronisation.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "blockscale GEMM TFLOP/s (% FP8 MFMA peak); group-quant GB/s (% HBM peak)"
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
FP8_PEAK_TFLOPS = 5000.0       # MI355X dense FP8 MFMA
# The reference's own tuner measurement for the prefill shape on gfx950 / 256 CUs
# (aiter/configs/model_configs/a8w8_blockscale_tuned_gemm_ds_v3.csv:6382).
REF_PREFILL_TFLOPS = 2108.5


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="quant", choices=["quant", "prefill", "decode", "decode9", "sweep", "moe", "fused", "norm", "copy", "stream", "ceiling"],
                    help="'copy' is a plain 1 GiB device copy used to calibrate the rocprofv3 FETCH_SIZE / "
                    "WRITE_SIZE counters; it is not part of the path")
    ap.add_argument("--no-also", action="store_true", help="time only the primary workload")
    ap.add_argument("--rotate-mb", type=int, default=640,
                    help="decode workloads: cycle through this many MB of weight copies (default 640, "
                    "more than twice the last-level cache; 0 keeps three copies, which stay cached)")
    ap.add_argument("--layout", default="plain", choices=["plain", "preshuffled"],
                    help="GEMM workloads: row-major weights (gemm_a8w8_blockscale) or weights shuffled "
                    "(16,16) with column-major x_scale (gemm_a8w8_blockscale_bpreshuffle)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--kernel-name", default="", help="kernelName handed to the expert kernel of --workload moe")
    ap.add_argument("--rows", type=int, default=2048, help="rows of --workload norm (config 5 has 2048)")
    return ap.parse_args()


WARM_SECONDS = 0.12  # untimed work before a measurement (the primary one, `also`, per-shape tables)


def time_steps(torch, fn, steps, warmup, settle=False):
    """Average seconds per call of fn over exactly `steps` calls, HIP events on the current stream.
    `settle`: besides the `warmup` calls, keep calling for WARM_SECONDS first, so that a short
    timed region is not measured while the clocks still ramp up from idle."""
    for _ in range(warmup):
        fn()
    if settle:
        torch.cuda.synchronize()
        t_warm = time.perf_counter()
        while time.perf_counter() - t_warm < WARM_SECONDS:
            for _ in range(20):  # back to back: a device that idles between calls does not raise its clocks
                fn()
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / steps


def time_launches(torch, fn, steps, warmup):
    """Seconds per launch when `steps` launches run back to back on the device: the calls are
    captured into a HIP graph on a side stream and the graph is replayed (a Python call costs
    several times what a decode kernel takes).  Every replay is bracketed by HIP events on the
    stream it is launched on; the median of five replays is returned.  Kernels replayed back to
    back overlap one launch's tail with the next one's head, so this figure can be below the
    duration a profiler reports for the kernel alone: the fields that carry it say "replay"."""
    torch.zeros(1, device="cuda")  # a fill kernel: cuts a kernel trace of the run into its measurements
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(steps):
                fn()
        # untimed replays until the clocks have settled (a launch sequence that starts on an idle
        # chip runs its first tens of milliseconds at lower clocks)
        t_warm = time.perf_counter()
        while True:
            graph.replay()
            side.synchronize()
            if time.perf_counter() - t_warm > WARM_SECONDS:
                break
        times = []
        for _ in range(5):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(side)
            graph.replay()
            b.record(side)
            side.synchronize()
            times.append(a.elapsed_time(b) * 1e-3 / steps)
    return sorted(times)[len(times) // 2]


def gemm_bytes(m, n, k):
    # algorithmic bytes: fp8 operands read once, 16-bit output written once, fp32 scales read once
    return m * k + n * k + 2 * m * n + 4 * m * (k // 128) + 4 * ((n + 127) // 128) * (k // 128)


def quant_weight_gpu(torch, fp8, n, k, seed, dev):
    """w ~ N(0, 0.02) in bf16, quantised per 128x128 block by the library's own weight quantiser
    (setup only, never timed)."""
    import aiter_amd

    gw = torch.Generator(device=dev).manual_seed(seed)
    w = (torch.randn(n, k, generator=gw, device=dev) * 0.02).bfloat16()
    return aiter_amd.weight_per_128x128_quant(w, quant_dtype=fp8)


PROBES_PATH = os.path.join(ROOT, "libbench_probes.so")
_probes = None


def load_probes():
    """ctypes handle of libbench_probes.so (bench_probes.hip): the calibration kernels of the
    `stream` and `ceiling` workloads.  Built by __graft_entry__.build(); never built here."""
    global _probes
    if _probes is None:
        import ctypes

        if not os.path.exists(PROBES_PATH):
            raise RuntimeError(f"{PROBES_PATH} is missing: run `python __graft_entry__.py` (build) first")
        lib = ctypes.CDLL(PROBES_PATH)
        lib.probe_stream.restype = ctypes.c_int
        lib.probe_stream.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]
        lib.probe_mfma.restype = ctypes.c_int
        lib.probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                   ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        _probes = lib
    return _probes


class GpuSampler:
    """Samples the socket power and the shader clock of GPU 0 from a host thread while a
    measurement runs.  Power: the amdgpu hwmon file power1_average / power1_input (microwatts).
    Clock: hwmon freq1_input (Hz) or the starred line of pp_dpm_sclk where one of them can be read;
    otherwise `rocm-smi --showclocks --json`, asked every tenth sample (it takes a quarter of a
    second)."""

    def __init__(self, period=0.02):
        import glob
        import shutil

        self.period = period
        self.samples = []  # (t, sclk_mhz or None, watts or None)
        self._stop = False
        self._thread = None
        self.power_file = self.freq_file = self.dpm_file = None
        for dev in sorted(glob.glob("/sys/class/drm/card*/device")):
            for hw in sorted(glob.glob(os.path.join(dev, "hwmon", "hwmon*"))):
                for n in ("power1_average", "power1_input"):
                    if self.power_file is None and self._number(os.path.join(hw, n)) is not None:
                        self.power_file = os.path.join(hw, n)
                if self.freq_file is None and self._number(os.path.join(hw, "freq1_input")) is not None:
                    self.freq_file = os.path.join(hw, "freq1_input")
            if self.dpm_file is None and self._dpm(os.path.join(dev, "pp_dpm_sclk")) is not None:
                self.dpm_file = os.path.join(dev, "pp_dpm_sclk")
            if self.power_file or self.freq_file or self.dpm_file:
                break
        self.smi = shutil.which("rocm-smi") if not (self.freq_file or self.dpm_file) else None
        self.source = {"power": self.power_file, "clock": self.freq_file or self.dpm_file or self.smi}

    @staticmethod
    def _number(path):
        try:
            with open(path) as f:
                return float(f.read().strip())
        except (OSError, ValueError):
            return None

    @staticmethod
    def _dpm(path):
        """MHz of the level that pp_dpm_sclk marks as current ("1: 2400Mhz *")."""
        import re

        try:
            with open(path) as f:
                for ln in f:
                    if "*" in ln:
                        m = re.search(r"(\d+(?:\.\d+)?)\s*mhz", ln.lower())
                        if m:
                            return float(m.group(1))
        except OSError:
            pass
        return None

    def _smi_clock(self):
        import re
        import subprocess

        try:
            out = subprocess.run([self.smi, "--showclocks", "--json"], capture_output=True, text=True, timeout=5).stdout
            card = json.loads(out)
            card = card[sorted(card)[0]]
            for k, v in card.items():
                if "sclk clock speed" in k.lower():
                    m = re.search(r"(\d+(?:\.\d+)?)\s*mhz", str(v).lower())
                    if m:
                        return float(m.group(1))
        except Exception:
            pass
        return None

    def _read_once(self, i):
        watts = self._number(self.power_file) if self.power_file else None
        if watts is not None:
            watts /= 1e6
        mhz = None
        if self.freq_file:
            mhz = self._number(self.freq_file)
            mhz = mhz / 1e6 if mhz is not None else None
        elif self.dpm_file:
            mhz = self._dpm(self.dpm_file)
        elif self.smi and i % 10 == 5:
            mhz = self._smi_clock()
        return mhz, watts

    def __enter__(self):
        import threading

        def loop():
            i = 0
            while not self._stop:
                mhz, watts = self._read_once(i)
                self.samples.append((time.perf_counter(), mhz, watts))
                i += 1
                time.sleep(self.period)

        self._thread = threading.Thread(target=loop, daemon=True)
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        self._thread.join()

    def summary(self, t_from, t_to):
        """Mean clock (MHz) and power (W) over the samples taken in [t_from, t_to]."""
        sel = [x for x in self.samples if t_from <= x[0] <= t_to]
        clk = [x[1] for x in sel if x[1] is not None]
        pw = [x[2] for x in sel if x[2] is not None]
        return {"sclk_mhz": sum(clk) / len(clk) if clk else None, "sclk_samples": len(clk),
                "socket_watts": sum(pw) / len(pw) if pw else None, "power_samples": len(pw), "source": self.source}


def sustained(torch, fn, seconds, launches_per_sync=4):
    """Keeps calling fn for `seconds`, then reports the seconds per call over the second half
    of that time (HIP events) with the clock and power sampled over the same half."""
    with GpuSampler() as sampler:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds / 2:
            for _ in range(launches_per_sync):
                fn()
            torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t1 = time.perf_counter()
        a.record()
        n = 0
        while time.perf_counter() - t1 < seconds / 2:
            for _ in range(launches_per_sync):
                fn()
            n += launches_per_sync
            torch.cuda.synchronize()
        b.record()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
    return a.elapsed_time(b) * 1e-3 / n, n, sampler.summary(t1, t2)


# ---------------------------------------------------------------- workloads


class QuantWorkload:
    name = "quant"
    M, K = 16384, 7168

    def setup(self, torch, dev):
        import aiter_amd
        from aiter_amd import dtypes
        from oracle import torch_ref as tr

        self.aiter = aiter_amd
        self.x_cpu = tr.make_activation(self.M, self.K, seed=0, outlier_frac=0.01)
        # rotate over several inputs so that no pass finds its input in the 256 MB last-level cache
        base = self.x_cpu.to(dev)
        self.xs = [base, base.clone(), base.clone()]
        # ... and over as many outputs (3 x (235 + 117 + 3.7) MB in rotation)
        self.ys = [torch.empty(self.M, self.K, dtype=dtypes.fp8, device=dev) for _ in self.xs]
        self.ss = [torch.empty(self.M, self.K // 128, dtype=torch.float32, device=dev) for _ in self.xs]
        self.i = 0

    def step(self):
        self.i = (self.i + 1) % len(self.xs)
        self.aiter.dynamic_per_token_scaled_quant(self.ys[self.i], self.xs[self.i].view(-1, 128), self.ss[self.i])

    def algorithmic_bytes(self):
        return self.M * self.K * 2 + self.M * self.K + self.M * (self.K // 128) * 4

    def describe(self):
        return {
            "workload": "config 2: standalone 1x128 dynamic FP8 group quant, x bf16 [16384,7168] "
            "N(0,1) with 1% of channels x50 -> fp8 e4m3fn [16384,7168] + fp32 scales [16384,56]",
            "M": self.M,
            "K": self.K,
            "group": 128,
            "kernel": "group_quant_kernel",
        }

    def result(self, sec):
        gbs = self.algorithmic_bytes() / sec / 1e9
        roof = {
            "bound": "hbm",
            "achieved": gbs,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": gbs / HBM_PEAK_GBS,
            "traffic": load_traffic("group_quant_kernel"),
        }
        return gbs, "GB/s", roof

    def cpu_baseline(self, torch):
        from oracle import torch_ref as tr

        rows = self.M  # the whole input
        x = self.x_cpu
        tr.per_1x128_quant(x)
        ts = []
        for _ in range(5):
            t0 = time.perf_counter()
            tr.per_1x128_quant(x)
            ts.append(time.perf_counter() - t0)
        sec = sorted(ts)[len(ts) // 2]
        by = rows * self.K * 3 + rows * (self.K // 128) * 4
        return {
            "value": by / sec / 1e9,
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"torch-CPU restatement of pertoken_quant on the whole input "
            f"([{rows},{self.K}] bf16), median of 5 runs, {sec * 1e3:.1f} ms each",
        }


class GemmWorkload:
    layout = "plain"  # set from --layout before setup()
    rotate_mb = 640   # set from --rotate-mb before setup()
    rotate_always = False

    def __init__(self, name, m, n, k, label):
        self.name, self.M, self.N, self.K, self.label = name, m, n, k, label

    def setup(self, torch, dev):
        import aiter_amd
        from aiter_amd import dtypes

        self.aiter = aiter_amd
        g = torch.Generator(device=dev).manual_seed(0)
        m, n, k = self.M, self.N, self.K

        # Operands with the distribution the configs name: x ~ N(0,1) (1 % of channels x50 for the
        # prefill shape) quantised 1x128 by this library's own kernel, w ~ N(0,0.02) quantised
        # per 128x128 block (torch ops on the GPU; how the weights get quantised is not timed).
        x = torch.randn(m, k, generator=g, device=dev)
        if m >= 1024:
            ch = torch.randperm(k, generator=g, device=dev)[: max(1, k // 100)]
            x[:, ch] *= 50.0
        pre = self.layout == "preshuffled"
        self.xq, self.xs = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)(
            x.bfloat16(), quant_dtype=dtypes.fp8, transpose_scale=pre)
        del x

        # Rotate the weights so that no call finds them in a cache: three buffers for the
        # compute-bound shapes, and for the decode shapes (which are nothing but a weight read) as
        # many copies as it takes to cycle through 640 MB, more than twice the 256 MB last-level cache.
        nbuf = 1 if (n * k) > (1 << 28) else 3
        pairs = [quant_weight_gpu(torch, dtypes.fp8, n, k, 10 + i, dev) for i in range(nbuf)]
        self.wqs = [p[0] for p in pairs]
        if pre:
            self.wqs = [aiter_amd.shuffle_weight(w.view(torch.uint8)).view(w.dtype) for w in self.wqs]
        self.ws = pairs[0][1]
        if m <= 64 or self.rotate_always:
            want = -(-self.rotate_mb * 1_000_000 // (n * k))
            self.wqs += [self.wqs[i % nbuf].clone() for i in range(max(0, want - nbuf))]
        self.weight_bytes_rotated = len(self.wqs) * n * k
        self.out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
        self.i = 0

    def step(self):
        self.i = (self.i + 1) % len(self.wqs)
        if self.layout == "preshuffled":
            self.aiter.gemm_a8w8_blockscale_bpreshuffle_ck(self.xq, self.wqs[self.i], self.xs, self.ws, self.out)
        else:
            self.aiter.gemm_a8w8_blockscale_ck(self.xq, self.wqs[self.i], self.xs, self.ws, self.out, splitK=-1)

    def flops(self):
        return 2.0 * self.M * self.N * self.K

    def describe(self):
        return {"workload": self.label, "M": self.M, "N": self.N, "K": self.K, "layout": self.layout,
                "kernel": "gemm_a8w8_blockscale" + ("_bpreshuffle" if self.layout == "preshuffled" else "")}

    def result(self, sec):
        tf = self.flops() / sec / 1e12
        gbs = gemm_bytes(self.M, self.N, self.K) / sec / 1e9
        if self.M >= 1024:
            roof = {"bound": "mfma", "achieved": tf, "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": tf / FP8_PEAK_TFLOPS, "traffic": load_traffic("gemm_prefill")}
            return tf, "TFLOP/s", roof
        roof = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": gbs / HBM_PEAK_GBS, "traffic": None}
        return gbs, "GB/s", roof

    def cpu_baseline(self, torch):
        from oracle import torch_ref as tr

        if self.layout == "preshuffled":
            return None  # same arithmetic as the plain layout, whose run carries the CPU figure
        # rows are independent: a slice of at most 128 rows against every column, scaled linearly
        rows = min(self.M, 128)
        xq = self.xq[:rows].cpu()
        wq = self.wqs[0].cpu()
        xs = self.xs[:rows].cpu()
        ws = self.ws.cpu()
        tr.gemm_a8w8_blockscale_ref(xq, wq, xs, ws)
        ts = []
        for _ in range(5):
            t0 = time.perf_counter()
            tr.gemm_a8w8_blockscale_ref(xq, wq, xs, ws)
            ts.append(time.perf_counter() - t0)
        sec = sorted(ts)[len(ts) // 2]
        return {
            "value": 2.0 * rows * self.N * self.K / sec / 1e12,
            "unit": "TFLOP/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "extrapolated": rows < self.M,
            "sample": f"torch-CPU restatement (dequantise both operands to fp32 + F.linear) on rows 0..{rows - 1} "
            f"x all {self.N} columns, median of 5 runs, {sec * 1e3:.0f} ms each, weight dequantisation included"
            + (f"; the whole problem would take {self.M // rows} x as long with the weights dequantised every time"
               if rows < self.M else ""),
        }


class FusedWorkload:
    name = "fused"
    M, K, N = 2048, 7168, 4096

    def setup(self, torch, dev):
        import aiter_amd
        from aiter_amd import dtypes
        from oracle import torch_ref as tr

        self.aiter = aiter_amd
        self.x_cpu = tr.make_activation(self.M, self.K, seed=0)
        g = torch.Generator().manual_seed(1)
        self.w_cpu = (torch.rand(self.K, generator=g) + 0.5).bfloat16()
        self.x = self.x_cpu.to(dev)
        self.nw = self.w_cpu.to(dev)
        self.y = torch.empty(self.M, self.K, dtype=dtypes.fp8, device=dev)
        self.s = torch.empty(self.M, self.K // 128, dtype=torch.float32, device=dev)
        self.wq, self.ws = quant_weight_gpu(torch, dtypes.fp8, self.N, self.K, 2, dev)
        self.out = torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev)

    def step(self):
        self.aiter.rmsnorm2d_fwd_with_dynamicquant(self.y, self.x, self.s, self.nw, 1e-6, 0, group_size=128)
        self.aiter.gemm_a8w8_blockscale_ck(self.y, self.wq, self.s, self.ws, self.out, splitK=-1)

    def step_norm_only(self):
        # For the norm's own share of HBM: rows, codes and scales rotate through enough sets (640 MB, more
        # than twice the 256 MB last-level cache) that no launch finds its input in a cache.  The fused
        # step above keeps one set, as a layer does whose input the previous kernel has just written.
        if not hasattr(self, "rot"):
            import torch

            sets = -(-640_000_000 // self.norm_bytes())
            self.rot = [(self.x.clone(), torch.empty_like(self.y), torch.empty_like(self.s)) for _ in range(sets)]
            self.rot_i = 0
        x, y, s = self.rot[self.rot_i]
        self.rot_i = (self.rot_i + 1) % len(self.rot)
        self.aiter.rmsnorm2d_fwd_with_dynamicquant(y, x, s, self.nw, 1e-6, 0, group_size=128)

    def step_norm_cached(self):
        # the same on the fused step's one set of buffers: what the kernel takes inside a layer, where the
        # 256 MB last-level cache still holds the rows the previous kernel wrote
        self.aiter.rmsnorm2d_fwd_with_dynamicquant(self.y, self.x, self.s, self.nw, 1e-6, 0, group_size=128)

    def describe(self):
        return {
            "workload": "config 5: fused RMSNorm + 1x128 FP8 quant on x bf16 [2048,7168], then blockscale "
            "GEMM with N=4096, K=7168",
            "M": self.M, "N": self.N, "K": self.K, "kernel": "rmsnorm_kernel + gemm_a8w8_blockscale",
        }

    def norm_bytes(self):
        return self.M * self.K * 3 + self.K * 2 + self.M * (self.K // 128) * 4

    def result(self, sec):
        tf = 2.0 * self.M * self.N * self.K / sec / 1e12
        roof = {"bound": "mfma", "achieved": tf, "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": tf / FP8_PEAK_TFLOPS, "traffic": None}
        return tf, "TFLOP/s", roof

    def cpu_baseline(self, torch):
        from oracle import torch_ref as tr

        rows = 512
        x = self.x_cpu[:rows]
        tr.rmsnorm_quant_ref(x, self.w_cpu, 1e-6)
        ts = []
        for _ in range(5):
            t0 = time.perf_counter()
            tr.rmsnorm_quant_ref(x, self.w_cpu, 1e-6)
            ts.append(time.perf_counter() - t0)
        sec = sorted(ts)[len(ts) // 2]
        by = rows * self.K * 3 + self.K * 2 + rows * (self.K // 128) * 4
        return {"value": by / sec / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"torch-CPU F.rms_norm + pertoken_quant on rows 0..{rows - 1}, median of 5 runs, "
                f"{sec * 1e3:.1f} ms each (the norm + quant half; the GEMM half has the prefill workload's baseline)"}


def load_traffic(kernel):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE, calibrated on
    a plain copy kernel); the numbers live in profiles/traffic.json beside the rocprof summaries."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(kernel, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


DECODE_SHAPES = [(m, n, k) for (n, k) in [(7168, 2048), (24576, 1536), (2112, 7168)] for m in (1, 16, 64)]


class CopyCalibration:
    """Plain device-to-device copy of a known size (torch's copy kernel): reads NBYTES, writes NBYTES."""

    name = "copy"
    NBYTES = 1 << 30

    def setup(self, torch, dev):
        self.src = torch.empty(self.NBYTES, dtype=torch.uint8, device=dev).random_(0, 255)
        self.dst = torch.empty_like(self.src)

    def step(self):
        self.dst.copy_(self.src)

    def describe(self):
        return {"workload": "calibration: plain 1 GiB device copy", "bytes_read": self.NBYTES,
                "bytes_written": self.NBYTES, "kernel": "torch elementwise copy"}

    def result(self, sec):
        gbs = 2 * self.NBYTES / sec / 1e9
        return gbs, "GB/s", {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": gbs / HBM_PEAK_GBS, "traffic": None}

    def cpu_baseline(self, torch):
        return None


class StreamCeilings:
    """The quant kernel with its arithmetic taken out (probe_stream of bench_probes.hip: same grid, same
    32 bytes in and 16 bytes out per lane, same cache policy) on config 2's byte counts: a
    read-only pass over the 235 MB input, a write-only pass over the 117 MB output, and the 2 : 1
    mix of both.  The ceiling the quant kernel is held against."""

    name = "stream"
    M, K = 16384, 7168

    def setup(self, torch, dev):
        self.torch = torch
        self.lib = load_probes()
        n = self.M * self.K
        self.xs = [torch.randn(n, device=dev).bfloat16() for _ in range(3)]
        self.ys = [torch.empty(n, dtype=torch.uint8, device=dev) for _ in range(3)]
        self.i = 0

    def _probe(self, mode):
        self.i = (self.i + 1) % len(self.xs)
        x, y = self.xs[self.i], self.ys[self.i]
        rc = self.lib.probe_stream(mode, x.data_ptr(), y.data_ptr(), y.numel() // 16,
                                   self.torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(f"probe_stream: hipError {rc}")

    def step(self):  # the mix
        self._probe(2)

    def step_read(self):
        self._probe(0)

    def step_write(self):
        self._probe(1)

    def describe(self):
        return {"workload": "streaming ceilings for config 2's byte mix (the quant kernel without arithmetic): "
                            "headline value is the 2:1 read/write mix; read-only and write-only ride in per_shape",
                "kernel": "stream_probe_kernel"}

    def result(self, sec):
        by = self.M * self.K * 3
        gbs = by / sec / 1e9
        return gbs, "GB/s", {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": gbs / HBM_PEAK_GBS, "traffic": None}

    def per_shape(self, torch, steps, warmup):
        n = self.M * self.K
        out = []
        for what, fn, by in (("read-only, 2 B per element", self.step_read, 2 * n),
                             ("write-only, 1 B per element", self.step_write, n),
                             ("2 B read + 1 B written per element", self.step, 3 * n)):
            sec = time_steps(torch, fn, steps, warmup, settle=True)
            out.append({"what": what, "bytes": by, "us": sec * 1e6, "GB/s": by / sec / 1e9,
                        "frac_of_hbm_peak": by / sec / 1e9 / HBM_PEAK_GBS})
        return out

    def cpu_baseline(self, torch):
        return None


class ComputeCeiling:
    """What the chip gives the prefill GEMM's arithmetic alone.  probe_mfma (bench_probes.hip) runs the
    product kernel's inner instruction stream -- v_mfma_f32_16x16x128_f8f6f4 on real fp8 codes, each
    product folded into fp32 accumulators by four v_fmac_f32 two MFMA slots later -- on operands that
    never leave the registers: one workgroup per compute unit, no LDS, no global memory, no barrier.
    Every variant runs for SECONDS with the shader clock and the socket power sampled beside it;
    then the prefill kernel itself (config 4, both weight layouts) runs under the same sampling."""

    name = "ceiling"
    SECONDS = 4.0
    ITERS = 60000  # passes of 32 MFMAs per wave and launch: about 60 ms per launch

    def setup(self, torch, dev):
        import aiter_amd
        from aiter_amd import dtypes

        self.torch, self.dev = torch, dev
        self.lib = load_probes()
        self.cus = torch.cuda.get_device_properties(0).multi_processor_count
        g = torch.Generator(device=dev).manual_seed(0)
        # operands with the code distribution of config 4: x ~ N(0,1) with 1 % of the channels x 50,
        # quantised 1 x 128; w ~ N(0, 0.02) quantised 128 x 128
        x = torch.randn(512, 7168, generator=g, device=dev)
        ch = torch.randperm(7168, generator=g, device=dev)[:71]
        x[:, ch] *= 50.0
        xq, _ = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)(x.bfloat16(), quant_dtype=dtypes.fp8)
        wq, _ = quant_weight_gpu(torch, dtypes.fp8, 512, 7168, 10, dev)
        self.real = (wq.view(torch.uint8).flatten()[: 8 * 512 * 32].contiguous(),
                     xq.view(torch.uint8).flatten()[: 4 * 512 * 32].contiguous())
        self.zero = (torch.zeros_like(self.real[0]), torch.zeros_like(self.real[1]))
        self.scales = torch.full((4 * 512,), 1e-9, dtype=torch.float32, device=dev)
        self.sink = torch.empty(self.cus * 512, dtype=torch.float32, device=dev)
        self.variant = (4, 512, self.real)

    def _launch(self, fmas, threads, codes, iters, wide=0):
        rc = self.lib.probe_mfma(fmas, threads, wide, codes[0].data_ptr(), codes[1].data_ptr(), self.scales.data_ptr(),
                                 self.sink.data_ptr(), iters, self.cus, self.torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(f"probe_mfma: hipError {rc}")

    def flops_per_launch(self, threads, iters):
        return self.cus * (threads // 64) * iters * 32 * 65536.0

    def step(self):  # the headline: MFMA + 4 FMA, two waves per SIMD, real codes
        self._launch(4, 512, self.real, self.ITERS // 8)

    def describe(self):
        return {"workload": "compute ceiling of the prefill GEMM's arithmetic: register-resident fp8 MFMA + 4 scale "
                            "FMAs per MFMA, one workgroup of 8 waves per compute unit, no LDS, no global memory; "
                            "headline value is a short run, the sustained figures with clock and power ride in per_shape",
                "kernel": "mfma_ceiling_kernel (bench_probes.hip)"}

    def result(self, sec):
        tf = self.flops_per_launch(512, self.ITERS // 8) / sec / 1e12
        return tf, "TFLOP/s", {"bound": "mfma", "achieved": tf, "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                               "frac": tf / FP8_PEAK_TFLOPS, "traffic": None}

    def per_shape(self, torch, steps, warmup):
        out = []
        variants = [
            ("MFMA + 4 FMA, 8 waves per CU, config-4 codes", 4, 512, self.real),
            ("MFMA only, 8 waves per CU, config-4 codes", 0, 512, self.real),
            ("MFMA + 4 FMA, 4 waves per CU, config-4 codes", 4, 256, self.real),
            ("MFMA only, 4 waves per CU, config-4 codes", 0, 256, self.real),
            ("MFMA + 4 FMA, 8 waves per CU, all-zero codes", 4, 512, self.zero),
            ("32x32x64 MFMA + 4 FMA per 16x16 of output, 8 waves per CU, config-4 codes", 4, 512, self.real, 1),
            ("32x32x64 MFMA only, 8 waves per CU, config-4 codes", 0, 512, self.real, 1),
        ]
        for what, fmas, threads, codes, *wide in variants:
            wide = wide[0] if wide else 0
            iters = self.ITERS if threads == 512 else 2 * self.ITERS
            sec, n, smp = sustained(torch, lambda: self._launch(fmas, threads, codes, iters, wide), self.SECONDS, 2)
            tf = self.flops_per_launch(threads, iters) / sec / 1e12
            row = {"what": what, "ms_per_launch": sec * 1e3, "launches_timed": n, "TFLOP/s": tf,
                   "frac_of_fp8_peak": tf / FP8_PEAK_TFLOPS,
                   # the clock at which a matrix pipe that is never idle would deliver this rate
                   "mfma_issue_ghz": (threads // 256) * iters * 32 * 32 / sec / 1e9}
            row.update(smp)
            out.append(row)
        del self.sink
        for layout in ("plain", "preshuffled"):
            torch.cuda.empty_cache()
            w = GemmWorkload("prefill", 8192, 36864, 7168, "config 4")
            w.layout = layout
            w.setup(torch, self.dev)
            sec, n, smp = sustained(torch, w.step, self.SECONDS, 8)
            tf = w.flops() / sec / 1e12
            row = {"what": f"prefill kernel, config 4, {layout} weights", "ms_per_launch": sec * 1e3, "launches_timed": n,
                   "TFLOP/s": tf, "frac_of_fp8_peak": tf / FP8_PEAK_TFLOPS,
                   "frac_of_ceiling": tf / out[0]["TFLOP/s"]}
            row.update(smp)
            out.append(row)
            del w
        return out

    def cpu_baseline(self, torch):
        return None


class NormWorkload(FusedWorkload):
    """The norm + quant half of config 5 by itself, on rows that come from HBM (buffers rotate)."""
    name = "norm"

    def __init__(self, rows=2048):
        self.M = rows

    def step(self):
        self.step_norm_only()

    def describe(self):
        return {"workload": f"fused RMSNorm + 1x128 FP8 quant on x bf16 [{self.M},{self.K}] (config 5's first half), "
                "inputs and outputs rotating through 640 MB", "M": self.M, "K": self.K, "kernel": "rmsnorm_kernel"}

    def result(self, sec):
        gb = self.norm_bytes() / sec / 1e9
        roof = {"bound": "hbm", "achieved": gb, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gb / HBM_PEAK_GBS,
                "traffic": None}
        return gb, "GB/s", roof


class DecodeAllWorkload:
    """All nine decode shapes of config 3, one launch each per step (shape after shape, so a kernel
    trace of the run lists them in DECODE_SHAPES order)."""

    name = "decode9"

    def setup(self, torch, dev):
        self.parts = [GemmWorkload("decode", m, n, k, "decode") for (m, n, k) in DECODE_SHAPES]
        for w in self.parts:
            w.setup(torch, dev)

    def step(self):
        for w in self.parts:
            w.step()

    def bytes(self):
        return sum(gemm_bytes(w.M, w.N, w.K) for w in self.parts)

    def describe(self):
        return {"workload": "config 3: the nine decode blockscale GEMM shapes, one launch each per step",
                "shapes": [list(sh) for sh in DECODE_SHAPES], "kernel": "gemm_a8w8_blockscale (decode_stream)"}

    def result(self, sec):
        gbs = self.bytes() / sec / 1e9
        return gbs, "GB/s", {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": gbs / HBM_PEAK_GBS, "traffic": None}

    def per_shape(self, torch, steps, warmup):
        out = []
        for w in self.parts:
            s3 = time_launches(torch, w.step, steps, warmup)
            gbs = gemm_bytes(w.M, w.N, w.K) / s3 / 1e9
            out.append({"M": w.M, "N": w.N, "K": w.K, "replay_us_per_launch": s3 * 1e6, "GB/s": gbs,
                        "frac_of_hbm_peak": gbs / HBM_PEAK_GBS})
        return out

    def cpu_baseline(self, torch):
        return self.parts[-1].cpu_baseline(torch)


# Durations (us) the reference's tuner recorded on gfx950 for these shapes
# (aiter/configs/model_configs/a8w8_blockscale_tuned_gemm_ds_v3.csv, column "us").
SWEEP_REFERENCE_US = {
    (128, 7168, 2048): 9.4978, (256, 7168, 2048): 13.6951, (512, 7168, 2048): 20.7712,
    (1024, 7168, 2048): 34.0461, (2048, 7168, 2048): 68.5722, (4096, 7168, 2048): 120.1982,
    (128, 24576, 1536): 17.3757, (256, 24576, 1536): 27.2881, (512, 24576, 1536): 46.3688,
    (1024, 24576, 1536): 84.1555, (2048, 24576, 1536): 153.4331, (4096, 24576, 1536): 282.6274,
    (128, 2112, 7168): 21.1709, (256, 2112, 7168): 23.0603, (512, 2112, 7168): 32.0652,
    (1024, 2112, 7168): 51.2969, (2048, 2112, 7168): 88.3043, (4096, 2112, 7168): 91.0323,
    (128, 4096, 7168): 23.6181, (256, 4096, 7168): 24.9567, (512, 4096, 7168): 44.5905,
    (1024, 4096, 7168): 63.9434, (2048, 4096, 7168): 114.7033, (4096, 4096, 7168): 209.3355,
}


class SweepWorkload:
    """Token counts between decode and prefill (M = 128 ... 4096) on the four DeepSeek-V3 projection
    shapes, each launch timed by graph replay with the weights cycled through --rotate-mb."""

    name = "sweep"

    def setup(self, torch, dev):
        self.torch, self.dev = torch, dev
        self.shapes = list(SWEEP_REFERENCE_US)
        # the headline number of this workload is one shape; the table rides in per_shape
        self.head = GemmWorkload("sweep", 1024, 4096, 7168, "sweep")
        self.head.rotate_always = True
        self.head.setup(torch, dev)

    def step(self):
        self.head.step()

    def describe(self):
        return {"workload": "blockscale GEMM, M = 128..4096 on (N,K) = (7168,2048), (24576,1536), (2112,7168), "
                            "(4096,7168); headline value is (1024, 4096, 7168)",
                "layout": GemmWorkload.layout, "kernel": "gemm_a8w8_blockscale (automatic kernel choice)"}

    def result(self, sec):
        tf = self.head.flops() / sec / 1e12
        return tf, "TFLOP/s", {"bound": "mfma", "achieved": tf, "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                               "frac": tf / FP8_PEAK_TFLOPS, "traffic": None}

    def per_shape(self, torch, steps, warmup):
        del self.head
        out = []
        for (m, n, k) in self.shapes:
            torch.cuda.empty_cache()
            w = GemmWorkload("sweep", m, n, k, "sweep")
            w.rotate_always = True
            w.setup(torch, self.dev)
            s3 = time_launches(torch, w.step, steps, warmup)
            ref = SWEEP_REFERENCE_US[(m, n, k)]
            out.append({"M": m, "N": n, "K": k, "replay_us_per_launch": s3 * 1e6, "TFLOP/s": w.flops() / s3 / 1e12,
                        "reference_tuned_us": ref, "reference_over_ours": ref / (s3 * 1e6)})
            del w
        return out

    def cpu_baseline(self, torch):
        return None


# Durations (us) the reference's tuner recorded on a 256-CU part for the DeepSeek-V3 expert layer
# (dim 7168, inter 256, 256 routed + 1 shared expert, top-8 + shared, fp8 per_1x128):
# aiter/configs/model_configs/a8w8_blockscale_tuned_fmoe_ds_v3.csv, column "us" (both GEMM stages).
MOE_REFERENCE_US = {1: 77.49, 16: 112.68, 32: 158.48, 64: 212.99, 128: 241.60, 256: 249.58, 512: 260.97, 1024: 359.48}


class MoeWorkload:
    """Block-scale expert layer of DeepSeek-V3 at one GPU's share: tokens x (8 of 256 routed experts
    + the shared one), dim 7168, inter 256.  Timed: fmoe_fp8_blockscale_g1u1 on sorted tokens; the
    routing is redrawn for every launch of a replayed graph so that weights come from HBM."""

    name = "moe"
    DIM, INTER, ROUTED, TOPK = 7168, 256, 256, 8
    kernel_name = ""  # set from --kernel-name before setup()

    def setup(self, torch, dev):
        import aiter_amd
        from aiter_amd import dtypes

        self.torch, self.dev, self.aiter, self.fp8 = torch, dev, aiter_amd, dtypes.fp8
        E = self.ROUTED + 1
        g = torch.Generator(device=dev).manual_seed(0)
        w1 = (torch.randn(E * 2 * self.INTER, self.DIM, generator=g, device=dev) * 0.1).bfloat16()
        self.w1q, w1s = aiter_amd.weight_per_128x128_quant(w1)
        del w1
        w2 = (torch.randn(E * self.DIM, self.INTER, generator=g, device=dev) * 0.1).bfloat16()
        self.w2q, w2s = aiter_amd.weight_per_128x128_quant(w2)
        del w2
        self.w1q = aiter_amd.shuffle_weight(self.w1q.view(E, 2 * self.INTER, self.DIM).view(torch.uint8)).view(dtypes.fp8)
        self.w2q = aiter_amd.shuffle_weight(self.w2q.view(E, self.DIM, self.INTER).view(torch.uint8)).view(dtypes.fp8)
        self.w1s, self.w2s = w1s.view(E, -1).contiguous(), w2s.view(E, -1).contiguous()
        self.gen = g
        self.prepare(32)

    def prepare(self, tokens, routings=8):
        torch, dev, aiter_amd = self.torch, self.dev, self.aiter
        E = self.ROUTED + 1
        x = torch.randn(tokens, self.DIM, generator=self.gen, device=dev).bfloat16()
        self.xq, self.xs = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)(
            x, quant_dtype=self.fp8, transpose_scale=True)
        self.xs = self.xs.view(self.DIM // 128, tokens)
        self.tokens = tokens
        self.sorted = []
        self.experts_hit = 0
        for _ in range(routings):
            score = torch.randn(tokens, self.ROUTED, generator=self.gen, device=dev)
            tw, ti = aiter_amd.fused_topk(x, score, self.TOPK, True)
            ti = torch.cat([ti, torch.full((tokens, 1), self.ROUTED, dtype=ti.dtype, device=dev)], dim=1)
            tw = torch.cat([tw, torch.ones(tokens, 1, dtype=tw.dtype, device=dev)], dim=1)
            self.sorted.append(aiter_amd.moe_sorting(ti.contiguous(), tw.contiguous(), E, self.DIM, torch.bfloat16))
            self.experts_hit += ti.unique().numel()
        self.experts_hit /= routings
        self.ids_for_sort = (ti.contiguous(), tw.contiguous())
        self.i = 0

    def step(self):
        self.i = (self.i + 1) % len(self.sorted)
        s_ids, s_w, s_e, nv, out = self.sorted[self.i]
        self.aiter.fmoe_fp8_blockscale_g1u1(out, self.xq, self.w1q, self.w2q, s_ids, s_w, s_e, nv, self.TOPK + 1,
                                            self.xs, self.w1s, self.w2s, self.kernel_name)

    def step_sort(self):
        self.aiter.moe_sorting(self.ids_for_sort[0], self.ids_for_sort[1], self.ROUTED + 1, self.DIM,
                               self.torch.bfloat16)

    def bytes(self):
        # weights of the experts that are hit (read once), tokens and scales in, output out
        per_expert = 3 * self.INTER * self.DIM + 4 * (3 * self.INTER // 128) * (self.DIM // 128)
        return self.experts_hit * per_expert + self.tokens * self.DIM * (1 + 2) + 4 * self.tokens * self.DIM // 128

    def flops(self):
        return 2.0 * self.tokens * (self.TOPK + 1) * 3 * self.INTER * self.DIM

    def describe(self):
        return {"workload": "block-scale expert layer, dim 7168, inter 256, 256 routed + 1 shared expert, top-8 + "
                            "shared; headline value is 32 tokens",
                "kernel": "fmoe_fp8_blockscale_g1u1 (sorting timed separately)"}

    def result(self, sec):
        gbs = self.bytes() / sec / 1e9
        return gbs, "GB/s", {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": gbs / HBM_PEAK_GBS, "traffic": None}

    def per_shape(self, torch, steps, warmup):
        out = []
        for tokens, ref in MOE_REFERENCE_US.items():
            self.prepare(tokens)
            s = time_launches(torch, self.step, steps, warmup)
            ss = time_launches(torch, self.step_sort, steps, warmup)
            out.append({"tokens": tokens, "experts_hit": self.experts_hit, "replay_us_per_launch": s * 1e6,
                        "sorting_us": ss * 1e6, "GB/s": self.bytes() / s / 1e9, "TFLOP/s": self.flops() / s / 1e12,
                        "reference_tuned_us": ref, "reference_over_ours": ref / (s * 1e6)})
        return out

    def cpu_baseline(self, torch):
        return None


ARGS_ROWS = [2048]  # --rows, for --workload norm


def make_workload(name):
    if name == "moe":
        return MoeWorkload()
    if name == "sweep":
        return SweepWorkload()
    if name == "copy":
        return CopyCalibration()
    if name == "stream":
        return StreamCeilings()
    if name == "ceiling":
        return ComputeCeiling()
    if name == "quant":
        return QuantWorkload()
    if name == "prefill":
        return GemmWorkload("prefill", 8192, 36864, 7168,
                            "config 4: prefill blockscale GEMM M=8192 N=36864 K=7168 (fused gate+up FFN), "
                            "fp8 e4m3fn operands, 1x128 / 128x128 fp32 scales, bf16 out")
    if name == "decode":
        return GemmWorkload("decode", 64, 24576, 1536,
                            "config 3: decode blockscale GEMM M=64 N=24576 K=1536 (largest of the nine decode shapes)")
    if name == "fused":
        return FusedWorkload()
    if name == "norm":
        return NormWorkload(ARGS_ROWS[0])
    if name == "decode9":
        return DecodeAllWorkload()
    raise ValueError(name)


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU's throughput; --gpus {args.gpus} is not supported in this build "
              "(nothing on this path uses a second GPU).", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists for the product path)", file=sys.stderr)
        sys.exit(1)
    dev = "cuda:0"
    torch.cuda.set_device(0)

    GemmWorkload.layout = args.layout
    GemmWorkload.rotate_mb = args.rotate_mb
    MoeWorkload.kernel_name = args.kernel_name
    ARGS_ROWS[0] = args.rows
    wl = make_workload(args.workload)
    wl.setup(torch, dev)
    # besides the `warmup` calls asked for, untimed calls for WARM_SECONDS (field `clock_settle_s`): a launch
    # sequence that starts on an idle chip runs its first 20-40 ms at lower clocks
    sec = time_steps(torch, wl.step, args.steps, args.warmup, settle=True)
    value, unit, roof = wl.result(sec)
    if args.workload == "decode":
        # the roofline figure uses the kernel's own duration, `value` the call rate the host achieves
        _, _, roof = wl.result(time_launches(torch, wl.step, args.steps, args.warmup))

    line = {
        "metric": METRIC,
        "value": value,
        "unit": unit,
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "clock_settle_s": WARM_SECONDS,
        "ms_per_step": sec * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn (fp32 scales and accumulation)",
        "data": "synthetic",
        "config": wl.describe(),
        "roofline": roof,
    }
    if args.workload == "prefill":
        line["vs_reference_tuned_csv"] = value / REF_PREFILL_TFLOPS
    if args.workload in ("decode9", "sweep", "moe", "stream", "ceiling"):
        # shape after shape: steps + warmup launches each, in DECODE_SHAPES order
        line["per_shape"] = wl.per_shape(torch, args.steps, args.warmup)
        args.no_also = True

    if not args.no_cpu and args.workload not in ("copy", "stream", "ceiling"):
        torch.set_num_threads(os.cpu_count() or 1)
        line["cpu_baseline"] = wl.cpu_baseline(torch)

    if not args.no_also and args.workload != "copy":
        also = {}
        del wl
        torch.cuda.empty_cache()
        for name in ("quant", "prefill", "prefill_preshuffled", "fused"):
            if name == args.workload:
                continue
            w2 = make_workload(name.split("_")[0])
            if name == "prefill_preshuffled":
                w2.layout = "preshuffled"  # the documented fast path: shuffle_weight once, then the bpreshuffle entry
            w2.setup(torch, dev)
            steps2 = 10 if name.startswith("prefill") else 30
            s2 = time_steps(torch, w2.step, steps2, 3, settle=True)
            v2, u2, r2 = w2.result(s2)
            entry = {"value": v2, "unit": u2, "us_per_step": s2 * 1e6, "steps": steps2, "roofline": r2,
                     "config": w2.describe()}
            if name.startswith("prefill"):
                entry["vs_reference_tuned_csv"] = v2 / REF_PREFILL_TFLOPS
            if name == "fused":
                sn = time_steps(torch, w2.step_norm_only, 30, 3, settle=True)
                gb = w2.norm_bytes() / sn / 1e9
                sc = time_steps(torch, w2.step_norm_cached, 30, 3, settle=True)
                entry["norm_quant"] = {"us": sn * 1e6, "GB/s": gb, "frac_of_hbm_peak": gb / HBM_PEAK_GBS,
                                       "buffers": "rotating through 640 MB: every launch reads its rows from HBM",
                                       "us_with_rows_in_last_level_cache": sc * 1e6}
            if not args.no_cpu and name in ("prefill", "fused"):
                torch.set_num_threads(os.cpu_count() or 1)
                entry["cpu_baseline"] = w2.cpu_baseline(torch)
            also[name] = entry
            del w2
            torch.cuda.empty_cache()
        dec = []
        for (m, n, k) in DECODE_SHAPES:
            w3 = GemmWorkload("decode", m, n, k, "decode")
            w3.setup(torch, dev)
            wall = time_steps(torch, w3.step, 50, 5)
            s3 = time_launches(torch, w3.step, 50, 5)
            gbs = gemm_bytes(m, n, k) / s3 / 1e9
            dec.append({"M": m, "N": n, "K": k, "replay_us_per_launch": s3 * 1e6, "GB/s": gbs,
                        "frac_of_hbm_peak": gbs / HBM_PEAK_GBS, "us_per_call_incl_host_launch": wall * 1e6,
                        "weight_MB_rotated": w3.weight_bytes_rotated / 1e6})
            if not args.no_cpu and (m, n, k) == (64, 24576, 1536):
                dec[-1]["cpu_baseline"] = w3.cpu_baseline(torch)
            del w3
        also["decode"] = dec
        mid = []
        for (m, n, k) in [(256, 4096, 7168), (512, 7168, 2048), (1024, 7168, 2048), (1024, 4096, 7168), (4096, 2112, 7168)]:
            w4 = GemmWorkload("sweep", m, n, k, "sweep")
            w4.rotate_always = True
            w4.setup(torch, dev)
            s4 = time_launches(torch, w4.step, 30, 5)
            mid.append({"M": m, "N": n, "K": k, "replay_us_per_launch": s4 * 1e6, "TFLOP/s": w4.flops() / s4 / 1e12,
                        "reference_tuned_us": SWEEP_REFERENCE_US[(m, n, k)],
                        "reference_over_ours": SWEEP_REFERENCE_US[(m, n, k)] / (s4 * 1e6)})
            del w4
            torch.cuda.empty_cache()
        also["mid_m"] = mid
        w5 = MoeWorkload()
        w5.setup(torch, dev)
        moe = []
        for tokens in (16, 32, 128):
            w5.prepare(tokens)
            s5 = time_launches(torch, w5.step, 16, 3)
            moe.append({"tokens": tokens, "replay_us_per_launch": s5 * 1e6, "GB/s": w5.bytes() / s5 / 1e9,
                        "reference_tuned_us": MOE_REFERENCE_US[tokens],
                        "reference_over_ours": MOE_REFERENCE_US[tokens] / (s5 * 1e6)})
        del w5
        also["moe"] = moe
        line["also"] = also

    print(json.dumps(line))


if __name__ == "__main__":
    main()
