#!/usr/bin/env python3
"""Benchmark of the INT8 linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extras]

One "step" is one pass of BASELINE config 1, the Flux-style MLP in W8A8 rowwise:
    quantise x [4608,3072] -> GEMM with W_up [12288,3072] (+bias)
    quantise h [4608,12288] (synthetic half-normal) -> GEMM with W_dn [3072,12288] (+bias)
with every input already resident in HBM.  The headline `value` is the int8 GEMM work of
the step (2*M*N*K per GEMM) divided by the wall time of the WHOLE step, quantisers
included, in TOP/s.  The JSON line also carries
    roofline      the dominant kernel (the MFMA GEMM) against the dense int8 peak, from HIP
                  events recorded around its launches inside the timed region
    cpu_baseline  the reference's torch CPU path (oracle/torch_path.py) on a bounded sample
    extras        the north-star target shape, the fused rotate+quant kernel against HBM
                  bandwidth, the LoRA merge, and ms per Flux-style DiT block (config 3)
Synthetic data, random-init weights; see make_config() for the seeded recipes.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, TOP/s
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, GB/s


# --------------------------------------------------------------------------- workloads
def _acts(g, M, K, frac, mul):
    x = torch.randn(M, K, generator=g)
    idx = torch.randperm(K, generator=g)[: int(K * frac)]
    x[:, idx] *= mul
    return x.bfloat16()


def make_config(i: int, rows: int | None = None) -> dict:
    """Seeded CPU tensors of BASELINE config i (0..4).  `rows` truncates the token dimension
    (the same leading rows) for CPU-sized checks; weights always have their full shape."""
    g = torch.Generator().manual_seed(1000 + i)
    if i == 0:   # single W8A8 linear, one weight scale, no bias
        x = _acts(g, 4096, 3072, 0.01, 20.0)
        w = (torch.randn(3072, 3072, generator=g) * 0.02).bfloat16()
        return {"x": x[:rows] if rows else x, "w": w, "scale_mode": "tensor", "bias": None}
    if i == 1:   # Flux MLP: up projection on N(0,1) activations, down projection on half-normal ones
        x = _acts(g, 4608, 3072, 0.01, 20.0)
        w_up = torch.randn(12288, 3072, generator=g) * 0.02
        b_up = (torch.randn(12288, generator=g) * 0.01).bfloat16()
        h = torch.randn(4608 if rows is None else rows, 12288, generator=g).abs_().bfloat16()
        w_dn = torch.randn(3072, 12288, generator=g) * 0.02
        b_dn = (torch.randn(3072, generator=g) * 0.01).bfloat16()
        return {"x": x[:rows] if rows else x, "w_up": w_up, "b_up": b_up, "h": h, "w_dn": w_dn, "b_dn": b_dn}
    if i == 2:   # QuaRot: heavy outliers, 128-block rotation, width 3840
        x = _acts(g, 4096, 3840, 0.02, 50.0)
        w = torch.randn(3840, 3840, generator=g) * 0.02
        return {"x": x[:rows] if rows else x, "w": w, "rotate": True}
    if i == 3:   # one double-stream DiT block, width 3072: shapes only (weights are drawn on the device)
        return {"hidden": 3072, "heads": 24, "img": 4096, "txt": 512,
                "linears": {"qkv": (9216, 3072), "proj": (3072, 3072), "up": (12288, 3072), "down": (3072, 12288),
                            "adaln": (18432, 3072)}}
    if i == 4:   # stochastic LoRA merge, then a skinny GEMM
        w = torch.randn(12288, 3072, generator=g) * 0.02
        down = torch.randn(32, 3072, generator=g) * 0.01
        up = torch.randn(12288, 32, generator=g) * 0.01
        noise = torch.rand(12288, 3072, generator=g)
        x = _acts(g, 256, 3072, 0.01, 20.0)
        return {"w": w, "up": up, "down": down, "alpha": 32.0, "noise": noise, "x": x}
    raise ValueError(i)


# HBM-side bytes per GEMM launch: measured by this run where rocprofv3 is at hand (live_traffic: two child runs of
# this file under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`, started before this process touches the GPU, each
# calibrated on a device copy of known size in the same run), else taken from profiles/gemm_hbm_traffic.txt, the
# figures of the same procedure per shape and tile configuration (used only while the library still picks the tile
# configuration a row was measured with).
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gemm_hbm_traffic.txt")
TRAFFIC_SHAPES = ((4608, 3072, 3072), (4608, 12288, 3072), (4608, 3072, 12288))
TRAFFIC_LAUNCHES = 6
TRAFFIC_COPY_BYTES = 20 * 1024 * 1024


def traffic_probe(L, dev):
    """What a child run under rocprofv3 --pmc executes: five device copies of TRAFFIC_COPY_BYTES (the calibration), then
    TRAFFIC_LAUNCHES launches of the GEMM for each of TRAFFIC_SHAPES in that order, nothing else from this library's
    GEMM kernel."""
    src = torch.randint(0, 255, (TRAFFIC_COPY_BYTES,), dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    for _ in range(5):
        dst.copy_(src)
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(5)
    for (M, N, K) in TRAFFIC_SHAPES:
        q, s = L.quant_rowwise(_acts(g, M, K, 0.01, 20.0).to(dev))
        wq, ws = L.quant_rowwise(torch.randn(N, K, device=dev) * 0.02)
        b = (torch.randn(N, device=dev) * 0.01).bfloat16()
        y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        torch.cuda.synchronize()
        for _ in range(TRAFFIC_LAUNCHES):
            L.linear_w8a8(q, s, wq, ws, b, torch.bfloat16, L.EPI_TORCH, y)
        torch.cuda.synchronize()
        del q, s, wq, ws, y


def live_traffic():
    """-> ({(M, N, K): HBM-side bytes per launch}, {"fetch_factor", "write_factor"}, None) measured now, or
    (None, None, reason).  Must run before this process initialises the GPU (it starts child processes)."""
    import csv
    import glob
    import shutil
    import subprocess
    import tempfile

    # Under a profiler this process has the GPU initialised before main() runs (the profiler's preloaded library does
    # that), and a process in that state must not start other programs: the figures then come from the profile file.
    if "rocprof" in os.environ.get("LD_PRELOAD", "").lower() or any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ):
        return None, None, "this run is itself under a profiler"
    exe = shutil.which("rocprofv3")
    if exe is None:
        return None, None, "rocprofv3 not found"
    kib = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        out = tempfile.mkdtemp(prefix="i8f_pmc_", dir="/tmp")
        cmd = [exe, "--pmc", counter, "--output-format", "csv", "-d", out, "-o", "t", "--", sys.executable,
               os.path.abspath(__file__), "--traffic-probe"]
        try:
            p = subprocess.run(cmd, cwd="/tmp", env={**os.environ, "TMPDIR": "/tmp"}, timeout=180, capture_output=True, text=True)
        except (subprocess.TimeoutExpired, OSError) as e:
            shutil.rmtree(out, ignore_errors=True)
            return None, None, f"rocprofv3 --pmc {counter}: {type(e).__name__}"
        files = glob.glob(os.path.join(out, "**", "*counter_collection.csv"), recursive=True)
        if p.returncode != 0 or not files:
            shutil.rmtree(out, ignore_errors=True)
            return None, None, f"rocprofv3 --pmc {counter} failed (exit {p.returncode})"
        rows = [r for r in csv.DictReader(open(files[0])) if r.get("Counter_Name") == counter]
        shutil.rmtree(out, ignore_errors=True)
        rows.sort(key=lambda r: int(r["Dispatch_Id"]))
        copies = [float(r["Counter_Value"]) for r in rows if "copyBuffer" in r["Kernel_Name"]]
        gemms = [float(r["Counter_Value"]) for r in rows if "gemm_i8_kernel" in r["Kernel_Name"]]
        if len(copies) < 3 or len(gemms) != TRAFFIC_LAUNCHES * len(TRAFFIC_SHAPES) or statistics.median(copies) <= 0:
            return None, None, f"rocprofv3 --pmc {counter}: {len(copies)} copy and {len(gemms)} GEMM dispatches in the trace, not what the probe launches"
        kib[counter] = (TRAFFIC_COPY_BYTES / 1024 / statistics.median(copies[1:]),
                        [statistics.median(gemms[i * TRAFFIC_LAUNCHES + 1:(i + 1) * TRAFFIC_LAUNCHES]) for i in range(len(TRAFFIC_SHAPES))])
    f_fetch, f_write = kib["FETCH_SIZE"][0], kib["WRITE_SIZE"][0]
    traffic = {shape: int((kib["FETCH_SIZE"][1][i] * f_fetch + kib["WRITE_SIZE"][1][i] * f_write) * 1024)
               for i, shape in enumerate(TRAFFIC_SHAPES)}
    return traffic, {"fetch_factor": round(f_fetch, 3), "write_factor": round(f_write, 3)}, None


LIVE_TRAFFIC = None   # filled by main() before the GPU is touched


def gemm_traffic(L, M, N, K):
    """HBM-side bytes of one M x N x K GEMM launch: this run's own measurement, else the profile's, else None (with
    the reason)."""
    if LIVE_TRAFFIC is not None and (M, N, K) in LIVE_TRAFFIC:
        return LIVE_TRAFFIC[(M, N, K)], None
    tile = L.gemm_tile(M, N, K)
    try:
        lines = open(TRAFFIC_FILE).read().splitlines()
    except OSError:
        return None, "profiles/gemm_hbm_traffic.txt is missing"
    f_fetch = f_write = None
    row = None
    for ln in lines:
        t = ln.split()
        if len(t) >= 5 and t[0] == "calibration":
            f_fetch, f_write = float(t[2]), float(t[4])
        if len(t) >= 8 and t[0] == "traffic" and t[1] == f"{M}x{N}x{K}":
            row = (t[3], float(t[5]), float(t[7]))
    if row is None or f_fetch is None:
        return None, f"no row for {M}x{N}x{K} in profiles/gemm_hbm_traffic.txt"
    if row[0] != f"{tile[0]}x{tile[1]}":
        return None, f"the profile row was measured with tile {row[0]}, the library now picks {tile[0]}x{tile[1]}: not measured for this tile"
    return int((row[1] * f_fetch + row[2] * f_write) * 1024), None


def gemm_algorithmic_bytes(M, N, K, out_bytes=2, bias=True):
    return M * K + N * K + out_bytes * M * N + 4 * M + 4 * N + (2 * N if bias else 0)


# --------------------------------------------------------------------------- timing helpers
def _events(n):
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def time_kernel(fn, iters=50, warmup=5, sets=1, burst=1, ramp_s=0.05):
    """Median / min / mean device time of ONE fn(set_index) launch in microseconds, from HIP events on
    the launch stream.  `sets` distinct argument sets are cycled so that a bandwidth kernel does not
    find its operands in the 256 MB memory-side cache.  With burst > 1 each event pair brackets that
    many back-to-back launches and the time is divided by it: for kernels of a few microseconds a
    pair of events around a single launch mostly measures the gap between dispatches."""
    for i in range(warmup):
        fn(i % sets)
    torch.cuda.synchronize()
    t_ramp, i = time.perf_counter(), 0
    while time.perf_counter() - t_ramp < ramp_s:   # keep the GPU at its sustained clocks (see main)
        for _ in range(20):
            fn(i % sets)
            i += 1
        torch.cuda.synchronize()
    starts, stops = _events(iters), _events(iters)
    k = 0
    for i in range(iters):
        starts[i].record()
        for _ in range(burst):
            fn(k % sets)
            k += 1
        stops[i].record()
    torch.cuda.synchronize()
    us = [s.elapsed_time(e) * 1e3 / burst for s, e in zip(starts, stops)]
    return {"median_us": statistics.median(us), "min_us": min(us), "mean_us": statistics.fmean(us)}


# --------------------------------------------------------------------------- the step
class MlpStep:
    """Config 1 resident on the device."""

    def __init__(self, L, dev):
        c = make_config(1)
        self.L = L
        self.x = c["x"].to(dev)
        self.h = c["h"].to(dev)
        self.wq_up, self.ws_up = L.quant_rowwise(c["w_up"].to(dev))
        self.wq_dn, self.ws_dn = L.quant_rowwise(c["w_dn"].to(dev))
        self.b_up, self.b_dn = c["b_up"].to(dev), c["b_dn"].to(dev)
        M = self.x.shape[0]
        self.y_up = torch.empty(M, 12288, dtype=torch.bfloat16, device=dev)
        self.y_dn = torch.empty(M, 3072, dtype=torch.bfloat16, device=dev)
        self.gemm_ops = 2 * M * 12288 * 3072   # per GEMM launch; both GEMMs of the step have this many
        self.quant_bytes = M * 3072 * 3 + 4 * M + M * 12288 * 3 + 4 * M

    def run(self, ev=None):
        L = self.L
        q, s = L.quant_rowwise(self.x)
        if ev:
            ev[0].record()
        L.linear_w8a8(q, s, self.wq_up, self.ws_up, self.b_up, torch.bfloat16, L.EPI_TORCH, self.y_up)
        if ev:
            ev[1].record()
        q2, s2 = L.quant_rowwise(self.h)
        if ev:
            ev[2].record()
        L.linear_w8a8(q2, s2, self.wq_dn, self.ws_dn, self.b_dn, torch.bfloat16, L.EPI_TORCH, self.y_dn)
        if ev:
            ev[3].record()


# --------------------------------------------------------------------------- extras
def extras(L, dev, quick=False):
    out = {}
    iters = 20 if quick else 100
    g = torch.Generator().manual_seed(99)

    # north-star target shape: M=4608, K=N=3072, W8A8 rowwise.  Warm: the same 23.6 MB of operands in a loop (they
    # sit in the 256 MB memory-side cache).  Cold: 12 operand sets in turn (283 MB of int8 operands + 340 MB of
    # outputs), which is what a layer inside a model sees.
    M, N, K = 4608, 3072, 3072
    x = _acts(g, M, K, 0.01, 20.0).to(dev)
    wq, ws = L.quant_rowwise((torch.randn(N, K, generator=g) * 0.02).to(dev))
    q, s = L.quant_rowwise(x)
    y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    t = time_kernel(lambda i: L.linear_w8a8(q, s, wq, ws, None, torch.bfloat16, L.EPI_TORCH, y), max(10, iters // 4), burst=8)
    nset = 12
    cq = [q] + [L.quant_rowwise(_acts(g, M, K, 0.01, 20.0).to(dev)) [0] for _ in range(nset - 1)]
    cw = [wq] + [L.quant_rowwise(torch.randn(N, K, device=dev) * 0.02)[0] for _ in range(nset - 1)]
    cy = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(nset)]
    tc = time_kernel(lambda i: L.linear_w8a8(cq[i], s, cw[i], ws, None, torch.bfloat16, L.EPI_TORCH, cy[i]), max(10, iters // 4),
                     sets=nset, burst=nset)
    ops = 2 * M * N * K
    tops, tops_c = ops / t["median_us"] / 1e6, ops / tc["median_us"] / 1e6
    out["target_gemm_4608x3072x3072"] = {"median_us": round(t["median_us"], 2), "min_us": round(t["min_us"], 2),
                                          "tops": round(tops, 1), "frac_of_int8_peak": round(tops / PEAK_INT8_TOPS, 4),
                                          "cold_operands_median_us": round(tc["median_us"], 2), "cold_operands_tops": round(tops_c, 1),
                                          "cold_operands_frac_of_int8_peak": round(tops_c / PEAK_INT8_TOPS, 4),
                                          "tile": "%dx%d" % L.gemm_tile(M, N, K)[:2]}
    # the vendor library's int8 product on the same box and operands (torch._int_mm = hipBLASLt: int32 result, no
    # epilogue, so it does less than the launch above), warm loop like the first figure; bench-only, not product code
    try:
        wt = wq.t()
        t_v = time_kernel(lambda i: torch._int_mm(q, wt), max(10, iters // 4), burst=8)
        out["target_gemm_4608x3072x3072"]["vendor_int_mm_median_us"] = round(t_v["median_us"], 2)
        out["target_gemm_4608x3072x3072"]["vendor_int_mm_note"] = "torch._int_mm(q, w.T): int32 accumulators only, no dequantisation epilogue"
    except Exception as e:   # a torch build without the routine says so in the line
        out["target_gemm_4608x3072x3072"]["vendor_int_mm_median_us"] = None
        out["target_gemm_4608x3072x3072"]["vendor_int_mm_note"] = f"torch._int_mm unavailable: {type(e).__name__}"
    del cq, cw, cy

    # fused rotate + quant at the same shape, cycling 8 buffer sets (> 256 MB in total), bursts of 8
    # launches per event pair; a plain device copy of the same byte count is timed beside them
    sets = 8
    xs = [x] + [_acts(g, M, K, 0.01, 20.0).to(dev) for _ in range(sets - 1)]
    qs = [torch.empty(M, K, dtype=torch.int8, device=dev) for _ in range(sets)]
    ss = [torch.empty(M, 1, dtype=torch.float32, device=dev) for _ in range(sets)]
    lib, ptr, stream = L.lib(), L._ptr, L._stream(x)
    qbytes = M * K * 3 + 4 * M
    reps = max(5, iters // 8)
    for name, rb in (("quant_4608x3072", 0), ("rotate_quant_4608x3072", 128)):
        # argument tuples built beforehand: the launches are 7-9 us apart and the host must stay ahead of them
        qargs = [(ptr(xs[i]), L.BF16, M, K, K, rb, ptr(qs[i]), ptr(ss[i]), stream) for i in range(sets)]

        def call(i, qargs=qargs, fn=lib.i8f_quant_rowwise):
            rc = fn(*qargs[i])
            assert rc == 0, rc
        t = time_kernel(call, reps, sets=sets, burst=sets)
        gbs = qbytes / t["median_us"] / 1e3
        out[name] = {"median_us": round(t["median_us"], 2), "min_us": round(t["min_us"], 2), "gbs": round(gbs, 1),
                     "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4), "bytes": qbytes, "buffer_sets": sets}
    half = qbytes // 2
    srcs = [xs[i].view(torch.uint8).reshape(-1)[:half] for i in range(sets)]
    dsts = [torch.empty(half, dtype=torch.uint8, device=dev) for _ in range(sets)]
    t = time_kernel(lambda i: dsts[i].copy_(srcs[i]), reps, sets=sets, burst=sets)
    out["device_copy_same_bytes"] = {"median_us": round(t["median_us"], 2), "gbs": round(2 * half / t["median_us"] / 1e3, 1),
                                     "note": "torch copy_ of 21.2 MB -> 21.2 MB over the same rotation of buffers, for comparison"}
    # the quantiser with the elementwise operation in front of the layer applied on the fly, against the same
    # operation as a torch kernel of its own followed by the plain quantiser
    import torch.nn.functional as F
    sc, sh = (torch.randn(1, K, device=dev) * 0.3).bfloat16(), torch.randn(1, K, device=dev).bfloat16()
    def fused_call(i, kind, src, dq, ds, cols):
        rc = lib.i8f_quant_rowwise_prologue(ptr(src[i]), L.BF16, M, cols, cols, kind, ptr(sc), ptr(sh), M, 0, ptr(dq[i]), ptr(ds[i]), stream)
        assert rc == 0, rc

    def plain_call(src, dq, ds, cols):
        rc = lib.i8f_quant_rowwise(ptr(src), L.BF16, M, cols, cols, 0, ptr(dq), ptr(ds), stream)
        assert rc == 0, rc

    def mod_unfused(i):
        plain_call((1 + sc) * xs[i] + sh, qs[i], ss[i], K)

    t_f = time_kernel(lambda i: fused_call(i, L.PRO_MODULATE, xs, qs, ss, K), reps, sets=sets, burst=sets)
    t_u = time_kernel(mod_unfused, reps, sets=sets, burst=sets)
    out["modulate_quant_4608x3072"] = {"fused_median_us": round(t_f["median_us"], 2), "torch_ops_then_quant_median_us": round(t_u["median_us"], 2),
                                       "fused_gbs": round(qbytes / t_f["median_us"] / 1e3, 1)}

    # the whole adaLN producer of a DiT block, LayerNorm without affine and the modulation, inside the quantiser
    def norm_fused(i):
        rc = lib.i8f_quant_rowwise_norm_modulate(ptr(xs[i]), L.BF16, M, K, K, 1e-6, ptr(sc), ptr(sh), M, 0, 0, ptr(qs[i]), ptr(ss[i]), stream)
        assert rc == 0, rc

    def norm_unfused(i):
        plain_call((1 + sc) * F.layer_norm(xs[i], (K,), eps=1e-6) + sh, qs[i], ss[i], K)

    t_f = time_kernel(norm_fused, reps, sets=sets, burst=sets)
    t_u = time_kernel(norm_unfused, reps, sets=sets, burst=sets)
    out["norm_modulate_quant_4608x3072"] = {"fused_median_us": round(t_f["median_us"], 2), "torch_ops_then_quant_median_us": round(t_u["median_us"], 2),
                                            "fused_gbs": round(qbytes / t_f["median_us"] / 1e3, 1),
                                            "note": "layer_norm (no affine) + (1 + scale) * y + shift + quantise: one launch against torch's four kernels and the quantiser"}
    hs = [torch.randn(M, 12288, device=dev).bfloat16() for _ in range(3)]
    hq = [torch.empty(M, 12288, dtype=torch.int8, device=dev) for _ in range(3)]

    def gelu_unfused(i):
        plain_call(F.gelu(hs[i], approximate="tanh"), hq[i], ss[i], 12288)

    t_p = time_kernel(lambda i: plain_call(hs[i], hq[i], ss[i], 12288), reps, sets=3, burst=3)
    t_f = time_kernel(lambda i: fused_call(i, L.PRO_GELU_TANH, hs, hq, ss, 12288), reps, sets=3, burst=3)
    t_u = time_kernel(gelu_unfused, reps, sets=3, burst=3)
    hbytes = M * 12288 * 3 + 4 * M
    out["gelu_quant_4608x12288"] = {"fused_median_us": round(t_f["median_us"], 2), "torch_gelu_then_quant_median_us": round(t_u["median_us"], 2),
                                    "plain_quant_median_us": round(t_p["median_us"], 2), "fused_gbs": round(hbytes / t_f["median_us"] / 1e3, 1),
                                    "plain_gbs": round(hbytes / t_p["median_us"] / 1e3, 1),
                                    "note": "config 1's down-projection input: the fused form never writes the 113 MB activated tensor"}
    t_f = time_kernel(lambda i: fused_call(i, L.PRO_GELU_ERF, hs, hq, ss, 12288), reps, sets=3, burst=3)
    t_u = time_kernel(lambda i: plain_call(F.gelu(hs[i]), hq[i], ss[i], 12288), reps, sets=3, burst=3)
    out["gelu_erf_quant_4608x12288"] = {"fused_median_us": round(t_f["median_us"], 2), "torch_gelu_then_quant_median_us": round(t_u["median_us"], 2),
                                        "fused_gbs": round(hbytes / t_f["median_us"] / 1e3, 1),
                                        "note": "GELU in its exact form (erf), 13 vector + 2 transcendental instructions per element"}

    # RMSNorm with its weight and the scale-only modulation behind it (z-image's modulate(norm(x), scale), width 3840)
    Kz = 3840
    zs = [torch.randn(M, Kz, device=dev).bfloat16() for _ in range(sets)]
    zq = [torch.empty(M, Kz, dtype=torch.int8, device=dev) for _ in range(sets)]
    nw, zsc = (torch.randn(Kz, device=dev) * 0.2 + 1).bfloat16(), (torch.randn(1, Kz, device=dev) * 0.3).bfloat16()

    def rms_fused(i):
        rc = lib.i8f_quant_rowwise_rms_norm(ptr(zs[i]), L.BF16, M, Kz, Kz, 1e-5, ptr(nw), ptr(zsc), None, M, 0, 0, ptr(zq[i]), ptr(ss[i]), stream)
        assert rc == 0, rc

    def rms_unfused(i):
        plain_call(F.rms_norm(zs[i], (Kz,), nw, 1e-5) * (1 + zsc), zq[i], ss[i], Kz)

    t_f = time_kernel(rms_fused, reps, sets=sets, burst=sets)
    t_u = time_kernel(rms_unfused, reps, sets=sets, burst=sets)
    out["rms_norm_modulate_quant_4608x3840"] = {"fused_median_us": round(t_f["median_us"], 2), "torch_ops_then_quant_median_us": round(t_u["median_us"], 2),
                                                "fused_gbs": round((M * Kz * 3 + 4 * M) / t_f["median_us"] / 1e3, 1),
                                                "note": "rms_norm(x, w) * (1 + scale) + quantise: one launch against torch's three kernels and the quantiser"}
    del zs, zq

    # the input of linear2 of a single-stream block, cat((attn [M,3072], gelu(mlp [M,12288])), -1): one launch that reads
    # both operands and writes int8, against torch's gelu and cat kernels followed by the plain quantiser
    Kc = K + 12288
    cq = [torch.empty(M, Kc, dtype=torch.int8, device=dev) for _ in range(3)]

    def concat_fused(i):
        rc = lib.i8f_quant_rowwise_concat_gelu(ptr(xs[i]), L.BF16, M, K, K, ptr(hs[i]), 12288, 12288, 0, ptr(cq[i]), ptr(ss[i]), stream)
        assert rc == 0, rc

    def concat_unfused(i):
        plain_call(torch.cat((xs[i], F.gelu(hs[i], approximate="tanh")), -1), cq[i], ss[i], Kc)

    t_f = time_kernel(concat_fused, reps, sets=3, burst=3)
    t_u = time_kernel(concat_unfused, reps, sets=3, burst=3)
    cbytes = M * Kc * 3 + 4 * M
    out["concat_gelu_quant_4608x3072+12288"] = {"fused_median_us": round(t_f["median_us"], 2), "torch_ops_then_quant_median_us": round(t_u["median_us"], 2),
                                                "fused_gbs": round(cbytes / t_f["median_us"] / 1e3, 1),
                                                "note": "neither the activated tensor nor the 141 MB concatenation is written"}
    del hq, cq
    del xs, qs, ss, srcs, dsts, hs

    # config 4: stochastic LoRA merge (rank 32 rebuilt in the kernel, float noise) and the skinny GEMM
    c = make_config(4)
    w4q, w4s = L.quant_rowwise(c["w"].to(dev))
    up, down = c["up"].to(dev), c["down"].to(dev)
    Nw, Kw, r = 12288, 3072, 32
    noises = [c["noise"].to(dev)] + [torch.rand(Nw, Kw, device=dev) for _ in range(2)]
    outs = [torch.empty_like(w4q) for _ in range(3)]
    mbytes = Nw * Kw * 6 + 4 * Nw + 4 * r * (Nw + Kw)
    w4s_row = w4s.reshape(-1).contiguous()

    def merge_call(i):
        rc = lib.i8f_lora_merge_sr(ptr(w4q), ptr(w4s_row), 0.0, L.SCALE_ROW, None, ptr(up), ptr(down), r, 1.0, ptr(noises[i]), Nw, Kw,
                                   ptr(outs[i]), stream)
        assert rc == 0, rc

    t = time_kernel(merge_call, max(10, iters // 4), sets=3, burst=3)
    gbs = mbytes / t["median_us"] / 1e3
    out["lora_merge_fused_12288x3072_r32"] = {"median_us": round(t["median_us"], 2), "gbs": round(gbs, 1),
                                              "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4), "bytes": mbytes}
    x4 = c["x"].to(dev)
    q4, s4 = L.quant_rowwise(x4)
    y4 = torch.empty(256, Nw, dtype=torch.bfloat16, device=dev)
    t = time_kernel(lambda i: L.linear_w8a8(q4, s4, outs[0], w4s, None, torch.bfloat16, L.EPI_TORCH, y4), max(10, iters // 4), burst=8)
    out["skinny_gemm_256x12288x3072"] = {"median_us": round(t["median_us"], 2),
                                         "tops": round(2 * 256 * Nw * Kw / t["median_us"] / 1e6, 1)}
    # the load-time and patch-time forms of the same machinery, at config 4's weight shape: stochastic rounding of a
    # given float delta alone and merged into the weights, the 128-block rotation of a float delta, the rotating
    # quantiser on float32 weights (on-the-fly quantisation of a QuaRot layer) and the one-scale quantiser
    nk = Nw * Kw
    deltas = [torch.randn(Nw, Kw, device=dev) * 0.003 for _ in range(2)]
    rot_out = torch.empty(Nw, Kw, device=dev)
    dq = torch.empty(Nw, Kw, dtype=torch.int8, device=dev)
    sw1 = torch.empty(Nw, 1, device=dev)
    few = max(6, iters // 8)

    def load_time(name, call, nbytes, sets=2):
        t = time_kernel(call, few, sets=sets, burst=sets)
        gbs = nbytes / t["median_us"] / 1e3
        out[name] = {"median_us": round(t["median_us"], 2), "gbs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4),
                     "bytes": nbytes}

    def chk(rc):
        assert rc == 0, rc

    load_time("sr_quant_delta_12288x3072", lambda i: chk(lib.i8f_sr_quant_delta(
        ptr(deltas[i]), ptr(w4s_row), 0.0, L.SCALE_ROW, ptr(noises[i]), Nw, Kw, ptr(dq), stream)), nk * 9 + 4 * Nw)
    load_time("lora_merge_given_delta_12288x3072", lambda i: chk(lib.i8f_lora_merge_sr(
        ptr(w4q), ptr(w4s_row), 0.0, L.SCALE_ROW, ptr(deltas[i]), None, None, 0, 1.0, ptr(noises[i]), Nw, Kw, ptr(outs[i]), stream)),
        nk * 10 + 4 * Nw)
    load_time("rotate128_f32_12288x3072", lambda i: chk(lib.i8f_rotate128(ptr(deltas[i]), L.F32, Nw, Kw, Kw, ptr(rot_out), stream)), nk * 8)
    load_time("weight_rotate_quant_f32_12288x3072", lambda i: chk(lib.i8f_quant_rowwise(
        ptr(deltas[i]), L.F32, Nw, Kw, Kw, 128, ptr(dq), ptr(sw1), stream)), nk * 5 + 4 * Nw)
    wb = [(torch.randn(Nw, Kw, device=dev) * 0.02).bfloat16() for _ in range(4)]
    load_time("weight_quant_one_scale_bf16_12288x3072", lambda i: L.quant_tensorwise(wb[i]), nk * 5 + 4, sets=4)
    out["weight_quant_one_scale_bf16_12288x3072"]["note"] = "two passes over the tensor (absmax, then quantise): 2+2 bytes read, 1 written per element"
    del noises, outs, deltas, rot_out, dq, wb

    # few tiles and a long K (the text stream's down-projection of a DiT block): the K range of a tile dealt over
    # several workgroups through a workspace, against the same call without one; weights rotate through > 256 MB
    Ms, Ns, Ks, nset = 512, 3072, 12288, 8
    sq = [torch.randint(-127, 128, (Ms, Ks), dtype=torch.int8, device=dev) for _ in range(nset)]
    sw = [torch.randint(-127, 128, (Ns, Ks), dtype=torch.int8, device=dev) for _ in range(nset)]
    sxs, sws = torch.rand(Ms, 1, device=dev) * 0.01 + 0.001, torch.rand(Ns, device=dev) * 0.01 + 0.001
    sy = [torch.empty(Ms, Ns, dtype=torch.bfloat16, device=dev) for _ in range(nset)]
    work = torch.zeros(lib.i8f_linear_w8a8_workspace_bytes(), dtype=torch.uint8, device=dev)
    sargs = [(ptr(sq[i]), ptr(sxs), ptr(sw[i]), ptr(sws), 0.0, L.SCALE_ROW, None, 0, None, ptr(sy[i]), L.BF16, Ms, Ns, Ks, L.EPI_TORCH)
             for i in range(nset)]

    def split_call(i, ws_ptr, ws_bytes):
        rc = lib.i8f_linear_w8a8_splitk(*sargs[i], ws_ptr, ws_bytes, stream)
        assert rc == 0, rc

    t_one = time_kernel(lambda i: split_call(i, None, 0), max(10, iters // 4), sets=nset, burst=nset)
    t_split = time_kernel(lambda i: split_call(i, ptr(work), work.numel()), max(10, iters // 4), sets=nset, burst=nset)
    out["k_split_gemm_512x3072x12288"] = {"one_workgroup_per_tile_median_us": round(t_one["median_us"], 2),
                                          "k_split_median_us": round(t_split["median_us"], 2),
                                          "k_split_tops": round(2 * Ms * Ns * Ks / t_split["median_us"] / 1e6, 1),
                                          "note": "weights from HBM (8 sets of 37.7 MB); results are bit-identical"}
    del sq, sw, sy, work

    # dynamic (unmerged) LoRA side branch, rank 32, on config 1's up-projection: the second rank-r product and the
    # addition inside the GEMM epilogue, against torch's F.linear for the [M,N] side tensor + the addition in the epilogue
    Mu, Nu, Ku, r = 4608, 12288, 3072, 32
    xu = _acts(g, Mu, Ku, 0.01, 20.0).to(dev)
    wqu, wsu = L.quant_rowwise(torch.randn(Nu, Ku, device=dev) * 0.02)
    bu = (torch.randn(Nu, device=dev) * 0.01).bfloat16()
    lA, lB = (torch.randn(r, Ku, device=dev) * 0.02).bfloat16(), (torch.randn(Nu, r, device=dev) * 0.02).bfloat16()
    qu, su = L.quant_rowwise(xu)
    yu = torch.empty(Mu, Nu, dtype=torch.bfloat16, device=dev)

    def lora_fused(_i):
        L.linear_w8a8_lora(qu, su, wqu, wsu, bu, F.linear(xu, lA), lB, None, torch.bfloat16, L.EPI_TORCH, yu)

    def lora_side_tensor(_i):
        L.linear_w8a8(qu, su, wqu, wsu, bu, torch.bfloat16, L.EPI_TORCH, yu, addend=F.linear(F.linear(xu, lA), lB))

    t_plain = time_kernel(lambda i: L.linear_w8a8(qu, su, wqu, wsu, bu, torch.bfloat16, L.EPI_TORCH, yu), max(10, iters // 4))
    t_f = time_kernel(lora_fused, max(10, iters // 4))
    t_u = time_kernel(lora_side_tensor, max(10, iters // 4))
    out["dynamic_lora_r32_4608x12288x3072"] = {"gemm_alone_median_us": round(t_plain["median_us"], 2),
                                               "side_branch_in_epilogue_median_us": round(t_f["median_us"], 2),
                                               "side_tensor_then_add_in_epilogue_median_us": round(t_u["median_us"], 2),
                                               "note": "both include the first product x @ A.T in torch (9.5 us of GPU time); the side operands of a tile are staged in LDS and every tile configuration has the side form (here 288x256)"}
    del xu, wqu, yu

    # the residual update of an adaLN-Zero block behind config 1's down-projection, x + gate * linear(h): both elementwise
    # operations inside the GEMM epilogue against the plain layer followed by torch's two kernels
    Mg, Ng, Kg = 4608, 3072, 12288
    hq, hs_ = L.quant_rowwise(_acts(g, Mg, Kg, 0.01, 20.0).to(dev))
    wqg, wsg = L.quant_rowwise(torch.randn(Ng, Kg, device=dev) * 0.02)
    bg = (torch.randn(Ng, device=dev) * 0.01).bfloat16()
    gate_v = torch.randn(1, Ng, device=dev).bfloat16()
    res = torch.randn(Mg, Ng, device=dev).bfloat16()
    og = torch.empty(Mg, Ng, dtype=torch.bfloat16, device=dev)

    def gated_fused(_i):
        L.linear_w8a8(hq, hs_, wqg, wsg, bg, torch.bfloat16, L.EPI_TORCH, og, addend=res, gate=gate_v)

    def gated_unfused(_i):
        y = L.linear_w8a8(hq, hs_, wqg, wsg, bg, torch.bfloat16, L.EPI_TORCH, og)
        return res + gate_v * y

    t_gf = time_kernel(gated_fused, max(10, iters // 4))
    t_gu = time_kernel(gated_unfused, max(10, iters // 4))
    t_gp = time_kernel(lambda i: L.linear_w8a8(hq, hs_, wqg, wsg, bg, torch.bfloat16, L.EPI_TORCH, og), max(10, iters // 4))
    out["gated_residual_4608x3072x12288"] = {"gemm_alone_median_us": round(t_gp["median_us"], 2),
                                             "gate_and_residual_in_epilogue_median_us": round(t_gf["median_us"], 2),
                                             "gemm_then_torch_mul_and_add_median_us": round(t_gu["median_us"], 2),
                                             "note": "x + gate * linear(h) with bf16 tensors: the fused form reads the residual (28 MB) inside the "
                                                     "GEMM; torch's two kernels move 142 MB"}
    del hq, wqg, res, og

    # The MLP half of an adaLN-Zero block on config 1's shapes, x + gate * down(gelu(up((1 + scale) * norm(x) + shift))):
    # every elementwise operation inside a quantiser or an epilogue (4 launches) against the same two quantised layers
    # with torch's kernels around them (LayerNorm, modulation, GELU, gate, residual: 8 more launches)
    Mm, Dm, Hm = 4608, 3072, 12288
    xm = _acts(g, Mm, Dm, 1.0, 20.0).to(dev)
    w_up, s_up = L.quant_rowwise(torch.randn(Hm, Dm, device=dev) * 0.02)
    w_dn, s_dn = L.quant_rowwise(torch.randn(Dm, Hm, device=dev) * 0.02)
    b_up, b_dn = (torch.randn(Hm, device=dev) * 0.01).bfloat16(), (torch.randn(Dm, device=dev) * 0.01).bfloat16()
    m_sc, m_sh, m_gate = ((torch.randn(1, Dm, device=dev) * 0.3).bfloat16() for _ in range(3))
    h_buf = torch.empty(Mm, Hm, dtype=torch.bfloat16, device=dev)
    o_buf = torch.empty(Mm, Dm, dtype=torch.bfloat16, device=dev)

    def mlp_fused(_i):
        q1, s1 = L.quant_rowwise(xm, prologue=L.PRO_NORM_MODULATE, mod_scale=m_sc, mod_shift=m_sh, eps=1e-6)
        L.linear_w8a8(q1, s1, w_up, s_up, b_up, torch.bfloat16, L.EPI_TORCH, h_buf)
        q2, s2 = L.quant_rowwise(h_buf, prologue=L.PRO_GELU_TANH)
        L.linear_w8a8(q2, s2, w_dn, s_dn, b_dn, torch.bfloat16, L.EPI_TORCH, o_buf, addend=xm, gate=m_gate)

    def mlp_unfused(_i):
        z = (1 + m_sc) * F.layer_norm(xm, (Dm,), eps=1e-6) + m_sh
        q1, s1 = L.quant_rowwise(z)
        L.linear_w8a8(q1, s1, w_up, s_up, b_up, torch.bfloat16, L.EPI_TORCH, h_buf)
        q2, s2 = L.quant_rowwise(F.gelu(h_buf, approximate="tanh"))
        y = L.linear_w8a8(q2, s2, w_dn, s_dn, b_dn, torch.bfloat16, L.EPI_TORCH, o_buf)
        return xm + m_gate * y

    t_mf = time_kernel(mlp_fused, max(10, iters // 4))
    t_mu = time_kernel(mlp_unfused, max(10, iters // 4))
    out["adaln_zero_mlp_4608x3072x12288"] = {"ms_all_elementwise_work_fused": round(t_mf["median_us"] / 1e3, 4),
                                             "ms_torch_kernels_around_the_layers": round(t_mu["median_us"] / 1e3, 4),
                                             "note": "x + gate * down(gelu(up((1 + scale) * layer_norm(x) + shift))), bf16, M = 4608: 2 quantiser "
                                                     "launches (LayerNorm + modulation, tanh-GELU) and 2 GEMMs (the second with gate and residual) "
                                                     "against the same layers with 8 torch kernels around them"}
    del w_up, w_dn, h_buf

    # separate q, k and v projections of one tensor (4608 x 3072 -> 3 x 3072): one quantiser for the three GEMMs against
    # the reference's one per Linear.forward
    wf = [L.quant_rowwise(torch.randn(Dm, Dm, device=dev) * 0.02) for _ in range(3)]
    of = [torch.empty(Mm, Dm, dtype=torch.bfloat16, device=dev) for _ in range(3)]

    def fan_shared(_i):
        q1, s1 = L.quant_rowwise(xm)
        for (wq_, ws_), o_ in zip(wf, of):
            L.linear_w8a8(q1, s1, wq_, ws_, None, torch.bfloat16, L.EPI_TORCH, o_)

    def fan_separate(_i):
        for (wq_, ws_), o_ in zip(wf, of):
            q1, s1 = L.quant_rowwise(xm)
            L.linear_w8a8(q1, s1, wq_, ws_, None, torch.bfloat16, L.EPI_TORCH, o_)

    t_fs = time_kernel(fan_shared, max(10, iters // 4))
    t_fp = time_kernel(fan_separate, max(10, iters // 4))
    out["qkv_fanout_4608x3072_to_3x3072"] = {"one_quantiser_median_us": round(t_fs["median_us"], 2),
                                             "a_quantiser_per_layer_median_us": round(t_fp["median_us"], 2),
                                             "note": "forward_fanout / compile_ops.share_quantisation: layers that read one tensor share its int8 rows"}
    del xm, wf, of, o_buf

    # config 2: QuaRot layer (width 3840, 2 % of the channels x50): time of the rotated path and what the
    # rotation buys in accuracy against the bf16 product
    c2 = make_config(2)
    x2, w2 = c2["x"].to(dev), c2["w"].to(dev)
    wq_r, ws_r = L.quant_rowwise(w2, rotate=True)
    wq_p, ws_p = L.quant_rowwise(w2)
    y2 = torch.empty(x2.shape[0], w2.shape[0], dtype=torch.bfloat16, device=dev)

    def rot_linear(_i):
        q_, s_ = L.quant_rowwise(x2, rotate=True)
        L.linear_w8a8(q_, s_, wq_r, ws_r, None, torch.bfloat16, L.EPI_TORCH, y2)

    t = time_kernel(rot_linear, max(10, iters // 4))
    ref2 = x2.float() @ w2.bfloat16().float().T
    rot_linear(0)
    err_rot = ((y2.float() - ref2).norm() / ref2.norm()).item()
    q_, s_ = L.quant_rowwise(x2)
    err_plain = ((L.linear_w8a8(q_, s_, wq_p, ws_p, None, torch.bfloat16, L.EPI_TORCH).float() - ref2).norm() / ref2.norm()).item()
    out["quarot_linear_4096x3840x3840"] = {"median_us": round(t["median_us"], 2),
                                           "tops": round(2 * 4096 * 3840 * 3840 / t["median_us"] / 1e6, 1),
                                           "rel_frobenius_error_rotated": round(err_rot, 5),
                                           "rel_frobenius_error_unrotated": round(err_plain, 5),
                                           "note": "rotate + quantise + GEMM; errors against the bf16 product x @ W.T"}
    del x2, w2, ref2, y2

    # config 3: the linears of one double-stream DiT block (attention stays bf16 and is not counted)
    c3 = make_config(3)
    lin = {m: {} for m in (4096, 512)}   # the image and the text stream have their own weights
    for m in lin:
        for name, (n_out, k_in) in c3["linears"].items():
            wq_, ws_ = L.quant_rowwise(torch.randn(n_out, k_in, device=dev) * 0.02)
            lin[m][name] = (wq_, ws_, (torch.randn(n_out, device=dev) * 0.01).bfloat16())
    acts = {m: {k: torch.randn(m, k, device=dev).bfloat16() for k in (3072, 12288)} for m in (4096, 512)}
    vec = torch.randn(1, 3072, device=dev).bfloat16()
    bufs = {(m, n): torch.empty(m, n, dtype=torch.bfloat16, device=dev) for m in (4096, 512) for n in (9216, 3072, 12288)}

    def block(_i):
        # image stream, text stream: the modulation vectors of each, both small-batch layers in one launch
        L.linear_w8a16_small_m_grouped([(vec,) + lin[m]["adaln"] for m in (4096, 512)])
        # each projection for both streams: their activations are quantised by one launch (they share the width,
        # not the weights), and their GEMMs go out together where the text stream's tiles fit into the CUs that the
        # image stream's last round leaves idle (the two projections into 3072 columns), else one launch per stream
        for name, k in (("qkv", 3072), ("proj", 3072), ("up", 3072), ("down", 12288)):
            quantised = L.quant_rowwise_grouped([acts[4096][k], acts[512][k]])
            n_out = lin[4096][name][0].shape[0]
            L.linear_w8a8_grouped([(q_, s_) + lin[m][name] for m, (q_, s_) in zip((4096, 512), quantised)], torch.bfloat16, L.EPI_TORCH,
                                  outs=[bufs[(4096, n_out)], bufs[(512, n_out)]])

    def block_quant_grouped(_i):   # grouped quantiser launches, one GEMM launch per stream
        for m in (4096, 512):
            L.linear_w8a16_small_m(vec, *lin[m]["adaln"])
        for name, k in (("qkv", 3072), ("proj", 3072), ("up", 3072), ("down", 12288)):
            quantised = L.quant_rowwise_grouped([acts[4096][k], acts[512][k]])
            for m, (q_, s_) in zip((4096, 512), quantised):
                wq_, ws_, b_ = lin[m][name]
                L.linear_w8a8(q_, s_, wq_, ws_, b_, torch.bfloat16, L.EPI_TORCH, bufs[(m, wq_.shape[0])])

    def block_separate(_i):   # the same block with one quantiser launch per layer, as the reference's operator is called
        for m in (4096, 512):
            L.linear_w8a16_small_m(vec, *lin[m]["adaln"])
            for name, k in (("qkv", 3072), ("proj", 3072), ("up", 3072), ("down", 12288)):
                wq_, ws_, b_ = lin[m][name]
                q_, s_ = L.quant_rowwise(acts[m][k])
                L.linear_w8a8(q_, s_, wq_, ws_, b_, torch.bfloat16, L.EPI_TORCH, bufs[(m, wq_.shape[0])])

    # the adaLN projection alone (M = 1, W8A16): a stream over the int8 weight, two weight sets in turn
    ada = [lin[m]["adaln"] for m in (4096, 512)]
    t = time_kernel(lambda i: L.linear_w8a16_small_m(vec, *ada[i]), max(10, iters // 4), sets=2, burst=8)
    abytes = ada[0][0].numel()
    out["adaln_w8a16_m1_18432x3072"] = {"median_us": round(t["median_us"], 2), "gbs": round(abytes / t["median_us"] / 1e3, 1),
                                        "frac_of_hbm_peak": round(abytes / t["median_us"] / 1e3 / PEAK_HBM_GBS, 4), "bytes": abytes,
                                        "note": "two 56.6 MB weights in turn: partly served by the 256 MB memory-side cache"}
    # (through the C entry point with the argument table built once: the Python wrapper's checks take longer than the launch)
    pair = (L._SmallMGroup * 2)()
    pair_out = [torch.empty(1, a_[0].shape[0], dtype=torch.bfloat16, device=dev) for a_ in ada]
    for g_, (wq_, ws_, b_), o_ in zip(pair, ada, pair_out):
        g_.a, g_.M, g_.K, g_.ldx, g_.w, g_.w_scale, g_.w_scale_host = vec.data_ptr(), 1, wq_.shape[1], wq_.shape[1], wq_.data_ptr(), ws_.data_ptr(), 0.0
        g_.bias, g_.out, g_.N = b_.data_ptr(), o_.data_ptr(), wq_.shape[0]

    def pair_call(_i):
        rc = lib.i8f_linear_w8a16_small_m_grouped(pair, 2, L.BF16, L.SCALE_ROW, L.BF16, stream)
        assert rc == 0, rc

    tg = time_kernel(pair_call, max(10, iters // 4))
    out["adaln_w8a16_m1_pair_in_one_launch"] = {"median_us": round(tg["median_us"], 2), "gbs": round(2 * abytes / tg["median_us"] / 1e3, 1),
                                                "frac_of_hbm_peak": round(2 * abytes / tg["median_us"] / 1e3 / PEAK_HBM_GBS, 4), "bytes": 2 * abytes,
                                                "note": "the modulation projections of both streams of a block (113 MB of weights) as one grid"}

    t_sep = time_kernel(block_separate, max(10, iters // 4))
    t_qg = time_kernel(block_quant_grouped, max(10, iters // 4))
    t = time_kernel(block, max(10, iters // 4))
    # the same block captured in a HIP graph (what torch.compile's reduce-overhead mode replays): no host between launches
    graph_ms = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            block(0)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            block(0)
        graph_ms = round(time_kernel(lambda i: graph.replay(), max(10, iters // 4))["median_us"] / 1e3, 4)
        del graph
    except Exception as e:   # the figure is an extra: a capture problem must not cost the benchmark line
        graph_ms = f"not measured: {type(e).__name__}: {e}"[:200]
    ops = sum(2 * m * n * k for m in (4096, 512) for (n, k) in [c3["linears"][x] for x in ("qkv", "proj", "up", "down")])
    out["dit_block_linears"] = {"ms": round(t["median_us"] / 1e3, 4), "gemm_gop": round(ops / 1e9, 1),
                                "tops": round(ops / t["median_us"] / 1e6, 1),
                                "ms_one_launch_per_layer_and_kernel": round(t_sep["median_us"] / 1e3, 4),
                                "ms_grouped_quantiser_only": round(t_qg["median_us"] / 1e3, 4),
                                "ms_replayed_from_a_hip_graph": graph_ms,
                                "note": "8 W8A8 linears and 2 adaLN W8A16 linears at M=1, separate weights for the image (4096 tokens) "
                                        "and the text stream (512 tokens), 340 MB in all; per projection one quantiser launch for both "
                                        "streams and, for the two projections into 3072 columns, one GEMM launch for both (192 + 24 "
                                        "tiles on 256 CUs); attention not included"}
    return out


# --------------------------------------------------------------------------- the north-star launch alone
def target_only(L, dev, mode, steps, warmup):
    """Nothing but launches of the north-star GEMM (M=4608, N=K=3072, W8A8 rowwise, bf16 out), for profilers:
    `warm` repeats one operand set (resident in the memory-side cache), `cold` walks 12 sets (623 MB).  Every GEMM
    launch of the process is one of these, so a counter file needs no filtering beyond the kernel name."""
    M, N, K = 4608, 3072, 3072
    g = torch.Generator().manual_seed(99)
    nset = 12 if mode == "cold" else 1
    q, s = L.quant_rowwise(_acts(g, M, K, 0.01, 20.0).to(dev))
    wq, ws = L.quant_rowwise((torch.randn(N, K, generator=g) * 0.02).to(dev))
    qs = [q] + [q.clone() for _ in range(nset - 1)]
    wqs = [wq] + [wq.clone() for _ in range(nset - 1)]
    ys = [torch.empty(M, N, dtype=torch.bfloat16, device=dev) for _ in range(nset)]
    t = time_kernel(lambda i: L.linear_w8a8(qs[i], s, wqs[i], ws, None, torch.bfloat16, L.EPI_TORCH, ys[i]),
                    iters=max(1, steps // nset), warmup=warmup, sets=nset, burst=nset)
    ops = 2 * M * N * K
    return {"kernel": "gemm_i8_kernel", "shape": "4608x3072x3072", "operands": mode, "tile": "%dx%d" % L.gemm_tile(M, N, K)[:2],
            "median_us": round(t["median_us"], 2), "min_us": round(t["min_us"], 2),
            "frac_of_int8_peak": round(ops / t["median_us"] / 1e6 / PEAK_INT8_TOPS, 4)}


def quant_only(L, dev, mode, steps, warmup):
    """Nothing but launches of the per-row quantiser at the north-star shape (4608 x 3072 bf16), with (`rot`) or without
    (`plain`) the 128-block rotation, over 8 buffer sets (> 256 MB), for profilers."""
    M, K, sets = 4608, 3072, 8
    g = torch.Generator().manual_seed(99)
    xs = [_acts(g, M, K, 0.01, 20.0).to(dev) for _ in range(sets)]
    qs = [torch.empty(M, K, dtype=torch.int8, device=dev) for _ in range(sets)]
    ss = [torch.empty(M, 1, dtype=torch.float32, device=dev) for _ in range(sets)]
    lib, ptr, stream = L.lib(), L._ptr, L._stream(xs[0])
    qargs = [(ptr(xs[i]), L.BF16, M, K, K, 128 if mode == "rot" else 0, ptr(qs[i]), ptr(ss[i]), stream) for i in range(sets)]

    def call(i):
        rc = lib.i8f_quant_rowwise(*qargs[i])
        assert rc == 0, rc
    t = time_kernel(call, iters=max(1, steps // sets), warmup=warmup, sets=sets, burst=sets)
    qbytes = M * K * 3 + 4 * M
    return {"kernel": "quant16_kernel", "shape": "4608x3072 bf16", "rotation": mode == "rot", "median_us": round(t["median_us"], 2),
            "min_us": round(t["min_us"], 2), "frac_of_hbm_peak": round(qbytes / t["median_us"] / 1e3 / PEAK_HBM_GBS, 4)}


# --------------------------------------------------------------------------- CPU baseline
def cpu_baseline(reps=3):
    """The reference's torch CPU path on config 1.  A 512-row probe sizes the sample: the whole
    workload (4608 rows) if that takes under about 10 s per run on this host, else the probe itself."""
    from oracle import torch_path as T

    def run(c, wq_up, ws_up, wq_dn, ws_dn):
        t0 = time.perf_counter()
        T.linear_w8a8(c["x"], wq_up, ws_up, c["b_up"], torch.bfloat16)
        T.linear_w8a8(c["h"], wq_dn, ws_dn, c["b_dn"], torch.bfloat16)
        return time.perf_counter() - t0

    full = make_config(1)
    wq_up, ws_up = T.quant_rowwise(full["w_up"])
    wq_dn, ws_dn = T.quant_rowwise(full["w_dn"])
    probe = {"x": full["x"][:512], "h": full["h"][:512], "b_up": full["b_up"], "b_dn": full["b_dn"]}
    run(probe, wq_up, ws_up, wq_dn, ws_dn)
    t_probe = run(probe, wq_up, ws_up, wq_dn, ws_dn)
    rows, c = (4608, full) if t_probe * 9 < 10.0 else (512, probe)
    t = statistics.median(run(c, wq_up, ws_up, wq_dn, ws_dn) for _ in range(reps))
    ops = 2 * 2 * rows * 12288 * 3072
    what = "all 4608 token rows" if rows == 4608 else "first 512 of 4608 token rows"
    return {"value": round(ops / t / 1e12, 4), "unit": "TOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{what} of config 1 (quantise + int8 matmul + dequant for both projections, full K and N), "
                      f"torch CPU restatement of the reference's slow path, median of {reps} runs, {t:.3f} s per run"}


# --------------------------------------------------------------------------- main
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--clock-ramp-s", type=float, default=0.2,
                    help="seconds of untimed steps before the warm-up, so that the GPU is at its sustained clocks")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--quick", action="store_true", help="fewer iterations in the extra measurements")
    ap.add_argument("--target-only", choices=("warm", "cold"),
                    help="profiling aid: launch nothing but the north-star GEMM (4608x3072x3072) on warm or cold operands, "
                         "print its timing and exit")
    ap.add_argument("--quant-only", choices=("rot", "plain"),
                    help="profiling aid: launch nothing but the per-row quantiser at 4608x3072 bf16, with or without rotation")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="what the traffic measurement runs under rocprofv3 --pmc: a few device copies and GEMM launches, no output")
    ap.add_argument("--no-live-traffic", action="store_true",
                    help="take the HBM-side bytes of the GEMM launches from profiles/gemm_hbm_traffic.txt instead of measuring them "
                         "in two child runs under rocprofv3 --pmc")
    ap.add_argument("--zero-operands", action="store_true",
                    help="diagnostic: all-zero activations and weights (same instructions, no switching in the multipliers), "
                         "to show what the power limit costs; the line says data = zeros and is not a benchmark result")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: the INT8 linear path has no multi-GPU part (run with --gpus 1)")

    # The counters need child processes: they run first, while this process has not touched the GPU yet.
    global LIVE_TRAFFIC
    traffic_source, live_note = "profiles/gemm_hbm_traffic.txt", None
    if not (a.traffic_probe or a.target_only or a.quant_only or a.no_live_traffic):
        LIVE_TRAFFIC, calibration, live_note = live_traffic()
        if LIVE_TRAFFIC is not None:
            traffic_source = (f"this run: two child runs under rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), calibrated on a device copy "
                              f"of {TRAFFIC_COPY_BYTES} bytes (fetch x {calibration['fetch_factor']}, write x {calibration['write_factor']})")

    import __graft_entry__ as ge

    pkg = ge.load_package()
    L = pkg._lib
    L.lib()   # fails loudly if the HIP library is not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if a.traffic_probe:
        traffic_probe(L, dev)
        return
    if a.target_only:
        print(json.dumps(target_only(L, dev, a.target_only, a.steps, a.warmup)))
        return
    if a.quant_only:
        print(json.dumps(quant_only(L, dev, a.quant_only, a.steps, a.warmup)))
        return
    step = MlpStep(L, dev)
    if a.zero_operands:
        for t in (step.x, step.h, step.wq_up, step.wq_dn):
            t.zero_()
    # torch creates the HIP event behind an Event at its first record(): do that here, not inside
    # the timed region
    evs = [_events(4) for _ in range(a.steps)]
    for e4 in evs:
        for e in e4:
            e.record()
    torch.cuda.synchronize()
    # Clock ramp: after idling, the GPU needs about 30 ms of load to reach its sustained clocks (the
    # first steps run up to twice slower).  Untimed steps bring it there before the W warm-up steps.
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < a.clock_ramp_s:
        for _ in range(10):
            step.run()
        torch.cuda.synchronize()
    for _ in range(a.warmup):
        step.run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(a.steps):
        step.run(evs[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    gemm_us = [e[0].elapsed_time(e[1]) * 1e3 for e in evs] + [e[2].elapsed_time(e[3]) * 1e3 for e in evs]
    avg_gemm_us = statistics.fmean(gemm_us)
    achieved = step.gemm_ops / avg_gemm_us / 1e6
    ms_per_step = wall / a.steps * 1e3
    value = 2 * step.gemm_ops / (ms_per_step * 1e-3) / 1e12

    tr = [gemm_traffic(L, 4608, 12288, 3072), gemm_traffic(L, 4608, 3072, 12288)]
    traffic = None if any(t[0] is None for t in tr) else (tr[0][0] + tr[1][0]) // 2
    traffic_note = "; ".join(t[1] for t in tr if t[1]) or None
    alg_bytes = (gemm_algorithmic_bytes(4608, 12288, 3072) + gemm_algorithmic_bytes(4608, 3072, 12288)) // 2

    line = {
        "metric": "INT8 GEMM TOPS (% of int8 MFMA peak) + ms per Flux-style DiT block, 1 GPU",
        "value": round(value, 1),
        "unit": "TOP/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "zeros (power diagnostic, not a result)" if a.zero_operands else "synthetic",
        "clock_ramp_s": a.clock_ramp_s,
        "config": {"workload": "BASELINE config 1: Flux MLP W8A8 rowwise, M=4608, 3072->12288->3072, bf16 in/out, bias; "
                               "quantise + GEMM for both projections, inputs resident in HBM"},
        "pct_of_int8_peak": round(100 * value / PEAK_INT8_TOPS, 2),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": round(achieved / PEAK_INT8_TOPS, 4), "traffic": traffic,
                     "traffic_unit": "bytes per launch beyond L2, mean of the two GEMM launches of the step",
                     "traffic_source": traffic_source,
                     "algorithmic_bytes": alg_bytes,
                     "traffic_over_algorithmic": None if traffic is None else round(traffic / alg_bytes, 2),
                     "kernel": "gemm_i8_kernel (int8 MFMA GEMM + dequant epilogue)",
                     "tiles": {"4608x12288x3072": "%dx%d" % L.gemm_tile(4608, 12288, 3072)[:2],
                               "4608x3072x12288": "%dx%d" % L.gemm_tile(4608, 3072, 12288)[:2]},
                     "ops_per_launch": step.gemm_ops, "avg_launch_us": round(avg_gemm_us, 2),
                     "launches_timed": len(gemm_us)},
    }
    if traffic_note:
        line["roofline"]["traffic_note"] = traffic_note
    if live_note:
        line["roofline"]["live_traffic_note"] = "not measured in this run (" + live_note + "): figures of the same procedure from the profile"
    extra = extras(L, dev, quick=a.quick) if not a.no_extras else None   # before the CPU leg: the GPU is still warm
    if not a.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline()
    if extra is not None:
        # the north-star shape as a roofline block of its own (the `roofline` block above is the step's GEMMs)
        tg = extra["target_gemm_4608x3072x3072"]
        t_traffic, t_note = gemm_traffic(L, 4608, 3072, 3072)
        t_alg = gemm_algorithmic_bytes(4608, 3072, 3072, bias=False)
        # headline = operands that are NOT in the memory-side cache (12 operand sets in turn), which is what a layer
        # inside a model sees; the loop over one operand set is reported beside it
        line["roofline_target"] = {"bound": "mfma", "shape": "M=4608, N=K=3072, W8A8 rowwise, bf16 out", "tile": tg["tile"],
                                   "ops_per_launch": 2 * 4608 * 3072 * 3072, "avg_launch_us": tg["cold_operands_median_us"],
                                   "achieved": tg["cold_operands_tops"], "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                                   "frac": tg["cold_operands_frac_of_int8_peak"],
                                   "operands": "12 operand sets in turn (623 MB: none of them in the 256 MB memory-side cache)",
                                   "cold_operands_avg_launch_us": tg["cold_operands_median_us"],
                                   "cold_operands_frac": tg["cold_operands_frac_of_int8_peak"],
                                   "warm_operands_avg_launch_us": tg["median_us"], "warm_operands_frac": tg["frac_of_int8_peak"],
                                   "vendor_int_mm_warm_us": tg.get("vendor_int_mm_median_us"),
                                   "traffic": t_traffic, "traffic_source": traffic_source, "algorithmic_bytes": t_alg,
                                   "traffic_over_algorithmic": None if t_traffic is None else round(t_traffic / t_alg, 2)}
        if t_note:
            line["roofline_target"]["traffic_note"] = t_note
        rq = extra["rotate_quant_4608x3072"]
        line["roofline_rotate_quant"] = {"bound": "hbm", "kernel": "quant16_kernel (rotate + absmax + int8, one pass)",
                                         "bytes_per_launch": rq["bytes"], "avg_launch_us": rq["median_us"],
                                         "achieved": rq["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": rq["frac_of_hbm_peak"]}
        line["extras"] = extra
        if "dit_block_linears" in extra:
            line["dit_block_ms"] = extra["dit_block_linears"]["ms"]
    print(json.dumps(line))


if __name__ == "__main__":
    main()
