"""Where one GEMM launch spends its time, per workgroup: prologue, main loop, epilogue.

    python comfyui-int8-fast_amd/build.py --probes
    python comfyui-int8-fast_amd/profiling/gemm_phase_trace.py 4608x3072x3072 [--probe trace|mfma_only|dma_only|no_store]
                                                               [--data real|rand|zero] [--tile 256x256]

The probe libraries are the product GEMM compiled with -DI8F_TRACE: thread 0 of every workgroup
writes 100 MHz wall-clock stamps (start, first K-tile landed, loop done, all waves done) into a
buffer whose address travels in the environment variable I8F_TRACE_PTR.  The ablation probes drop
one part of the main loop (results are then wrong; only the timing is of interest):
mfma_only = no global->LDS loads and no LDS fragment reads, dma_only = no MFMAs and no fragment
reads, no_store = the epilogue's global stores are compiled in but never taken.
--data chooses the int8 operand values: quantised Gaussian activations with outlier channels and
Gaussian weights (real), uniform full-range bytes (rand), or zeros; the matrix pipe's sustained
rate depends on them.
"""
import argparse
import ctypes
import os
import sys
import time

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def operands(M, N, K, data, dev):
    g = torch.Generator().manual_seed(5)
    if data == "zero":
        return torch.zeros(M, K, dtype=torch.int8, device=dev), torch.zeros(N, K, dtype=torch.int8, device=dev)
    if data == "rand":
        return (torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g).to(dev),
                torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g).to(dev))
    x = torch.randn(M, K, generator=g)
    x[:, torch.randperm(K, generator=g)[:max(1, K // 100)]] *= 20
    w = torch.randn(N, K, generator=g)
    q = lambda t: torch.round(t / (t.abs().amax(1, keepdim=True) / 127)).to(torch.int8).to(dev)
    return q(x), q(w)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("shape", help="MxNxK")
    ap.add_argument("--probe", default="trace")
    ap.add_argument("--data", default="real", choices=("real", "rand", "zero"))
    ap.add_argument("--tile", default=None, help="BMxBN the library picks for this shape (default: as the host code does)")
    a = ap.parse_args()
    M, N, K = (int(v) for v in a.shape.split("x"))
    path = os.path.join(HERE, f"libi8f_probe_{a.probe}.so")
    if not os.path.exists(path):
        sys.exit(f"{path} is missing: python comfyui-int8-fast_amd/build.py --probes")
    lib = ctypes.CDLL(path)
    vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
    lib.i8f_linear_w8a8.argtypes = [vp, vp, vp, vp, f32, i32, vp, i32, vp, i32, i64, i64, i64, i32, vp]
    if a.tile:
        BM, BN = (int(v) for v in a.tile.split("x"))
    else:   # the host-side choice of gemm_i8.hip
        cd = lambda p, q: (p + q - 1) // q
        big, mid = cd(M, 256) * cd(N, 256), cd(M, 128) * cd(N, 128)
        cost = lambda bm, bn, per_op: cd(cd(M, bm) * cd(N, bn), 256) * bm * bn * per_op
        if big >= 128:
            cands = [(cost(256, 256, 100), (256, 256)), (cd(mid, 512) * 2 * 128 * 128 * 141, (128, 128)),
                     (cost(288, 256, 102), (288, 256)), (cost(256, 288, 102), (256, 288)), (cost(256, 192, 108), (256, 192))]
            BM, BN = min(cands, key=lambda c: c[0])[1]      # ties go to the first, as in the library
        elif mid >= 256:
            w96 = cd(M, 256) * cd(N, 96)
            BM, BN = (256, 96) if cd(w96, 256) * 352 < cd(mid, 512) * 512 else (128, 128)
        else:   # few tiles: bytes the busiest CU fetches per K-step; ties go to the first, as in the library
            fetch = lambda bm, bn: cd(cd(M, bm) * cd(N, bn), 256) * (bm + bn)
            BM, BN = min([(128, 128), (128, 96), (128, 64), (64, 64)], key=lambda t: fetch(*t))
    dev = torch.device("cuda:0")
    x, w = operands(M, N, K, a.data, dev)
    xs, ws = torch.rand(M, device=dev) * 0.01, torch.rand(N, device=dev) * 0.01
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    nblk = -(-M // BM) * -(-N // BN)
    tr = torch.zeros(nblk * 8, dtype=torch.int64, device=dev)
    os.environ["I8F_TRACE_PTR"] = str(tr.data_ptr())
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # the stamps read back are those of the LAST launch of a back-to-back series that is long enough
    # for the GPU to reach its sustained clocks (about 30 ms after idle); every launch overwrites them
    def launch():
        rc = lib.i8f_linear_w8a8(x.data_ptr(), xs.data_ptr(), w.data_ptr(), ws.data_ptr(), 0.0, 1, None, 0,
                                 out.data_ptr(), 0, M, N, K, 0, None)
        assert rc == 0, rc
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.1:
        for _ in range(20):
            launch()
        torch.cuda.synchronize()
    for _ in range(50):
        launch()
    e0.record()
    launch()
    e1.record()
    torch.cuda.synchronize()
    t = tr.cpu().numpy().reshape(nblk, 8).astype(np.float64) * 10e-3     # 100 MHz ticks -> microseconds
    if not t[:, 3].all():
        sys.exit("some workgroups left no stamp: --tile does not match what the library launched")
    t0, KT = t[:, 0].min(), -(-K // 128)
    pro, loop, epi = t[:, 1] - t[:, 0], t[:, 2] - t[:, 1], t[:, 3] - t[:, 2]
    med, pc = np.median, np.percentile
    print(f"{M}x{N}x{K} tile {BM}x{BN} probe={a.probe} data={a.data}: {nblk} workgroups, "
          f"events {e0.elapsed_time(e1) * 1e3:.1f} us, first start to last end {t[:, 3].max() - t0:.1f} us")
    print(f"  prologue   median {med(pro):6.2f} us   p90 {pc(pro, 90):6.2f}")
    print(f"  main loop  median {med(loop):6.2f} us   p10 {pc(loop, 10):6.2f}  p90 {pc(loop, 90):6.2f}   "
          f"= {med(loop) / KT:.3f} us per 128-wide K-tile")
    print(f"  epilogue   median {med(epi):6.2f} us   p90 {pc(epi, 90):6.2f}   "
          f"(operand preload {med(t[:, 4] - t[:, 2]):.2f}, convert + LDS write {med(t[:, 5] - t[:, 4]):.2f}, "
          f"read back + stores {med(t[:, 6] - t[:, 5]):.2f})")
    print(f"  workgroup  median {med(t[:, 3] - t[:, 0]):6.2f} us   last start {t[:, 0].max() - t0:.1f} us after the first")


if __name__ == "__main__":
    main()
