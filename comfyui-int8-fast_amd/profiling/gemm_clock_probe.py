"""40 launches of the 4608 x 3072 x 12288 GEMM on all-zero operands, then 40 on realistic ones, for a
counter run that tells the shader clock during the kernel:

    cd /tmp && TMPDIR=/tmp rocprofv3 --pmc GRBM_GUI_ACTIVE SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES --kernel-trace \
        --output-format csv -d out -o f -- python3 <repo>/comfyui-int8-fast_amd/profiling/gemm_clock_probe.py

GRBM_GUI_ACTIVE (summed over the 8 XCDs) / 8 is the kernel's length in shader cycles; divided by the
duration in the kernel trace it is the average clock.  SQ_VALU_MFMA_BUSY_CYCLES / (216 CUs x 4 SIMDs)
over the same cycle count is the matrix-pipe utilisation in cycles, which does not depend on the clock.
"""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import __graft_entry__ as ge  # noqa: E402


def main():
    L = ge.load_package()._lib
    dev = torch.device("cuda:0")
    M, N, K = 4608, 3072, 12288
    xs, ws = torch.rand(M, 1, device=dev) * 0.01, torch.rand(N, device=dev) * 0.01
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    for data in ("zero", "real"):
        if data == "zero":
            a = torch.zeros(M, K, dtype=torch.int8, device=dev)
            w = torch.zeros(N, K, dtype=torch.int8, device=dev)
        else:
            a, _ = L.quant_rowwise(torch.randn(M, K, device=dev).abs().bfloat16())
            w, _ = L.quant_rowwise(torch.randn(N, K, device=dev))
        for _ in range(40):
            L.linear_w8a8(a, xs, w, ws, None, torch.bfloat16, 0, out)
        torch.cuda.synchronize()
    print("ok")


if __name__ == "__main__":
    main()
