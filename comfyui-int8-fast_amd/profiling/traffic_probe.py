"""One launch of each hot-path kernel next to a device copy of known size, for HBM-traffic counters.

    cd /tmp && TMPDIR=/tmp rocprofv3 --pmc FETCH_SIZE --output-format csv -d out_fetch -o t -- python3 <repo>/comfyui-int8-fast_amd/profiling/traffic_probe.py
    cd /tmp && TMPDIR=/tmp rocprofv3 --pmc WRITE_SIZE --output-format csv -d out_write -o t -- python3 <repo>/comfyui-int8-fast_amd/profiling/traffic_probe.py

The copy (256 MiB read, 256 MiB written) calibrates the counters: divide its known byte counts by
what FETCH_SIZE / WRITE_SIZE report for it and scale the other kernels' readings by that factor.
"""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import __graft_entry__ as ge  # noqa: E402
import bench  # noqa: E402


def main():
    pkg = ge.load_package()
    L = pkg._lib
    dev = torch.device("cuda:0")
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    step = bench.MlpStep(L, dev)                      # config 1: both quantisers and both GEMMs
    g = torch.Generator().manual_seed(1)
    x = bench._acts(g, 4608, 3072, 0.01, 20.0).to(dev)
    wq, ws = L.quant_rowwise((torch.randn(3072, 3072, generator=g) * 0.02).to(dev))
    c = bench.make_config(4)
    w4q, w4s = L.quant_rowwise(c["w"].to(dev))
    up, down, noise = c["up"].to(dev), c["down"].to(dev), c["noise"].to(dev)
    out4 = torch.empty_like(w4q)
    torch.cuda.synchronize()
    for _ in range(3):
        dst.copy_(src)
        step.run()
        q, s = L.quant_rowwise(x, rotate=True)        # fused rotate + quantise, 4608 x 3072
        L.linear_w8a8(q, s, wq, ws, None, torch.bfloat16, 0)   # the north-star shape 4608 x 3072 x 3072
        L.lora_merge_sr(w4q, w4s, noise, up=up, down=down, lora_scale=1.0, out=out4)
        torch.cuda.synchronize()
    print("ok")


if __name__ == "__main__":
    main()
