"""Build libi8f_gfx950.so from csrc/*.hip with hipcc, in-tree.

    python comfyui-int8-fast_amd/build.py [--force] [--keep-temps]

hipcc cross-compiles for gfx950 without a GPU.  The library is written next to
this file so that it travels with the source tree; nothing is installed.
"""
from __future__ import annotations

import argparse
import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libi8f_gfx950.so")

# -ffp-contract=off and correctly rounded division are part of the numerical
# contract (bit-exact quantiser, epilogue and merge); packed FP32 instructions
# are switched off for the device pass (the host pass does not know the feature
# and says so, harmlessly).
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-DI8F_BUILD_CONTRACT=1",   # i8f_common.hpp refuses to compile without it: a build that bypasses these flags fails
    "-Wall",
    "-Wno-unused-function",
    "-Wno-inline-asm",   # the global->LDS loads name m0 in their clobber list, which clang reports as "reserved"
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; install ROCm or set HIPCC")


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _stale(target: str, deps: list[str]) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = False, keep_temps: bool = False, verbose: bool = True) -> str:
    cc = hipcc()
    os.makedirs(OBJ, exist_ok=True)
    headers = glob.glob(os.path.join(CSRC, "*.hpp")) + glob.glob(os.path.join(HERE, "..", "include", "*.h"))
    jobs = []
    objs = []
    for src in sources():
        obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        if force or _stale(obj, [src] + headers):
            cmd = [cc, *FLAGS, "-c", src, "-o", obj]
            if keep_temps:
                cmd += ["-save-temps=obj"]
            jobs.append(cmd)

    def run(cmd):
        p = subprocess.run(cmd, capture_output=True, text=True)
        noise = "is not a recognized feature for this target"
        err = "\n".join(l for l in p.stderr.splitlines() if noise not in l)
        return p.returncode, cmd, err

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for rc, cmd, err in ex.map(run, jobs):
            if verbose and err.strip():
                print(err, file=sys.stderr)
            if rc != 0:
                raise RuntimeError("hipcc failed: " + " ".join(cmd) + "\n" + err)
    if force or jobs or _stale(LIB, objs):
        cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
        p = subprocess.run(cmd, capture_output=True, text=True)
        if p.returncode != 0:
            raise RuntimeError("link failed: " + p.stderr)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--keep-temps", action="store_true")
    a = ap.parse_args()
    print(build(force=a.force, keep_temps=a.keep_temps))
