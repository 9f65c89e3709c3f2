"""Build libuvmi.so (the C-ABI HIP library) for gfx950 in-tree.

    python -m ultraviolet_amd.csrc.build            # rebuild what is out of date
    python -m ultraviolet_amd.csrc.build --force    # recompile every source

hipcc cross-compiles without a GPU.  The packed-fp32 target feature is switched off for all device code.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["common.hip", "kv_quant.hip", "decode_attn.hip", "fused_sample.hip", "sched.hip", "model_ops.hip",
           "prefill_attn.hip", "prefill_attn_bwd.hip", "gemm.hip", "gemm_tile.hip", "gemm_big.hip"]
LIB = os.path.join(HERE, "libuvmi.so")
ARCH = "gfx950"
FLAGS = ["-O3", "-fPIC", "-std=c++17", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-result", "-Wno-unknown-warning-option",
         # keep MFMA accumulators in VGPRs: the attention kernels rescale them with VALU ops, and the AGPR form costs
         # an accvgpr read/write pair per register per step
         "-mllvm", "-amdgpu-mfma-vgpr-form=1",
         # the first kernel arguments arrive in SGPRs with the wave instead of through a load at kernel start
         "-mllvm", "-amdgpu-kernarg-preload-count=16"]


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    return "hipcc"


def _stale(obj: str, src: str) -> bool:
    if not os.path.exists(obj):
        return True
    deps = [src, os.path.join(HERE, "common.h"), os.path.join(HERE, "sched_commit.h"), os.path.join(HERE, "gemm_util.h"), os.path.join(HERE, "attn_mfma_util.h"), os.path.join(HERE, "..", "..", "include", "uvmi.h"), __file__]
    return any(os.path.getmtime(d) > os.path.getmtime(obj) for d in deps)


def build(force: bool = False, verbose: bool = True) -> str:
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    hipcc = _hipcc()
    jobs = []
    for s in srcs:
        src, obj = os.path.join(HERE, s), os.path.join(objdir, s.replace(".hip", ".o"))
        if force or _stale(obj, src):
            jobs.append([hipcc, *FLAGS, "-c", src, "-o", obj])

    def run(cmd):
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"{' '.join(cmd)}\n{r.stdout}\n{r.stderr}")
        return cmd[-1]

    if jobs:
        with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
            for o in ex.map(run, jobs):
                if verbose:
                    print("compiled", os.path.relpath(o, HERE), flush=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in srcs]
    if jobs or not os.path.exists(LIB):
        run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB, *objs])
        if verbose:
            print("linked", os.path.relpath(LIB, HERE), flush=True)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
