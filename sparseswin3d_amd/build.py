"""Builds ``libsswin3d.so`` (the C-ABI HIP library) for gfx950 with hipcc.

Usage: ``python -m sparseswin3d_amd.build``.  hipcc cross-compiles without a GPU.  The
``.hip`` sources are compiled as they are (no translation pass) and linked into one shared
object placed next to this file, which is where ``sparseswin3d_amd._lib`` looks for it.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libsswin3d.so")
SOURCES = ["index_ops.hip", "plan.hip", "block_matmul.hip", "softmax.hip", "fused_attention.hip",
           "window_attention.hip", "column_sum.hip", "voxel_grid.hip", "tall_linear.hip"]
ARCH = "gfx950"
# packed FP32 instructions are switched off for all device code on purpose
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-munsafe-fp-atomics",          # LDS float adds as ds_add_f32 instead of compare-and-swap loops
         "-mllvm", "-amdgpu-mfma-vgpr-form",   # MFMA accumulators in VGPRs: no copies to and from AGPRs
         "-Wno-unused-command-line-argument"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False) -> str:
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr[-4000:]}")
        if verbose and r.stderr.strip():
            print(r.stderr, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=5) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", OUT]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    return OUT


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
