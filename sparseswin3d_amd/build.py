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
           "window_attention.hip", "window_attention_x16.hip", "column_sum.hip", "voxel_grid.hip", "tall_linear.hip"]
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


PYBIND_SRC = os.path.join(CSRC, "custom_ops_pybind.cpp")
PYBIND_NAME = "custom_ops_pybind"


def build_pybind(verbose: bool = False) -> str:
    """Compile the pybind11 module with the reference's ten operator names over the C ABI
    (``sparseswin3d_amd/custom_ops_pybind*.so``).  hipcc compiles the one host source directly against
    PyTorch's HIP-native headers; nothing is translated."""
    import sysconfig

    import pybind11
    import torch
    from torch.utils import cpp_extension
    hipcc = _hipcc()
    out = os.path.join(HERE, PYBIND_NAME + sysconfig.get_config_var("EXT_SUFFIX"))
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    includes = [pybind11.get_include(), sysconfig.get_paths()["include"], *cpp_extension.include_paths("cuda")]
    cmd = [hipcc, "-O2", "-std=c++17", "-fPIC", "-shared", "-x", "c++", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-DTORCH_EXTENSION_NAME={PYBIND_NAME}", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *[f"-I{p}" for p in includes], PYBIND_SRC, "-o", out,
           f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
           f"-L{HERE}", "-lsswin3d", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}",
           "-Wno-unused-command-line-argument"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {PYBIND_SRC}:\n{r.stderr[-6000:]}")
    if verbose and r.stderr.strip():
        print(r.stderr, file=sys.stderr)
    return out


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
    if "--no-pybind" not in sys.argv:
        print(build_pybind(verbose="-v" in sys.argv))
