"""In-tree build of the two shared libraries of the fused W8A8 MoE operator for gfx950.

    python alpha-moe_amd/build.py            # both
    python alpha-moe_amd/build.py --hip-only

* alpha_moe/libalpha_moe_hip.so  - the HIP kernels behind the C ABI of include/alpha_moe_hip.h (hipcc, no torch)
* alpha_moe/alpha_moe_torch.so   - the PyTorch-ROCm binding (csrc/torch_interface.cpp), linked against the first

Stands in for the reference's setup.py (CUDAExtension, arch 9.0a), which would hipify the sources; here the
kernels are compiled by hipcc directly and the binding is an ordinary C++ file.
"""
import argparse
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "alpha_moe")
HIP_LIB = os.path.join(OUT, "libalpha_moe_hip.so")
TORCH_LIB = os.path.join(OUT, "alpha_moe_torch.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# packed-fp32 VALU forms are switched off for every kernel in this library
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
# Per-source extras.  The tile kernel scales every matrix-instruction result into vector-register accumulators, so
# the results must land in vector registers, not in accumulation registers that only a copy can read.
HIP_SOURCES = {
    "moe_api.hip": [],
    "moe_direct.hip": [],
    "moe_stream.hip": [],
    "moe_tile.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "moe_wide.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "moe_prep.hip": [],
}


def run(cmd):
    print("+", " ".join(cmd), flush=True)
    finish(cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))


def finish(cmd, proc):
    out, _ = proc.communicate()
    res = subprocess.CompletedProcess(cmd, proc.returncode, out)
    lines = [l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l]
    if lines:
        print("\n".join(lines), flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"command failed with exit code {res.returncode}: {' '.join(cmd)}")


def build_hip():
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    jobs, objs = [], []
    for src, extra in HIP_SOURCES.items():   # one compiler process per source, all at once
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [HIPCC, *HIP_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        jobs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for cmd, proc in jobs:
        finish(cmd, proc)
    run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB, *objs])
    return HIP_LIB


def build_torch():
    import torch
    from torch.utils import cpp_extension
    tdir = os.path.dirname(torch.__file__)
    inc = [f"-I{p}" for p in cpp_extension.include_paths()] + [f"-I{ROCM}/include"]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={abi}", *inc, os.path.join(CSRC, "torch_interface.cpp"), "-o", TORCH_LIB,
           f"-L{OUT}", "-lalpha_moe_hip", f"-L{tdir}/lib", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
           "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed"]
    run(cmd)
    return TORCH_LIB


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--hip-only", action="store_true")
    args = ap.parse_args(argv)
    build_hip()
    if not args.hip_only:
        build_torch()


if __name__ == "__main__":
    sys.exit(main())
