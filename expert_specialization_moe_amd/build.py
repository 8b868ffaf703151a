"""Build the native libraries in-tree with hipcc (gfx950 only).

    python expert_specialization_moe_amd/build.py            # everything
    python expert_specialization_moe_amd/build.py --no-torch # libesmoe.so only

(run it as a script: importing the package requires the libraries it builds)

Produces, next to this file:
  libesmoe.so   HIP kernels + the C ABI declared in include/esmoe.h
  _C.so         PyTorch operator registration (torch.ops.expert_specialization.*), links libesmoe.so
"""
import argparse
import os
import subprocess
import sys
import time

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
INCLUDE = os.path.join(ROOT, "include")
OBJ = os.path.join(PKG, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

HIP_SOURCES = ["grouped_gemm.hip", "mxfp8_quant.hip", "fp8_quant.hip", "routing.hip", "capi.hip"]
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-mcode-object-version=5",
    # packed fp32 VALU ops are kept out of the device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results go to VGPRs: the fp32 scale-and-accumulate of the FP8-blockwise path reads them with VALU ops
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument",
    f"-I{INCLUDE}", f"-I{CSRC}",
]


def run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_lib(verbose_resources=False):
    os.makedirs(OBJ, exist_ok=True)
    objs = []
    procs = []
    for src in HIP_SOURCES:
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        cmd = [HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose_resources:
            cmd.append("-Rpass-analysis=kernel-resource-usage")
        print("+", " ".join(cmd), flush=True)
        procs.append((subprocess.Popen(cmd), cmd))
        objs.append(obj)
    for p, cmd in procs:
        if p.wait() != 0:
            raise subprocess.CalledProcessError(p.returncode, cmd)
    out = os.path.join(PKG, "libesmoe.so")
    run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-Wno-unused-command-line-argument", "-o", out] + objs)
    return out


def build_torch_binding():
    import torch
    from torch.utils import cpp_extension as ce
    import sysconfig

    out = os.path.join(PKG, "_C.so")
    inc = [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}", f"-I{INCLUDE}",
                                                      "-I/opt/rocm/include"]
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-deprecated-declarations"] + inc + [
        os.path.join(CSRC, "torch_binding.cpp"), "-o", out,
        f"-L{PKG}", "-lesmoe", f"-L{libdir}", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
        "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{libdir}"]
    run(cmd)
    return out


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-torch", action="store_true")
    ap.add_argument("--resources", action="store_true", help="print per-kernel register/LDS usage")
    args = ap.parse_args(argv)
    t0 = time.time()
    build_lib(args.resources)
    if not args.no_torch:
        build_torch_binding()
    print(f"built in {time.time() - t0:.1f}s")


if __name__ == "__main__":
    main()
