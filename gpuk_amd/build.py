"""In-tree build of the shared libraries (run as `python -m gpuk_amd.build`).

  gpuk_amd/lib/libgpuk_amd.so : HIP kernels for gfx950 behind the C ABI of include/gpuk_amd.h (no torch)
  gpuk_amd/lib/libgpuk.so     : torch library `gpuk` (csrc/register.cpp + csrc/ops/*.cpp), links the former
  gpuk_amd/lib/libgpuk_amd_stamps.so : the first, compiled with -DGPUK_STAMPS: a profiling build whose kernels
                                record the shader clock at named phases (`python -m gpuk_amd.stamps`); `--stamps`
                                builds only this one

hipcc cross-compiles gfx950 code objects without a GPU, so this runs on a CPU-only builder; the
built files travel with the tree.  The reference builds with CMake for either CUDA or HIP
(CMakeLists.txt, cmake.py); this build is HIP-only.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(HERE, "build")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# -packed-fp32-ops off: keep the compiler from forming v_pk_*_f32 from scalar float code.
# -ffp-contract=off: the kernels reproduce a fixed sequence of roundings; HIP's default contraction fuses
# a half-precision product into a following add (v_fma_mix) and skips the product's rounding.  Fused
# multiply-adds are written explicitly where they are wanted.
DEVICE_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-ffp-contract=off",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall"]

KERNEL_SOURCES = ["kernels/add_rmsnorm_quant.hip", "kernels/rope_rms.hip", "kernels/calibration.hip", "kernels/capi.cpp"]
# Kernel-argument preload: the first 14 dwords of a kernel's arguments are placed in scalar registers when a wave is
# launched, so its first loads do not wait for a fetch of the argument block (the norm-quant kernel orders its
# and the rope kernels order their arguments for this).
EXTRA_FLAGS = {"kernels/add_rmsnorm_quant.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=14"],
               "kernels/rope_rms.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=14"]}
OP_SOURCES = ["register.cpp", "ops/allreduce_rms.cpp", "ops/fused_rope.cpp"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    if out.strip() and os.environ.get("GPUK_BUILD_VERBOSE"):
        print(out)


def _compile(args):
    src, obj, flags = args
    os.makedirs(os.path.dirname(obj), exist_ok=True)
    _run([HIPCC] + flags + ["-c", os.path.join(CSRC, src), "-o", obj])
    return obj


def build_kernels(jobs: int = 4, stamps: bool = False) -> str:
    """libgpuk_amd.so, or with stamps=True libgpuk_amd_stamps.so: the same sources compiled with -DGPUK_STAMPS, in
    which the kernels record the shader clock at named phases (read by `python -m gpuk_amd.stamps`)."""
    os.makedirs(LIB, exist_ok=True)
    work = []
    for s in KERNEL_SOURCES:
        flags = list(DEVICE_FLAGS)
        if s.endswith(".cpp"):
            flags = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include"]
        else:
            flags += EXTRA_FLAGS.get(s, [])
            if stamps:
                flags.append("-DGPUK_STAMPS")
        work.append((s, os.path.join(OBJ, ("stamps_" if stamps else "") + s.replace("/", "_") + ".o"), flags))
    with ThreadPoolExecutor(jobs) as ex:
        objs = list(ex.map(_compile, work))
    out = os.path.join(LIB, "libgpuk_amd_stamps.so" if stamps else "libgpuk_amd.so")
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", out] + objs)
    return out


def build_torch_library(jobs: int = 4) -> str:
    import torch
    from torch.utils import cpp_extension

    os.makedirs(LIB, exist_ok=True)
    inc = []
    for p in cpp_extension.include_paths():
        inc += ["-isystem", p]
    flags = ["-O2", "-std=c++17", "-fPIC", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DHIPBLAS_V2",
             "-D_GLIBCXX_USE_CXX11_ABI=" + str(int(torch._C._GLIBCXX_USE_CXX11_ABI)),
             "-I/opt/rocm/include", "-Wno-deprecated-declarations"] + inc
    # host-only translation units: compile them as plain C++ (hipcc is the clang driver)
    work = [(s, os.path.join(OBJ, "torch_" + s.replace("/", "_") + ".o"), ["-x", "c++"] + flags) for s in OP_SOURCES]
    with ThreadPoolExecutor(jobs) as ex:
        objs = list(ex.map(_compile, work))
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = os.path.join(LIB, "libgpuk.so")
    _run([HIPCC, "-shared", "-fPIC", "-o", out] + objs +
         ["-L" + LIB, "-lgpuk_amd", "-L" + torch_lib, "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
          "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed"])
    return out


def build_all(verbose: bool = True) -> None:
    a = build_kernels()
    if verbose:
        print("built", a)
    b = build_torch_library()
    if verbose:
        print("built", b)
    c = build_kernels(stamps=True)
    if verbose:
        print("built", c)


if __name__ == "__main__":
    if "--stamps" in sys.argv[1:]:
        print("built", build_kernels(stamps=True))
    else:
        build_all()
    sys.exit(0)
