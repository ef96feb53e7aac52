"""Build recipe of the native libraries (hipcc, gfx950 only).

  libfo_kernels.so    HIP kernels + host orchestration behind the C ABI of
                      include/flashoverlap.h (no torch dependency)
  libst_pybinding.so  TORCH_LIBRARY shim registering
                      torch.classes.flashoverlap_class.{OverlapImpl,BaselineImpl}
                      and torch.ops.flashoverlap_op.* on top of the C ABI; the
                      file name is the one the reference scripts load
                      (example/RMSNorm.py:5, README.md:69)

Both land in flashoverlap_amd/lib/; the shim is also copied to build/lib/ so that
`torch.ops.load_library("../build/lib/libst_pybinding.so")` keeps working from a
sub-directory of the repository root.

Run as `python -m flashoverlap_amd.build [--no-shim]`.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
KERNEL_LIB = os.path.join(LIBDIR, "libfo_kernels.so")
SHIM_LIB = os.path.join(LIBDIR, "libst_pybinding.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

KERNEL_SOURCES = ["fo_gemm.hip", "fo_aux.hip", "fo_algo.cpp", "fo_overlap.cpp"]
# fo_gemm256_inst.hip holds one instantiation of the 256x256 GEMM kernel per compilation
# (dtype fp16 / bf16 x plain / signal / scatter epilogue); each takes minutes, so they are separate jobs.
GEMM256_INSTANCES = [(d, m) for d in (0, 1) for m in (0, 1, 2)]

# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 from the float code here.
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # the K step of the 256x256 kernel is one fully unrolled body of 128 MFMAs built from nested constant loops
    "-mllvm", "-pragma-unroll-threshold=1000000",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + "\n")
        raise RuntimeError(f"build step failed: {cmd[0]} ... {cmd[-1]}")
    return proc.stdout


def build_kernels(extra_flags=()):
    os.makedirs(OBJDIR, exist_ok=True)

    def compile_one(job):
        src, defs, tag = job
        obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + tag + ".o")
        _run([HIPCC] + HIP_FLAGS + list(extra_flags) + defs + ["-c", os.path.join(CSRC, src), "-o", obj])
        return obj

    # the long jobs first
    jobs = [("fo_gemm256_inst.hip", [f"-DFO_INST_DTYPE={d}", f"-DFO_INST_MODE={m}"], f"_{d}_{m}")
            for d, m in GEMM256_INSTANCES]
    jobs += [(src, [], "") for src in KERNEL_SOURCES]
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 4)) as pool:
        objs = list(pool.map(compile_one, jobs))
    _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", KERNEL_LIB] + objs)
    return KERNEL_LIB


def build_shim():
    import torch
    from torch.utils import cpp_extension

    os.makedirs(OBJDIR, exist_ok=True)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    incs = []
    for p in cpp_extension.include_paths():
        incs += ["-isystem", p]
    abi = int(getattr(torch._C, "_GLIBCXX_USE_CXX11_ABI", True))
    obj = os.path.join(OBJDIR, "fo_torch_shim.o")
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-c", os.path.join(CSRC, "fo_torch_shim.cpp"),
          "-o", obj, "-I" + os.path.join(ROOT, "include"), "-isystem", "/opt/rocm/include",
          "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
          "-Wno-deprecated-declarations"] + incs)
    _run(["g++", "-shared", "-fPIC", "-o", SHIM_LIB, obj,
          "-L" + LIBDIR, "-lfo_kernels", "-Wl,-rpath,$ORIGIN",
          "-L" + torch_lib, "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip",
          "-Wl,-rpath," + torch_lib,
          "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"])
    dst_dir = os.path.join(ROOT, "build", "lib")
    os.makedirs(dst_dir, exist_ok=True)
    # Same directory layout as the reference build output; both libraries are
    # copied so that $ORIGIN resolves the kernel library there too.
    shutil.copy2(SHIM_LIB, os.path.join(dst_dir, "libst_pybinding.so"))
    shutil.copy2(KERNEL_LIB, os.path.join(dst_dir, "libfo_kernels.so"))
    return SHIM_LIB


def build_all(shim=True):
    out = [build_kernels()]
    if shim:
        out.append(build_shim())
    return out


if __name__ == "__main__":
    for path in build_all(shim="--no-shim" not in sys.argv):
        print("built", path)
