"""Builds the native parts in-tree:

  catch_amd/lib/libcatchq.so        hand-written gfx950 HIP kernels behind the C ABI of include/catchq.h
  catch_amd/lib/_catchq_torch.so    PyTorch-ROCm extension registering the torch_mlu::* ops on top of it

hipcc cross-compiles for gfx950 without a GPU.  Run ``python catch_amd/build.py [kernels|torch|all]`` (by path: the package itself cannot be
imported before its libraries exist).
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
INCLUDE = os.path.join(ROOT, "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

KERNEL_SOURCES = ["quantize.hip", "contract_direct.hip", "igemm_i8.hip", "igemm_i8_dma_gemm.hip", "igemm_i8_dma_conv.hip", "igemm_i8_dual.hip", "igemm_i8_chain.hip", "conv3x3_halo_i8.hip", "igemm_a16_dma.hip", "pw_i8.hip", "dwconv_i8.hip", "irb_i8.hip", "stem_pool_i8.hip", "conv1x1_gap_i8.hip", "pool.hip", "diag.hip", "capi.hip",
                  "host_math.cpp"]

# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 from the fp32 epilogue math.
# -ffp-contract=off: the epilogue's multiply/add order is part of the contract (no FMA).
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
             "-fvisibility=hidden", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-I" + INCLUDE, "-I" + CSRC]
# extra compiler flags for experiments, e.g. CATCHQ_EXTRA_HIPFLAGS=-DCATCHQ_TUNING (tile / load-path switches)
HIP_FLAGS += os.environ.get("CATCHQ_EXTRA_HIPFLAGS", "").split()


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_kernels(verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    objs = []
    procs = []
    for src in KERNEL_SOURCES:
        obj = os.path.join(LIBDIR, src.rsplit(".", 1)[0] + ".o")
        cmd = [HIPCC] + HIP_FLAGS + (["-x", "hip"] if src.endswith(".hip") else []) + \
              ["-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for cmd, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
        if verbose and out.strip():
            print(out)
    lib = os.path.join(LIBDIR, "libcatchq.so")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    return lib


def build_torch_ext(verbose=False):
    """g++ against the torch headers; links libcatchq.so (found through $ORIGIN at run time)."""
    import torch
    from torch.utils import cpp_extension as ce
    os.makedirs(LIBDIR, exist_ok=True)
    out = os.path.join(LIBDIR, "_catchq_torch.so")
    inc = ce.include_paths() + [os.path.join(ROCM, "include"), INCLUDE, sysconfig.get_paths()["include"]]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-Wno-deprecated-declarations"]
    cmd += ["-I" + p for p in inc]
    cmd += [os.path.join(CSRC, "torch_ops.cpp"), "-o", out]
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd += ["-L" + tlib, "-L" + LIBDIR, "-L" + os.path.join(ROCM, "lib"), "-lc10", "-lc10_hip", "-ltorch_cpu",
            "-ltorch_hip", "-ltorch", "-lcatchq", "-lamdhip64", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib]
    o = _run(cmd)
    if verbose and o.strip():
        print(o)
    return out


def build_all(verbose=False):
    return build_kernels(verbose), build_torch_ext(verbose)


if __name__ == "__main__":
    which = sys.argv[1] if len(sys.argv) > 1 else "all"
    if which in ("kernels", "all"):
        print(build_kernels(True))
    if which in ("torch", "all"):
        print(build_torch_ext(True))
