"""Builds libcam_mi355x.so (HIP kernels + C ABI) for gfx950 with hipcc, and libcam_torch_ops.so (the C++
registration of torch.ops.umdk_cam_op_lib on top of that ABI) with the host compiler, both in-tree.

`python -m umdk_original_amd.build --timeline` builds a second library beside them, libcam_mi355x_timeline.so:
the same sources with -DCAM_GEMM_TIMELINE, whose grouped-GEMM kernel stamps every tile of its schedule with
the device clock.  It is a profiling aid and is only loaded when CAM_MI355X_LIB names it.  libcam_calib.so holds the
calibration micro-benchmarks behind `bench.py --only calib` and nothing of the product."""
import os
import subprocess
import sys

_PKG = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_PKG, "csrc")
LIB_DIR = os.path.join(_PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcam_mi355x.so")
TIMELINE_LIB_PATH = os.path.join(LIB_DIR, "libcam_mi355x_timeline.so")
CALIB_LIB_PATH = os.path.join(LIB_DIR, "libcam_calib.so")  # calibration micro-benchmarks, loaded by bench.py only
ABI_CONSUMER_PATH = os.path.join(LIB_DIR, "abi_consumer")  # plain-C caller of the ABI (csrc/abi_consumer.c), for tests
SOURCES = ["abi.cpp", "plan.hip", "dispatch.hip", "combine.hip", "gemm.hip"]

# -packed-fp32-ops is switched off on purpose: packed fp32 VALU forms are not used by this library.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # the direct-to-LDS loads name m0 as clobbered; clang notes that it does not preserve reserved registers
    "-Wno-inline-asm",
]


def build(verbose=False, timeline=False):
    """Compile every source and link the shared library. Always recompiles."""
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    extra = ["-DCAM_GEMM_TIMELINE"] if timeline else []
    for src in SOURCES:
        obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + (".timeline.o" if timeline else ".o"))
        cmd = [hipcc] + HIPCC_FLAGS + extra + ["-x", "hip", "-c", os.path.join(_CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
        if verbose and out.strip():
            print(out)
    out_path = TIMELINE_LIB_PATH if timeline else LIB_PATH
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out_path] + objs
    subprocess.check_call(cmd)
    for o in objs:
        os.remove(o)
    if not timeline:
        build_calib(verbose)
        build_abi_consumer(verbose)
        build_torch_ops(verbose)
    return out_path


def build_abi_consumer(verbose=False):
    """csrc/abi_consumer.c, compiled as C by the host compiler: the header has to be a C header, and the library has
    to be usable with nothing but the HIP runtime beside it."""
    cc = os.environ.get("CC", "gcc")
    cmd = [cc, "-std=c11", "-O1", "-Wall", "-Wextra", "-Werror", "-I", "/opt/rocm/include",
           os.path.join(_CSRC, "abi_consumer.c"), "-o", ABI_CONSUMER_PATH,
           "-L", LIB_DIR, "-lcam_mi355x", "-L", "/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("building %s failed:\n%s" % (ABI_CONSUMER_PATH, p.stdout))
    return ABI_CONSUMER_PATH


def build_calib(verbose=False):
    """The calibration micro-benchmarks (csrc/calib.hip): a library of their own, never linked into the product."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-shared", "-x", "hip", os.path.join(_CSRC, "calib.hip"), "-o", CALIB_LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed on calib.hip:\n%s" % p.stdout)
    return CALIB_LIB_PATH


TORCH_OPS_PATH = os.path.join(LIB_DIR, "libcam_torch_ops.so")


def build_torch_ops(verbose=False):
    """The torch operator library: host C++ only (no device code), linked against torch and libcam_mi355x.so."""
    import torch
    from torch.utils import cpp_extension
    tdir = os.path.dirname(os.path.abspath(torch.__file__))
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in cpp_extension.include_paths() + ["/opt/rocm/include"]:
        cmd += ["-I", inc]
    cmd += [os.path.join(_CSRC, "torch_binding.cpp"), "-o", TORCH_OPS_PATH,
            "-L", os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
            "-L", LIB_DIR, "-lcam_mi355x", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(tdir, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("building %s failed:\n%s" % (TORCH_OPS_PATH, p.stdout))
    return TORCH_OPS_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, timeline="--timeline" in sys.argv))
