"""Builds libfrink_hip (shared for ctypes/FFI loaders, static for a Rust build.rs to link)
with hipcc for gfx950.  `python -m frink_amd.build` or `frink_amd.build.build_lib()`."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
SO = os.path.join(LIBDIR, "libfrink_hip.so")
STATIC = os.path.join(LIBDIR, "libfrink_hip.a")

SOURCES = ["frk_runtime.cpp", "frk_quant.hip", "frk_gemv.hip", "frk_gemv_fused.hip", "frk_gemm.hip", "frk_gemm_q6.hip", "frk_gemm_q8.hip", "frk_moe.hip", "frk_thin.hip", "frk_gemv_direct.hip", "frk_gemv_f32dot.hip", "frk_kinds.hip", "frk_probe.hip"]

# -ffp-contract=off: the bit-exact kernels must round every f32 operation separately, and the
# others spell fmaf() where they want a fused multiply-add.  Packed-FP32 instructions are
# switched off for the device pass (the host pass warns that it does not know the feature).
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unused-command-line-argument",
]


def hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    return "hipcc"


def build_lib(verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc()] + HIPCC_FLAGS + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l]
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, "\n".join(lines)))
        if verbose and lines:
            print("\n".join(lines))
    subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", SO] + objs)
    if os.path.exists(STATIC):
        os.remove(STATIC)
    subprocess.check_call(["ar", "rcs", STATIC] + objs)
    return SO


HOST_CHECK_SRC = os.path.join(os.path.dirname(HERE), "tests", "host_mirror_check.cpp")
HOST_CHECK_BIN = os.path.join(LIBDIR, "host_mirror_check")


def build_host_check():
    """The C++ host mirror's test driver (g++, host only), linked against the shared library."""
    os.makedirs(LIBDIR, exist_ok=True)
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", HOST_CHECK_SRC, "-o", HOST_CHECK_BIN,
                           "-L" + LIBDIR, "-lfrink_hip", "-Wl,-rpath," + LIBDIR, "-Wl,-rpath,/opt/rocm/lib"])
    return HOST_CHECK_BIN


if __name__ == "__main__":
    print(build_lib(verbose="-v" in sys.argv))
    print(build_host_check())
