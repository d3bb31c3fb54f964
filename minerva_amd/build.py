"""Builds the gfx950 operator library and the host layer in-tree.

  libmnv_hip.so   HIP kernels + C ABI (include/mnv_hip.h)   <- minerva_amd/csrc/*.hip
  libmnv_host.so  C++ host layer mirroring Minerva's operator and device interface,
                  linked against libmnv_hip.so              <- minerva_amd/host/*.cpp

hipcc cross-compiles for gfx950 without a GPU, so this runs anywhere ROCm is installed.
build() drives hipcc and g++ directly; build_with_cmake() runs the top-level CMakeLists.txt
(the build a Minerva tree consumes) with the libraries written to the same place.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB_HIP = os.path.join(LIBDIR, "libmnv_hip.so")
LIB_HOST = os.path.join(LIBDIR, "libmnv_host.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    # packed fp32 instructions are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-pthread",
              "-I" + os.path.join(ROOT, "include"), "-I" + HOST]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass of hipcc does not know the packed-fp32 feature and says so: harmless
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _compile_hip(src):
    obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
    _run([HIPCC] + HIP_FLAGS + ["-c", src, "-o", obj])
    return obj


def _compile_host(src):
    obj = os.path.join(OBJDIR, "host_" + os.path.basename(src) + ".o")
    _run(["g++"] + HOST_FLAGS + ["-c", src, "-o", obj])
    return obj


def build(verbose=True, jobs=8):
    os.makedirs(OBJDIR, exist_ok=True)
    hip_srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    host_srcs = sorted(glob.glob(os.path.join(HOST, "*.cpp")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        hip_objs = list(pool.map(_compile_hip, hip_srcs))
        host_objs = list(pool.map(_compile_host, host_srcs))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_HIP] + hip_objs)
    if verbose:
        print("built", LIB_HIP, "from", len(hip_srcs), "HIP sources")
    if host_objs:
        _run(["g++", "-shared", "-fPIC", "-pthread", "-o", LIB_HOST] + host_objs +
             ["-L" + LIBDIR, "-lmnv_hip", "-Wl,-rpath,$ORIGIN"])
        if verbose:
            print("built", LIB_HOST, "from", len(host_srcs), "host sources")
    return LIB_HIP


def build_with_cmake(build_dir=None, jobs=8, verbose=True):
    """Configures and builds the top-level CMake project; libraries go to minerva_amd/lib."""
    build_dir = build_dir or os.path.join(ROOT, "build")
    _run(["cmake", "-S", ROOT, "-B", build_dir, "-DCMAKE_BUILD_TYPE=Release",
          "-DMNV_OUTPUT_DIR=" + LIBDIR])
    _run(["cmake", "--build", build_dir, "-j%d" % jobs])
    if verbose:
        print("built", LIB_HIP, "and", LIB_HOST, "with cmake in", build_dir)
    return LIB_HIP


if __name__ == "__main__":
    if "--cmake" in sys.argv[1:]:
        build_with_cmake()
    else:
        build()
    sys.exit(0)
