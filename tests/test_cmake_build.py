"""The CMake build (CPU only: hipcc cross-compiles): configure and build both libraries and
the host test out of tree, run the test, install, and build a consumer project against the
installed package the way a Minerva tree would (find_package + target_link_libraries).
The reference's counterpart is its CUDA build, CMakeLists.txt:59-63,88-110 and
minerva/CMakeLists.txt:10-16."""
import ctypes
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(cmd, cwd=None, timeout=1500):
    proc = subprocess.run(cmd, cwd=cwd, capture_output=True, text=True, timeout=timeout)
    assert proc.returncode == 0, "%s\n%s" % (" ".join(cmd), (proc.stdout + proc.stderr)[-4000:])
    return proc.stdout


@pytest.mark.skipif(shutil.which("cmake") is None, reason="cmake is not installed")
def test_cmake_builds_installs_and_a_consumer_links(tmp_path):
    build, prefix, cons = str(tmp_path / "build"), str(tmp_path / "prefix"), str(tmp_path / "consumer")
    _run(["cmake", "-S", ROOT, "-B", build, "-DBUILD_TESTS=ON", "-DCMAKE_BUILD_TYPE=Release"])
    _run(["cmake", "--build", build, "-j8"])
    assert "100% tests passed" in _run(["ctest", "--output-on-failure"], cwd=build)
    hip = os.path.join(build, "lib", "libmnv_hip.so")
    host = os.path.join(build, "lib", "libmnv_host.so")
    assert os.path.exists(hip) and os.path.exists(host)
    # every entry point of the header is exported by the CMake-built library too
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "mnv_hip.h")).read(), flags=re.S)
    lib = ctypes.CDLL(hip)
    missing = [n for n in sorted(set(re.findall(r"\b(mnv_[a-z0-9_]+)\s*\(", text))) if not hasattr(lib, n)]
    assert not missing, missing
    ctypes.CDLL(host)  # resolves libmnv_hip.so through its $ORIGIN run path
    _run(["cmake", "--install", build, "--prefix", prefix])
    for rel in ("include/mnv_hip.h", "include/mnv_host.h", "include/minerva_amd/host/hip_ops.h",
                "lib/libmnv_hip.so", "lib/libmnv_host.so", "lib/cmake/MinervaAmd/MinervaAmdConfig.cmake"):
        assert os.path.exists(os.path.join(prefix, rel)), rel
    _run(["cmake", "-S", os.path.join(ROOT, "tests", "cmake_consumer"), "-B", cons,
          "-DCMAKE_PREFIX_PATH=" + prefix])
    _run(["cmake", "--build", cons])
    env = dict(os.environ, LD_LIBRARY_PATH=os.path.join(prefix, "lib"))
    out = subprocess.run([os.path.join(cons, "consumer")], capture_output=True, text=True, env=env,
                         timeout=60)
    assert out.returncode == 0 and "consumer OK" in out.stdout, out.stdout + out.stderr
