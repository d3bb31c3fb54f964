"""CPU tests of the host layer (no GPU):
 * PooledDataStore and ThreadedDevice (four workers, concurrent producers and frees, error
   path) with a malloc allocator, built and run under the address + undefined-behaviour
   sanitizers and under the thread sanitizer;
 * the host layer's operator functions, closures, enums and device classes held mechanically
   to the reference's interface (tests/golden/interface.json, written from the reference's
   headers by tests/golden/extract_reference_interface.py)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "minerva_amd", "host")
GOLD = os.path.join(ROOT, "tests", "golden")
sys.path.insert(0, GOLD)
import interface_parser as ip  # noqa: E402


@pytest.mark.parametrize("sanitizer", ["address,undefined", "thread"])
def test_threaded_device_and_pool_under_sanitizers(tmp_path, sanitizer):
    exe = str(tmp_path / "device_threads_test")
    srcs = [os.path.join(ROOT, "tests", "host_cpu", "device_threads_test.cpp"),
            os.path.join(HOST, "device.cpp"), os.path.join(HOST, "pooled_data_store.cpp")]
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer", "-pthread",
           "-fsanitize=" + sanitizer, "-fno-sanitize-recover=all", "-I" + HOST] + srcs + ["-o", exe]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr[-3000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1", TSAN_OPTIONS="halt_on_error=1")
    env.pop("LD_PRELOAD", None)
    run = subprocess.run([exe], capture_output=True, text=True, timeout=600, env=env)
    assert run.returncode == 0 and run.stdout.strip().endswith("OK"), (run.stdout + run.stderr)[-4000:]


@pytest.fixture(scope="module")
def ref():
    return json.load(open(os.path.join(GOLD, "interface.json")))


def _read(name):
    return open(os.path.join(HOST, name)).read()


# the parameter-server hook is outside the operator path (no such closure or function here)
OUT_OF_SCOPE = {"SyncWithPS", "SyncWithPSClosure"}


def test_operator_functions_have_the_reference_parameter_lists(ref):
    mine = ip.free_functions(_read("hip_ops.h"), "hip")
    for name, params in ref["operators"].items():
        if name in OUT_OF_SCOPE:
            continue
        assert name in mine, "hip::%s is missing" % name
        assert mine[name] == params, "hip::%s%r differs from cuda::%s%r" % (name, mine[name], name, params)
    extra = set(mine) - set(ref["operators"])
    # CPU-only operators of the reference installed on the GPU here, and the seed control
    assert extra <= {"ThresholdNorm", "SetRandomSeed"}, extra


def test_closures_and_enums_have_the_reference_fields(ref):
    types_h = _read("minerva_types.h")
    mine = ip.structs(types_h)
    for name, fields in ref["closures"].items():
        if name in OUT_OF_SCOPE:
            continue
        assert name in mine, "closure %s is missing" % name
        assert mine[name] == fields, "%s: %r vs the reference's %r" % (name, mine[name], fields)
    enums = ip.enums(types_h)
    for name, values in ref["enums"].items():
        assert enums.get(name) == values, name


def test_device_classes_have_the_reference_member_functions(ref):
    device_h = _read("device.h")
    for cls in ("Device", "ThreadedDevice"):
        mine, want = ip.class_methods(device_h, cls), ref["classes"][cls]
        assert mine["base"] == want["base"], cls
        for name, m in want["methods"].items():
            assert name in mine["methods"], "%s::%s is missing" % (cls, name)
            got = mine["methods"][name]
            for key in ("ret", "params", "const", "pure", "access"):
                assert got[key] == m[key], "%s::%s %s: %r vs %r" % (cls, name, key, got[key], m[key])
            assert got["virtual"] or got["override"], "%s::%s must be virtual" % (cls, name)
    # the GPU device overrides what the reference's GpuDevice overrides, with the same
    # parameter lists, from the same base
    hip, gpu = ip.class_methods(_read("hip_device.h"), "HipDevice"), ref["classes"]["GpuDevice"]
    assert hip["base"] == gpu["base"] == "ThreadedDevice"
    for name, m in gpu["methods"].items():
        got = hip["methods"].get(name)
        assert got and got["override"], "HipDevice must override %s" % name
        assert got["params"] == m["params"] and got["ret"] == m["ret"] and got["const"] == m["const"], name


def test_device_manager_has_the_reference_member_functions(ref):
    # minerva/device/device_manager.h:9-26
    want = ref["classes"]["DeviceManager"]
    mine = ip.class_methods(_read("device_manager.h"), "DeviceManager")
    assert mine is not None and mine["base"] == want["base"]
    assert set(mine["methods"]) == set(want["methods"])
    for name, m in want["methods"].items():
        got = mine["methods"][name]
        for key in ("ret", "params", "const", "access", "virtual"):
            assert got[key] == m[key], "DeviceManager::%s %s: %r vs %r" % (name, key, got[key], m[key])


def test_interface_fixture_is_what_the_extractor_writes():
    """Where the reference tree is present (the build container), the committed fixture must be
    what the extractor produces from it today."""
    ref_root = "/root/reference"
    if not os.path.isdir(os.path.join(ref_root, "minerva")):
        pytest.skip("the reference tree is not on this machine")
    read = lambda rel: open(os.path.join(ref_root, rel)).read()
    want = json.load(open(os.path.join(GOLD, "interface.json")))
    assert ip.free_functions(read("minerva/op/impl/cuda.h"), "cuda") == want["operators"]
    assert ip.structs(read("minerva/op/closure.h")) == want["closures"]
    assert ip.class_methods(read("minerva/device/device_manager.h"), "DeviceManager") == \
        want["classes"]["DeviceManager"]
