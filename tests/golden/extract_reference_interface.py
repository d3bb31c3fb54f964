"""Writes interface.json: the reference's operator and device interface as data, so that a
CPU test can hold this repository's host layer to it mechanically.

Reads the reference's headers as text only (nothing is compiled, imported or run):
  minerva/op/impl/cuda.h:10-48      GPU operator functions: names and parameter lists
  minerva/op/closure.h:8-176        enums, closure structs and their fields
  minerva/device/device.h:18-78     Device / ThreadedDevice / GpuDevice member functions
  minerva/device/device_manager.h:9-26   DeviceManager member functions

Usage (in the build container, where /root/reference is mounted):
  python tests/golden/extract_reference_interface.py [/root/reference]
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import interface_parser as ip  # noqa: E402


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    read = lambda rel: open(os.path.join(ref, rel)).read()
    closure_h = read("minerva/op/closure.h")
    device_h = read("minerva/device/device.h")
    manager_h = read("minerva/device/device_manager.h")
    out = {
        "source": {"operators": "minerva/op/impl/cuda.h", "closures": "minerva/op/closure.h",
                   "device": "minerva/device/device.h",
                   "device_manager": "minerva/device/device_manager.h"},
        "operators": ip.free_functions(read("minerva/op/impl/cuda.h"), "cuda"),
        "closures": ip.structs(closure_h),
        "enums": ip.enums(closure_h),
        "classes": dict({c: ip.class_methods(device_h, c) for c in ("Device", "ThreadedDevice", "GpuDevice")},
                        DeviceManager=ip.class_methods(manager_h, "DeviceManager")),
    }
    path = os.path.join(HERE, "interface.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", path, "-", len(out["operators"]), "operators,", len(out["closures"]), "closures")


if __name__ == "__main__":
    main()
