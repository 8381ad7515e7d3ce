"""Builds libanemone_hip.so in place: the C11 host side (gcc) and the HIP backend and kernels (hipcc, gfx950); and beside it
libanemone_probe.so, the measurement and self-check kernels (an instruction-rate probe, a plain copy, the exhaustive
arithmetic checks), which are evidence and tests, not part of the drop-in library: they add themselves to the backend's
kernel table when that library is loaded.

    python -m anemone_amd.build [--jobs N]

Cross-compiles without a GPU. The library is git-ignored (history stays source-only) but travels with the tree."""
import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")
LIBRARY = os.path.join(HERE, "libanemone_hip.so")
PROBE_LIBRARY = os.path.join(HERE, "libanemone_probe.so")
EXPORTS = os.path.join(HERE, "host", "exports.map")
BUILD = os.path.join(HERE, "build")

HOST_SOURCES = ["status.c", "prepare_common.c", "weight_format.c", "exl3.c", "exl3_tc.c", "router.c", "linear.c", "expert_fused.c", "site.c", "site_front.c", "step_experts.c", "exl3_layout.c", "sha256.c", "json_tree.c", "exl3_descriptor.c"]
HIP_SOURCES = ["kernel_exl3.hip", "kernel_exl3_tc.hip", "kernel_exl3_tcp.hip", "kernel_router.hip", "kernel_dense_linear.hip", "kernel_activation_quantize.hip", "kernel_wide_linear.hip", "kernel_native_linear.hip",
               "kernel_expert_linear.hip", "kernel_trunk_linear.hip", "kernel_hyper_connection.hip", "kernel_site_front.hip"]
PROBE_SOURCES = ["kernel_calibrate.hip", "kernel_selfcheck.hip"]

BACKEND_SOURCES = ["backend_hip.cpp"]  # host C++ over the HIP runtime API: no device code
BACKEND_FLAGS = ["-std=c++17", "-O2", "-fPIC", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include"]
HOST_FLAGS = ["-std=c11", "-D_GNU_SOURCE", "-O2", "-fPIC", "-ffp-contract=off", "-Wall", "-Wextra", "-Werror=implicit-function-declaration"]
# packed-fp32 instructions are switched off for every HIP translation unit; the host pass warns that it does not
# know the feature, which is harmless
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Xclang", "-target-feature",
             "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


# kernels whose weight loads are issued by hand into registers (csrc/native_device.cuh): the compiler keeps no book on
# when their bytes land, so a register it spilled between the load and the wait would be saved before it is filled.
# Their translation unit is compiled with the resource remarks on, and a kernel of it that spills a vector register
# fails the build.
NO_SPILL_SOURCES = ["kernel_native_linear.hip"]
RESOURCE_REMARKS = ["-Rpass-analysis=kernel-resource-usage", "-Wno-inline-asm"]


def spilling_kernels(output):
    """(kernel, spilled vector registers) of every kernel in a compile's resource remarks that spills one."""
    found, name = [], None
    for line in output.splitlines():
        if "remark:" not in line:
            continue
        text = line.split("remark:", 1)[1].split("[-Rpass", 1)[0].strip()
        if text.startswith("Function Name:"):
            name = text.split(":", 1)[1].strip()
        elif text.startswith("VGPRs Spill:") and int(text.split(":", 1)[1]) > 0:
            found.append((name, int(text.split(":", 1)[1])))
    return found


def run(command):
    result = subprocess.run(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    output = "\n".join(line for line in result.stdout.splitlines() if "packed-fp32-ops" not in line)
    if result.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(command), output))
    return output


def build(jobs=8, verbose=False):
    os.makedirs(BUILD, exist_ok=True)
    commands, objects = [], []
    for name in HOST_SOURCES:
        target = os.path.join(BUILD, name + ".o")
        objects.append(target)
        commands.append(["gcc", *HOST_FLAGS, "-I", INCLUDE, "-c", os.path.join(HERE, "host", name), "-o", target])
    for name in BACKEND_SOURCES:
        target = os.path.join(BUILD, name + ".o")
        objects.append(target)
        commands.append(["g++", *BACKEND_FLAGS, "-I", INCLUDE, "-I", os.path.join(HERE, "csrc"), "-c",
                         os.path.join(HERE, "csrc", name), "-o", target])
    probe_objects = []
    for name in HIP_SOURCES + PROBE_SOURCES:
        target = os.path.join(BUILD, name + ".o")
        (probe_objects if name in PROBE_SOURCES else objects).append(target)
        commands.append(["hipcc", *HIP_FLAGS, *(RESOURCE_REMARKS if name in NO_SPILL_SOURCES else []), "-I", INCLUDE, "-I",
                         os.path.join(HERE, "csrc"), "-c", os.path.join(HERE, "csrc", name), "-o", target])
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for command, output in zip(commands, pool.map(run, commands)):
            if RESOURCE_REMARKS[0] in command:
                spilling = spilling_kernels(output)
                if spilling:
                    raise RuntimeError("%s: kernels with hand-issued register loads spill vector registers: %s" % (command[-3], spilling))
                output = "\n".join(line for line in output.splitlines() if "kernel-resource-usage" not in line)
            if verbose and output.strip():
                print(output)
    run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,--version-script=" + EXPORTS, "-o", LIBRARY, *objects])
    run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROBE_LIBRARY, *probe_objects, "-L", HERE, "-lanemone_hip",
         "-Wl,-rpath,$ORIGIN"])
    return LIBRARY


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    parser.add_argument("--jobs", type=int, default=8)
    parser.add_argument("--verbose", action="store_true")
    arguments = parser.parse_args()
    try:
        print(build(arguments.jobs, arguments.verbose))
    except RuntimeError as error:
        print(error, file=sys.stderr)
        sys.exit(1)
