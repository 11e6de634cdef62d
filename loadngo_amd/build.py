"""Builds liblng_hip.so in-tree: the gfx950 code object from csrc/lng_kernels.hip
(``hipcc --genco``), embedded into the host library compiled from csrc/lng_hip.cpp, plus
csrc/lng_static.hip (the fixed device scratch array and the host code that finds it).

    python -m loadngo_amd.build
    python -m loadngo_amd.build --null-device   # the host library alone, against csrc/null_device, with sanitizers
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "liblng_hip.so")
HSACO = os.path.join(HERE, "lng_kernels.hsaco")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

# Packed-FP32 instruction selection is switched off for every kernel.
DEVICE_FLAGS = [
    "--genco", "--offload-arch=gfx950", "-O3", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout)
        raise RuntimeError("build step failed: " + " ".join(cmd))
    return proc.stdout


def build(verbose=False):
    """Compiles the kernels and the host library. Always recompiles."""
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    out = _run([hipcc] + DEVICE_FLAGS + [os.path.join(CSRC, "lng_kernels.hip"), "-o", HSACO])
    if verbose and out:
        print(out)
    # the fixed scratch array and its set-up: a HIP source of its own (device array + the host code that finds it)
    static_obj = os.path.join(HERE, "lng_static.o")
    out = _run([hipcc, "-c", "-fPIC", "--offload-arch=gfx950", "-O2", "-std=c++17",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                os.path.join(CSRC, "lng_static.hip"), "-o", static_obj])
    if verbose and out:
        print(out)
    out = _run([
        "g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wextra", "-Wno-unused-result", "-pthread",
        "-D__HIP_PLATFORM_AMD__", "-DLNG_HSACO_PATH=\"%s\"" % HSACO,
        "-I" + os.path.join(ROCM, "include"),
        os.path.join(CSRC, "lng_hip.cpp"), static_obj, "-o", LIB,
        "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(ROCM, "lib"),
    ])
    if verbose and out:
        print(out)
    return LIB


NULL_LIB = os.path.join(HERE, "liblng_hip_null.so")


def build_null_device(verbose=False):
    """The host library (csrc/lng_hip.cpp) against the null device of csrc/null_device - host memory for device
    memory, launches recorded instead of run - under AddressSanitizer and UndefinedBehaviorSanitizer. For the CPU
    tests of the host logic (tests/test_null_device.py); no GPU code, no ROCm needed."""
    null = os.path.join(CSRC, "null_device")
    out = _run([
        "g++", "-std=c++17", "-O1", "-g", "-fPIC", "-shared", "-Wall", "-Wextra", "-pthread", "-fno-omit-frame-pointer",
        "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-DLNG_NULL_DEVICE", "-I" + null,
        os.path.join(CSRC, "lng_hip.cpp"), os.path.join(null, "null_hip.cpp"), "-o", NULL_LIB,
    ])
    if verbose and out:
        print(out)
    return NULL_LIB


if __name__ == "__main__":
    if "--null-device" in sys.argv[1:]:
        print(build_null_device(verbose=True))
    else:
        print(build(verbose=True))
