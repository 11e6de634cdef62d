"""The host library without a GPU, under AddressSanitizer and UndefinedBehaviorSanitizer.

`python -m loadngo_amd.build --null-device` compiles loadngo_amd/csrc/lng_hip.cpp against the null device of
loadngo_amd/csrc/null_device (host memory for device memory, launches recorded instead of run);
tests/cpp/null_device.cpp then drives the C ABI: the refusals of metal-compute/src/apple.rs:860-906 and
1243-1277 (the reference's rejected shapes, slices of the wrong length, outside their buffer or off their
element size, outputs in resident memory or over an input, buffers of a batch in flight), the refusals of
copy_rows, prepare_attention and the Q8_0 products, the development switches (environment at open,
lng_hip_debug_set afterwards) and lng_hip_checksum, ownership and lifetimes (close racing the last free on two
threads), allocation failures while recording, and 100,000 random dispatches through the decode planner with
every grid, work table, chunk and scratch size checked on the host. Any sanitizer report fails the run."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_DIR = os.path.join(ROOT, "loadngo_amd")
SANITIZE = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer"]


def test_the_host_library_on_the_null_device_under_sanitizers(tmp_path):
    from loadngo_amd import build
    lib = build.build_null_device()
    assert os.path.exists(lib)
    exe = str(tmp_path / "null_device")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-pthread", "-Wall", "-Wextra", "-Werror", *SANITIZE, "-DLNG_NULL_DEVICE",
                           "-I", os.path.join(LIB_DIR, "csrc", "null_device"), os.path.join(ROOT, "tests", "cpp", "null_device.cpp"),
                           "-o", exe, "-L", LIB_DIR, "-llng_hip_null", "-Wl,-rpath," + LIB_DIR])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe, "100000"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600, env=env)
    assert run.returncode == 0, run.stdout[-4000:]
    assert "null device: all checks held" in run.stdout
    assert "100000 dispatches checked" in run.stdout
    assert "ERROR: AddressSanitizer" not in run.stdout and "runtime error:" not in run.stdout
