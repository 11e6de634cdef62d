"""The C++ host side (include/lng_compute.hpp: the reference's Gpu / Buffer / Resident / Slice / Batch /
GroupedShape / Completed / Error over the C ABI) under the reference's own operator tests, restated in
tests/cpp/attention_grouped.cpp (metal-compute/tests/attention_grouped.rs: same shapes, generator, float64
definition and bounds). Without a GPU the program must compile, link and refuse to run with NoDevice; with
one it must pass."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_DIR = os.path.join(ROOT, "loadngo_amd")
SRC = os.path.join(ROOT, "tests", "cpp", "attention_grouped.cpp")


def _build(tmp_path):
    if not os.path.exists(os.path.join(LIB_DIR, "liblng_hip.so")):
        pytest.fail("liblng_hip.so is not built: run `python -m loadngo_amd.build`")
    exe = str(tmp_path / "attention_grouped")
    subprocess.check_call(["g++", "-std=c++17", "-O2", "-fopenmp", "-pthread", "-Wall", "-Wextra", "-Werror",
                           "-I", os.path.join(ROOT, "include"), SRC, "-o", exe, "-L", LIB_DIR, "-llng_hip",
                           "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath,/opt/rocm/lib", "-Wl,-rpath-link,/opt/rocm/lib"])
    return exe


def test_the_cpp_host_layer_compiles_and_fails_loudly_without_a_device(tmp_path):
    import torch  # only to learn whether this machine has a GPU
    exe = _build(tmp_path)
    if torch.cuda.is_available():
        return
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 100 and "no HIP device" in out.stdout, (out.returncode, out.stdout, out.stderr)


@pytest.mark.gpu
def test_the_reference_operator_tests_pass_through_the_cpp_host_layer(tmp_path):
    exe = _build(tmp_path)
    out = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, (out.returncode, out.stdout[-3000:], out.stderr[-2000:])
    for name in ("matches_the_float64_definition", "tiled_matches_the_float64_definition",
                 "sinks_take_probability_without_value_on_gpt_oss_shapes", "rejects_shapes_it_cannot_run",
                 "ownership_residents_and_bf16"):
        assert "done " + name in out.stdout
    assert "0 failures" in out.stdout and "FAILED" not in out.stdout
