"""The C++ host side (include/lng_compute.hpp: the reference's Gpu / Buffer / Resident / Slice / Batch /
GroupedShape / Completed / Error over the C ABI) under the reference's own operator tests, restated in
tests/cpp/ (metal-compute/tests/attention_grouped.rs, q8_0_and_gpt_oss_glue.rs, glue.rs: same shapes,
generator, float64 definitions and bounds), and the entry points without a counterpart there against the
sequences of reference operators they stand for (tests/cpp/additions.cpp). Without a GPU the programs must compile, link and refuse to run
with NoDevice; with one they must pass."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_DIR = os.path.join(ROOT, "loadngo_amd")
PROGRAMS = {
    "additions": ("batched_decode_is_one_plain_call_per_sequence", "prepare_attention_is_the_reference_sequence_of_dispatches",
                  "q8_product_of_bf16_positions_is_the_f32_product", "decoding_products_fold_their_neighbours_in",
                  "checksum_is_the_xor_of_the_words_and_switches_pick_kernels"),
    "attention_grouped": ("matches_the_float64_definition", "tiled_matches_the_float64_definition",
                          "sinks_take_probability_without_value_on_gpt_oss_shapes", "rejects_shapes_it_cannot_run",
                          "ownership_residents_and_bf16"),
    "q8_0_and_glue": ("q8_0_products_match_the_float64_definition", "q8_0_rejects_partial_blocks",
                      "glue_adds_and_rotates_as_defined", "partial_rotation_is_as_defined",
                      "strided_rmsnorm_and_row_copy_touch_only_their_columns"),
}


def _build(tmp_path, name):
    if not os.path.exists(os.path.join(LIB_DIR, "liblng_hip.so")):
        pytest.fail("liblng_hip.so is not built: run `python -m loadngo_amd.build`")
    exe = str(tmp_path / name)
    subprocess.check_call(["g++", "-std=c++17", "-O2", "-fopenmp", "-pthread", "-Wall", "-Wextra", "-Werror",
                           "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "cpp", name + ".cpp"),
                           "-o", exe, "-L", LIB_DIR, "-llng_hip",
                           "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath,/opt/rocm/lib", "-Wl,-rpath-link,/opt/rocm/lib"])
    return exe


@pytest.mark.parametrize("name", sorted(PROGRAMS))
def test_the_cpp_host_layer_compiles_and_fails_loudly_without_a_device(tmp_path, name):
    from loadngo_amd import compute as C
    exe = _build(tmp_path, name)
    try:
        C.Gpu().close()
        return                      # a GPU is present: the gpu-marked test runs the program
    except C.NoDevice:
        pass
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 100 and "no HIP device" in out.stdout, (out.returncode, out.stdout, out.stderr)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(PROGRAMS))
def test_the_reference_operator_tests_pass_through_the_cpp_host_layer(tmp_path, name):
    exe = _build(tmp_path, name)
    out = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, (out.returncode, out.stdout[-3000:], out.stderr[-2000:])
    for test in PROGRAMS[name]:
        assert "done " + test in out.stdout
    assert "0 failures" in out.stdout and "FAILED" not in out.stdout
