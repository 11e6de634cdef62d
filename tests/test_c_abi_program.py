"""The C ABI from plain C: tests/c_abi/decode_once.c includes only include/lng_hip.h, links only
liblng_hip.so, and is what a foreign-function binding (a Rust crate over this C ABI)
would do. Without a GPU it must compile and link; with one it must run and agree with itself."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_DIR = os.path.join(ROOT, "loadngo_amd")
SRC = os.path.join(ROOT, "tests", "c_abi", "decode_once.c")


def _build(tmp_path):
    exe = str(tmp_path / "decode_once")
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-O1", "-I", os.path.join(ROOT, "include"),
                           SRC, "-o", exe, "-L", LIB_DIR, "-llng_hip", "-lm", "-Wl,-rpath," + LIB_DIR,
                           "-Wl,-rpath,/opt/rocm/lib", "-Wl,-rpath-link,/opt/rocm/lib"])
    return exe


def test_a_c_program_compiles_and_links_against_the_header_and_the_library(tmp_path):
    if not os.path.exists(os.path.join(LIB_DIR, "liblng_hip.so")):
        pytest.fail("liblng_hip.so is not built: run `python -m loadngo_amd.build`")
    _build(tmp_path)


@pytest.mark.gpu
def test_the_c_program_runs_a_decode_with_a_callback(tmp_path):
    exe = _build(tmp_path)
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, (out.returncode, out.stdout, out.stderr)
    assert "refused: unsupported grouped attention shape" in out.stdout
    assert "checksum" in out.stdout
