"""The three-instruction division of the FP8 quantisation kernels (``div16_exact`` in ``vllm_amd/csrc/vaq_common.h``)
equals the IEEE quotient: exhaustive check on the host (``tests/native/exact_div_check.c``) over every fp32 significand
of the divisor and every bfloat16 / float16 significand of the dividend, which covers all normal-range inputs."""
import os
import shutil
import subprocess

import pytest

SRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "exact_div_check.c")


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    exe = str(tmp_path_factory.mktemp("exact_div") / "exact_div_check")
    subprocess.run([gcc, "-O2", "-mfma", "-ffp-contract=off", "-fopenmp", SRC, "-o", exe, "-lm"], check=True)
    return exe


def test_device_code_states_the_checked_formula():
    text = open(os.path.join(os.path.dirname(SRC), "..", "..", "vllm_amd", "csrc", "vaq_common.h")).read()
    body = text[text.index("float div16_exact"):]
    body = body[:body.index("}")]
    assert "v_mul_f32 %0, %1, %2" in body and "v_fma_f32 %0, %1, %2, -%3" in body and "v_fma_f32 %0, -%1, %2, %3" in body


def test_bfloat16_dividends_exhaustive(checker):
    r = subprocess.run([checker, "7"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout


def test_float16_dividends_every_fourth_divisor(checker):
    # all 2^23 divisor significands take ~15 s of CPU time; every fourth one here, the full run is `exact_div_check 10`
    r = subprocess.run([checker, "10", "4"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout


def test_the_checker_can_fail(checker):
    r = subprocess.run([checker, "7", "64", "1"], capture_output=True, text=True)     # plain reciprocal multiply
    assert r.returncode == 1 and "mismatches=" in r.stdout
