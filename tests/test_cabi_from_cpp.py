"""The C ABI from a C++ program: tests/cabi/gemm_from_cpp.cpp includes include/daceml_hip.h, links against
libdaceml_hip.so and calls dmlhip_gemm_f16 with plain pointers. On the CPU the program is compiled and linked (the
header parses as C++, the symbols resolve); on a GPU it runs products in every operand layout and checks sampled
outputs against double-precision dot products computed inside the program."""
import os
import subprocess

import pytest

from tests.cabi import build as B


def test_program_compiles_and_links_against_the_library():
    exe = B.build()
    assert os.path.exists(exe)
    # without arguments it prints its usage and touches no GPU
    res = subprocess.run([exe], capture_output=True, text=True)
    assert res.returncode == 1 and "usage" in res.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("shape", ["512 384 256", "1000 264 192"])
@pytest.mark.parametrize("layouts", ["k k", "k r", "r k", "r r"])
def test_product_from_cpp(shape, layouts):
    if not os.path.exists(B.EXE):
        B.build()
    res = subprocess.run([B.EXE, *shape.split(), *layouts.split(), "-1", "2", "check"], capture_output=True, text=True,
                         timeout=100)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "check: 0 of 2000" in res.stdout


def test_the_measurement_program_compiles():
    """tests/cabi/simd_issue_probe.hip (instruction-issue measurements quoted in the design notes) keeps building."""
    assert os.path.exists(B.build_probe())
