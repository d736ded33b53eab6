"""Bolt's own Tensor-level operators (the reference's sources compiled into oracle/_ref/libboltref.so) and the gfx950
library through include/bolt_gfx950_tensor.hpp, side by side in one C++ program (tests/glue_test.cpp, built by
`make -C oracle glue` where the reference checkout is present): QuantizeLinear -> FullyConnected -> FullyConnected with the
activations resident in device memory between the operators, an int8 convolution through the six convolution_* calls, a
batched int8 matmul -- every result compared byte for byte with the reference's."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "oracle", "_ref", "glue_test")


@pytest.mark.gpu
def test_tensor_glue_matches_the_reference_operators():
    from checkers import host_has_vnni
    if not os.path.exists(EXE) or not host_has_vnni():
        pytest.skip("oracle/_ref/glue_test not built or host lacks avx512_vnni")
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "glue OK" in r.stdout and r.stdout.count("equal:") == 5


@pytest.mark.skipif(not os.path.isdir("/root/reference/compute/tensor"), reason="no reference checkout here")
def test_tensor_glue_compiles_against_the_reference_headers():
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "glue_syntax"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
