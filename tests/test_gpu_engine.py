"""The engine's operator classes for the gfx950 back end (include/bolt_gfx950_engine.hpp: FullyConnectedGFX950,
ConvolutionGFX950, MatMulGFX950, QuantizeLinearGFX950, derived from Bolt's own CPU classes) next to those CPU classes, in
one C++ program driven the way the engine drives an operator (tests/engine_test.cpp, built by `make -C oracle engine`
where the reference checkout is present): QuantizeLinear -> FullyConnected -> FullyConnected and Convolution ->
Convolution chains with the activations resident in device memory, fp32 weights quantised at load by each side's own
transform_filter, stored feature scales (dynamic, calibrated, -2), MatMul. Descs, bytes and tensor scales must be equal."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "oracle", "_ref", "engine_test")


@pytest.mark.gpu
def test_engine_operators_match_the_reference_classes():
    from checkers import host_has_vnni
    if not os.path.exists(EXE) or not host_has_vnni():
        pytest.skip("oracle/_ref/engine_test not built or host lacks avx512_vnni")
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "engine operators: all equal" in r.stdout and r.stdout.count("equal:") == 20


@pytest.mark.skipif(not os.path.isdir("/root/reference/inference/engine"), reason="no reference checkout here")
def test_engine_classes_and_factory_compile_against_the_reference_headers():
    """-fsyntax-only over the header with the factory switched on: FactoryGFX950 derives from FactoryCPU and needs every
    operator header of the engine, so it is compiled here and never linked."""
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "engine_syntax"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
