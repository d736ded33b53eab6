"""Runs the compile-time check of include/bolt_gfx950.h and include/bolt_types.h against the reference's own headers
(tests/abi_check.cpp: every blas_enhance twin has the reference's exact argument list, the inner tensor_computing
forms differ by a trailing Arch at most, struct sizes / field offsets / enum values agree). Needs the reference
checkout, so it is skipped where that is absent (the GPU box)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(not os.path.isdir("/root/reference/compute/blas_enhance"), reason="no reference checkout here")
def test_headers_match_the_reference():
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "abi"], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.skipif(not os.path.isdir("/root/reference/compute/blas_enhance"), reason="no reference checkout here")
def test_the_check_can_fail(tmp_path):
    """The same translation unit with one deliberately wrong assertion appended must not compile."""
    src = open(os.path.join(ROOT, "tests", "abi_check.cpp")).read()
    bad = tmp_path / "abi_bad.cpp"
    bad.write_text(src + "\nSAME(matrix_matrix_multiply, matrix_vector_multiply_gfx950x);\n".replace("gfx950x", "tmp_bytes_gfx950"))
    ref = "/root/reference"
    inc = [f"-I{ref}/{d}" for d in ("common/uni/include", "common/memory/include", "compute/blas_enhance/include",
                                     "compute/blas_enhance/src", "compute/tensor/include", "compute/tensor/src")]
    defs = ["-D_USE_OPENMP", "-D_USE_GENERAL", "-D_USE_X86", "-D_USE_FP32", "-D_USE_INT8", "-D_USE_INT32",
            "-D_USE_AVX512_VNNI"]
    r = subprocess.run(["g++", "-std=c++11", "-fsyntax-only", "-w"] + defs + inc + [f"-I{ROOT}/include", str(bad)],
                       capture_output=True, text=True)
    assert r.returncode != 0 and "differs from" in r.stderr
