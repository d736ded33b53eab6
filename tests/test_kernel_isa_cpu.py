"""Build-time guard for the GEMM loop whose B fragments are loaded by instructions issued as text
(gemm_u8s8_dma_kernel, PIPE 4): the compiler does not know those loads, so if it ever spilled a register inside the
loop it could store one whose data has not arrived yet -- silently wrong results on some shapes. The test compiles
gemm.hip to gfx950 assembly (no GPU needed) and checks, for every instantiation of that loop, that nothing is stored
to scratch between its first and its last matrix instruction, and that the text loads are there at all."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "bolt_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]   # the flags of bolt_amd/csrc/Makefile


@pytest.fixture(scope="module")
def gemm_asm():
    if not shutil.which(HIPCC):
        pytest.skip("hipcc not available")
    with tempfile.TemporaryDirectory() as d:
        out = os.path.join(d, "gemm.s")
        subprocess.check_call([HIPCC] + FLAGS + ["-S", "--cuda-device-only", os.path.join(CSRC, "gemm.hip"), "-o", out],
                              stderr=subprocess.DEVNULL)
        return open(out).read()


def kernels(asm):
    """name -> list of instruction lines, for every function of the file"""
    res, name = {}, None
    for line in asm.splitlines():
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name = m.group(1)
            res[name] = []
        elif line.startswith(".Lfunc_end"):
            name = None
        elif name and line.startswith("\t") and not line.startswith("\t;") and not line.startswith("\t."):
            res[name].append(line.strip())
    return res


def test_no_spill_stores_inside_the_register_b_loop(gemm_asm):
    ks = kernels(gemm_asm)
    # template arguments <WM, WN, TM, TN, STAGES, PIPE, ...>: PIPE == 4 is the sixth
    loops = {n: body for n, body in ks.items() if re.search(r"gemm_u8s8_dma_kernelILi\d+ELi\d+ELi\d+ELi\d+ELi\d+ELi4E", n)}
    assert len(loops) >= 2, "expected the register-B loop with and without the GELU epilogue, found %s" % sorted(loops)
    for name, body in loops.items():
        mf = [i for i, ins in enumerate(body) if ins.startswith("v_mfma_i32_16x16x64_i8")]
        assert mf, name
        region = body[mf[0]:mf[-1] + 1]
        text_loads = [ins for ins in region if ins.startswith("global_load_dwordx4") and ins.endswith("off")]
        assert len(text_loads) >= 12, "%s: the B loads issued as text are missing from the loop" % name
        stores = [ins for ins in region if ins.startswith("scratch_store")]
        assert not stores, "%s: the compiler spills inside the loop with hand-counted loads: %s" % (name, stores[:3])
