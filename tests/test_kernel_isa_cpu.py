"""Build-time guards for the GEMM loops that count their own memory operations (gemm_u8s8_dma_kernel: explicit
`s_waitcnt vmcnt(n)` around LDS-bound tile requests, and, with PIPE 4, B fragments loaded by instructions issued as
text). The compiler does not know the text loads, so a register it spilled or re-used while such a load is in flight
would be stored before its data arrived or overwritten when the load returns; and every scratch access is itself a
vector memory operation that the hand-written counts do not include. The tests compile gemm.hip to gfx950 assembly
(no GPU needed) and check that NO instantiation of that kernel uses scratch memory at all -- prologue, loop, tail and
epilogue alike -- that the text loads are there, and that the pinned-order loops keep their order."""
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


def resources(asm):
    """name -> {"ScratchSize": n, "NumVgprs": n, ...} from the compiler's per-kernel report"""
    res, name = {}, None
    for line in asm.splitlines():
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name = m.group(1)
        m = re.match(r"^; (NumVgprs|NumAgprs|ScratchSize|Occupancy): (\d+)", line)
        if m and name:
            res.setdefault(name, {})[m.group(1)] = int(m.group(2))
    return res


def test_no_scratch_in_any_loop_with_hand_counted_memory_operations(gemm_asm):
    """Whole-kernel check: the compiler's own resource report must say 0 bytes of scratch for every instantiation of
    gemm_u8s8_dma_kernel, and no scratch instruction may appear anywhere in their bodies (the stretch from the first
    tile request to the final drain included, and the epilogues behind it)."""
    rs, ks = resources(gemm_asm), kernels(gemm_asm)
    names = [n for n in rs if "gemm_u8s8_dma_kernel" in n]
    assert len(names) >= 12, sorted(names)
    pipes = set()
    for n in names:
        pipes.add(int(re.search(r"gemm_u8s8_dma_kernelILi\d+ELi\d+ELi\d+ELi\d+ELi\d+ELi(\d+)E", n).group(1)))
        assert rs[n]["ScratchSize"] == 0, "%s: %d bytes of scratch per lane" % (n, rs[n]["ScratchSize"])
        assert rs[n]["NumVgprs"] + rs[n]["NumAgprs"] <= 256, n    # two waves per SIMD
        assert not [ins for ins in ks[n] if ins.startswith("scratch_")], n
    assert {3, 4} <= pipes, "the whole-line loops (PIPE 3 and 4) are missing: %s" % sorted(pipes)
    # the convolution's filter-panel kernels keep 64 (TM = 4) accumulators in registers across a grid-wide exchange in
    # their epilogue: spilled there, every launch writes and re-reads a tensor's worth of scratch (25 MB at 32 x 64 x 56
    # x 56 -> 64 channels, seen as five times the result's bytes on the write counter)
    panels = [n for n in rs if "conv_u8s8_panel_kernel" in n]
    assert len(panels) == 4, sorted(panels)
    for n in panels:
        assert rs[n]["ScratchSize"] == 0, "%s: %d bytes of scratch per lane" % (n, rs[n]["ScratchSize"])
        assert not [ins for ins in ks[n] if ins.startswith("scratch_")], n


def test_no_spill_stores_inside_the_register_b_loop(gemm_asm):
    ks = kernels(gemm_asm)
    # template arguments <WM, WN, TM, TN, STAGES, PIPE, ...>: PIPE == 4 is the sixth
    loops = {n: body for n, body in ks.items() if re.search(r"gemm_u8s8_dma_kernelILi\d+ELi\d+ELi\d+ELi\d+ELi\d+ELi4E", n)}
    assert len(loops) >= 2, "expected the register-B loop with and without the GELU epilogue, found %s" % sorted(loops)
    for name, body in loops.items():
        mf = [i for i, ins in enumerate(body) if ins.startswith("v_mfma_i32_16x16x64_i8")]
        assert mf, name
        region = body[mf[0]:mf[-1] + 1]
        # (32-bit lane offset in a vector register + the wave's 64-bit base in a scalar pair)
        text_loads = [ins for ins in region if re.match(r"global_load_dwordx4 v\[\d+:\d+\], v\d+, s\[\d+:\d+\]", ins)]
        assert len(text_loads) >= 12, "%s: the B loads issued as text are missing from the loop" % name
        stores = [ins for ins in region if ins.startswith("scratch_store")]
        assert not stores, "%s: the compiler spills inside the loop with hand-counted loads: %s" % (name, stores[:3])


def test_pinned_order_loops_keep_their_order(gemm_asm):
    """The 128 x 128 loops whose K step is written out instruction by instruction (PIPE 7, and PIPE 8 = the same by two
    wave groups): their point is that every fragment read, tile request and re-bias sits BEHIND an MFMA, so that a
    wave alone on its SIMD issues it while the matrix pipe is busy. Checked on the generated code: inside the K loop no
    MFMA is preceded by more than a handful of vector / memory instructions, nothing spills, and a step's four
    tile requests and (but for a walk's last step) eight fragment reads are all there."""
    ks = kernels(gemm_asm)
    for pipe in (7, 8):
        names = [n for n in ks if re.search(r"gemm_u8s8_dma_kernelILi2ELi2ELi4ELi4ELi4ELi%dE" % pipe, n)]
        assert names, "no instantiation of the pinned-order loop (PIPE %d)" % pipe
        for name in names:
            body = ks[name]
            bars = [i for i, ins in enumerate(body) if ins == "s_barrier"]
            # a K step = the stretch between two barriers that holds exactly 16 MFMAs
            steps = []
            for b0, b1 in zip(bars, bars[1:]):
                seg = body[b0 + 1:b1]
                if sum(ins.startswith("v_mfma_i32_16x16x64_i8") for ins in seg) == 16:
                    steps.append(seg)
            assert len(steps) >= 2, "%s: found %d K steps of 16 MFMAs" % (name, len(steps))
            for seg in steps:
                assert not any(ins.startswith("scratch_") for ins in seg), name
                assert sum(ins.startswith("global_load_lds_dwordx4") for ins in seg) == 4, name
                # (the last step of a walk reads no fragments: nothing would use them)
                assert sum(ins.startswith("ds_read_b128") for ins in seg) in (0, 8), name
                run = 0  # vector ALU / LDS / memory instructions since the last MFMA (scalar ones issue beside them)
                first = True
                for ins in seg:
                    if ins.startswith("v_mfma"):
                        limit = 4 if first else 9  # in front of the first MFMA only address arithmetic may stand
                        assert run <= limit, "%s: %d vector instructions in front of an MFMA" % (name, run)
                        run, first = 0, False
                    elif ins.startswith(("v_", "ds_", "global_", "buffer_")):
                        run += 1

