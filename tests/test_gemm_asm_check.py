"""The MFMA GEMM kernels keep their MFMAs in inline assembly, which hides from the compiler that accumulator
blocks are still in flight after them.  tests/check_gemm_asm.py looks through the generated assembly
for what that can break (accumulator blocks copied or read too early, scratch memory, function calls, scalar
base addresses written by the vector unit right ahead of an LDS-DMA, MFMA operands written by the vector unit
right ahead of the MFMA).  Here it runs on every GEMM translation unit - the grouped formats, the dense GEMM, the
ring kernel - compiled for gfx950 on the CPU, all at once (two to three minutes on eight cores): the register
allocation of one format's variant says nothing about another's."""
import glob
import os
import subprocess
import sys

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ipex-llm_amd", "csrc")
CHECKER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "check_gemm_asm.py")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-fast-math", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-S", "--cuda-device-only"]


UNITS = ([os.path.basename(p) for p in sorted(glob.glob(os.path.join(CSRC, "gemm_grouped_*.hip")))]
         + ["gemm.hip", "gemm_ring.hip"])


@pytest.fixture(scope="module")
def listings(tmp_path_factory):
    """unit -> path of its assembly listing (or the compiler's return code), all units compiled concurrently"""
    out_dir = tmp_path_factory.mktemp("asm")
    procs = {}
    for unit in UNITS:
        listing = str(out_dir / (unit + ".s"))
        procs[unit] = (listing, subprocess.Popen([HIPCC] + FLAGS + ["-c", os.path.join(CSRC, unit), "-o", listing],
                                                 cwd=CSRC, stderr=subprocess.DEVNULL))
    return {unit: (listing if p.wait() == 0 else p.returncode) for unit, (listing, p) in procs.items()}


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
@pytest.mark.parametrize("unit", UNITS)
def test_generated_assembly_respects_the_mfma_hazards(unit, listings):
    listing = listings[unit]
    assert isinstance(listing, str), "hipcc failed on %s with code %s" % (unit, listing)
    # the 128-row DMA form is held to 128 vector registers, for two workgroups per compute unit, and spills a few;
    # the grouped tall form with eight waves (two per SIMD, 128 vector registers each) may spill outside its loops
    out = subprocess.run([sys.executable, CHECKER, listing, "--allow-scratch", "Lb1ELi4E",
                          "--allow-scratch-outside-loops", "Li8ELb1ELb1ELi8E"],
                         capture_output=True, text=True)
    assert out.returncode == 0, out.stdout[-4000:]
    assert out.stdout.count(": ok") >= 3, out.stdout


def test_the_checker_sees_a_copy_of_a_fresh_accumulator(tmp_path):
    bad = tmp_path / "bad.s"
    bad.write_text("_Z16gemm_mfma_kernelv:\n"
                   "\tv_accvgpr_write_b32 a0, 0\n"
                   "\tv_mfma_f32_32x32x16_bf16 a[0:15], v[0:3], v[4:7], a[0:15]\n"
                   "\tv_mfma_f32_32x32x16_bf16 a[16:31], v[0:3], v[4:7], a[16:31]\n"
                   "\ts_barrier\n"
                   "\tv_accvgpr_mov_b32 a40, a0\n"          # written two MFMAs ago: fine
                   "\tv_accvgpr_mov_b32 a41, a16\n"         # written by the MFMA just issued: not fine
                   "\ts_endpgm\n")
    out = subprocess.run([sys.executable, CHECKER, str(bad)], capture_output=True, text=True)
    assert out.returncode == 1
    assert "a41, a16" in out.stdout and "a40, a0" not in out.stdout


def test_the_checker_sees_an_mfma_operand_written_right_ahead_of_it(tmp_path):
    bad = tmp_path / "bad2.s"
    bad.write_text("_Z16gemm_mfma_kernelv:\n"
                   "\tv_pk_mul_f16 v3, v20, v21\n"
                   "\ts_nop 1\n"
                   "\tv_mfma_f32_32x32x16_f16 a[0:15], v[0:3], v[4:7], a[0:15]\n"      # two wait states: fine
                   "\tv_pk_mul_f16 v9, v20, v21\n"
                   "\tds_read_b128 v[30:33], v40\n"
                   "\tv_mfma_f32_32x32x16_f16 a[16:31], v[8:11], v[4:7], a[16:31]\n"   # one instruction between: not fine
                   "\tv_pk_mul_f16 v50, v20, v21\n"
                   "\tv_mfma_f32_32x32x16_f16 a[32:47], v[8:11], v[4:7], a[32:47]\n"   # writes another register: fine
                   "\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n"
                   "\ts_endpgm\n")
    out = subprocess.run([sys.executable, CHECKER, str(bad)], capture_output=True, text=True)
    assert out.returncode == 1
    assert out.stdout.count("MFMA operand written by VALU") == 1 and "v9, v20, v21" in out.stdout


def test_the_checker_keeps_checking_after_a_spill_and_tells_loops_from_straight_code(tmp_path):
    """A spill used to end the check of a kernel: an operand hazard behind it went unseen.  Spills outside loops
    can be allowed per kernel; inside a loop that holds MFMAs they never are."""
    text = ("_Z16gemm_mfma_kernelILi8ELb1ELb0ELi8EEv:\n"
            "\tscratch_store_dword off, v1, off\n"                 # outside any loop
            ".LBB0_1:                                ; =>This Inner Loop Header: Depth=1\n"
            "\tscratch_load_dword v1, off, off\n"                   # inside the MFMA loop
            "\tv_pk_mul_f16 v3, v20, v21\n"
            "\tv_mfma_f32_32x32x16_f16 a[0:15], v[0:3], v[4:7], a[0:15]\n"
            "\ts_cbranch_scc1 .LBB0_1\n"
            "; %bb.2:\n"
            "\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n"
            "\tscratch_load_dword v2, off, off\n"                   # behind the loop
            "\ts_endpgm\n")
    bad = tmp_path / "bad3.s"
    bad.write_text(text)
    out = subprocess.run([sys.executable, CHECKER, str(bad), "--allow-scratch-outside-loops", "Li8ELb1ELb0ELi8E"],
                         capture_output=True, text=True)
    assert out.returncode == 1
    assert out.stdout.count("scratch access") == 1 and "inside an MFMA loop" in out.stdout
    assert out.stdout.count("MFMA operand written by VALU") == 1
    out = subprocess.run([sys.executable, CHECKER, str(bad)], capture_output=True, text=True)
    assert "scratch access:" in out.stdout and "inside an MFMA loop" in out.stdout      # nothing allowed: both kinds


def test_the_checker_takes_the_innermost_loops_for_the_walks_along_k(tmp_path):
    """A loop around the K loops (a workgroup that takes tile after tile) holds code that runs once per tile: a
    spill there is like one outside loops.  The nested loop's header line carries 'Parent Loop', its own 'Loop
    Header' stands on the comment line below; a reload in it is still an error."""
    text = ("_Z16gemm_mfma_kernelILi8ELb1ELb0ELi8EEv:\n"
            ".LBB0_1:                                ; =>This Loop Header: Depth=1\n"
            "\tscratch_load_dword v2, off, off\n"                   # per tile: allowed when asked for
            "\tv_mfma_f32_32x32x16_f16 a[16:31], v[0:3], v[4:7], a[16:31]\n"   # (an MFMA outside the K loop)
            ".LBB0_2:                                ;   Parent Loop BB0_1 Depth=1\n"
            "                                        ; =>  This Inner Loop Header: Depth=2\n"
            "%s"
            "\tv_mfma_f32_32x32x16_f16 a[0:15], v[0:3], v[4:7], a[0:15]\n"
            "\ts_cbranch_scc1 .LBB0_2\n"
            "; %%bb.3:                                ;   in Loop: Header=BB0_1 Depth=1\n"
            "\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n"
            "\tscratch_store_dword off, v2, off\n"
            "\ts_cbranch_scc1 .LBB0_1\n"
            "; %%bb.4:\n"
            "\ts_endpgm\n")
    for inner, rc in (("", 0), ("\tscratch_load_dword v1, off, off\n", 1)):
        f = tmp_path / ("nested%d.s" % rc)
        f.write_text(text % inner)
        out = subprocess.run([sys.executable, CHECKER, str(f), "--allow-scratch-outside-loops", "Li8ELb1ELb0ELi8E"],
                             capture_output=True, text=True)
        assert out.returncode == rc, out.stdout
        assert out.stdout.count("inside an MFMA loop") == rc


def test_the_checker_counts_the_loads_behind_the_last_lds_dma_of_a_deep_step(tmp_path):
    body = ("_Z16gemm_mfma_kernelv:\n"
            "\tglobal_load_lds_dwordx4 v1, s[0:1]\n"
            "%s"
            "\tv_mfma_f32_32x32x16_f16 a[0:15], v[0:3], v[4:7], a[0:15]\n"
            "\ts_waitcnt vmcnt(3)\n"
            "\ts_barrier\n"
            "\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n"
            "\ts_endpgm\n")
    load = "\tglobal_load_dwordx4 v[8:11], v[20:21], off\n"
    for n_loads, rc in ((3, 0), (2, 1)):
        f = tmp_path / ("deep%d.s" % n_loads)
        f.write_text(body % (load * n_loads))
        out = subprocess.run([sys.executable, CHECKER, str(f)], capture_output=True, text=True)
        assert out.returncode == rc, out.stdout
        assert ("behind the last LDS-DMA" in out.stdout) == bool(rc)
    # x two steps ahead as well: the marked wait leaves a whole step's loads in flight, LDS-DMAs included
    step = ("\ts_barrier\n" + "\tglobal_load_lds_dwordx4 v1, s[0:1]\n" * 2 + "%s"
            "\t;;#ASMSTART\n\t; lowbit: this wait keeps the loads of one step in flight\n\t;;#ASMEND\n"
            "\ts_waitcnt vmcnt(4)\n\ts_barrier\n")
    for n_loads, rc in ((2, 0), (1, 1)):
        f = tmp_path / ("deep2_%d.s" % n_loads)
        f.write_text("_Z16gemm_mfma_kernelv:\n\tv_mfma_f32_32x32x16_f16 a[0:15], v[0:3], v[4:7], a[0:15]\n"
                     + step % (load * n_loads) + "\ts_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_endpgm\n")
        out = subprocess.run([sys.executable, CHECKER, str(f)], capture_output=True, text=True)
        assert out.returncode == rc, out.stdout
        assert ("since the barrier before it" in out.stdout) == bool(rc)
