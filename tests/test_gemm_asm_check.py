"""The MFMA GEMM kernels keep their MFMAs in inline assembly, which hides from the compiler that accumulator
blocks are still in flight after them.  ipex-llm_amd/csrc/check_gemm_asm.py looks through the generated assembly
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
    # the 128-row DMA form is held to 128 vector registers, for two workgroups per compute unit, and spills a few
    out = subprocess.run([sys.executable, os.path.join(CSRC, "check_gemm_asm.py"), listing, "--allow-scratch", "Lb1ELi4E"],
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
    out = subprocess.run([sys.executable, os.path.join(CSRC, "check_gemm_asm.py"), str(bad)], capture_output=True, text=True)
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
    out = subprocess.run([sys.executable, os.path.join(CSRC, "check_gemm_asm.py"), str(bad)], capture_output=True, text=True)
    assert out.returncode == 1
    assert out.stdout.count("MFMA operand written by VALU") == 1 and "v9, v20, v21" in out.stdout
