"""The compiled kernels keep the wait states a matrix instruction's result needs, on every
path (no GPU: hipcc cross-compiles to assembly, which is read here)."""
from concurrent.futures import ThreadPoolExecutor

import pytest

import isa_scan

# the sequence hipcc once made of `if (dt * 16 < hd) { o *= alpha; o = mfma(v, p, o); }` in
# the wave-level attention with two row tiles (head size 16 takes the first branch): the
# accumulator a31 is copied back two instructions after the branch
OLD_SEQUENCE = """
_Z3oldv:
.LBB0_1:
	v_accvgpr_write_b32 a31, v65
	s_and_b64 vcc, exec, s[20:21]
	s_nop 0
	v_mfma_f32_16x16x32_bf16 a[28:31], v[2:5], v[66:69], a[28:31]
	s_cbranch_vccnz .LBB0_3
	v_mul_f32_e32 v62, v129, v58
	v_mul_f32_e32 v63, v129, v59
	v_mul_f32_e32 v64, v129, v60
	v_mul_f32_e32 v61, v129, v61
	v_accvgpr_write_b32 a20, v62
	v_accvgpr_write_b32 a21, v63
	v_accvgpr_write_b32 a22, v64
	v_accvgpr_write_b32 a23, v61
	s_nop 0
	v_mfma_f32_16x16x32_bf16 a[20:23], v[6:9], v[66:69], a[20:23]
.LBB0_3:
	v_accvgpr_read_b32 v69, a35
	v_accvgpr_read_b32 v193, a39
	v_accvgpr_read_b32 v65, a31
	s_nop 3
	v_accvgpr_read_b32 v61, a23
	s_endpgm
.Lfunc_end0:
"""


def test_the_reader_finds_the_sequence_that_gave_wrong_sums():
    kernels = isa_scan.kernels_of(OLD_SEQUENCE)
    assert list(kernels) == ["_Z3oldv"]
    bad = isa_scan.early_uses(kernels["_Z3oldv"])
    # only the taken path to a31: a23 is read 8 wait states after its instruction
    assert [(b[1], b[2]) for b in bad] == [("v_accvgpr_read_b32 v65, a31", 3)]


def test_the_reader_counts_nops_branches_and_accumulator_chains():
    text = """
_Z2okv:
	v_mfma_f32_16x16x32_bf16 a[0:3], v[2:5], v[6:9], a[0:3]
	v_mfma_f32_16x16x32_bf16 a[0:3], v[2:5], v[6:9], a[0:3]
	s_nop 5
	v_add_f32_e32 v1, v2, v3
	v_accvgpr_read_b32 v9, a3
	s_endpgm
.Lfunc_end0:
"""
    assert isa_scan.early_uses(isa_scan.kernels_of(text)["_Z2okv"]) == []
    early = text.replace("s_nop 5", "s_nop 4")
    assert len(isa_scan.early_uses(isa_scan.kernels_of(early)["_Z2okv"])) == 1


MODULES = ("attention_bf16", "gemm_bf16", "gemm_wide_bf16", "gemm_tiled_bf16", "ceilings")


@pytest.fixture(scope="module")
def assemblies():
    with ThreadPoolExecutor(len(MODULES)) as pool:
        return dict(zip(MODULES, pool.map(isa_scan.assembly_of, MODULES)))


@pytest.mark.parametrize("module", MODULES)
def test_no_kernel_uses_a_matrix_result_too_early(assemblies, module):
    kernels = isa_scan.kernels_of(assemblies[module])
    with_matrix = [k for k, items in kernels.items()
                   if any(kind == "ins" and isa_scan._is_matrix(t.split()[0]) for kind, t in items)]
    assert with_matrix, f"{module}: no kernel with matrix instructions was found in the assembly"
    bad = {k: isa_scan.early_uses(kernels[k]) for k in with_matrix}
    bad = {k: v for k, v in bad.items() if v}
    assert not bad, bad


def test_registers_of_hand_written_loads_wait_for_their_data(assemblies):
    """gemm_tiled_bf16 requests x by asm loads; nothing may touch their registers before the
    asm wait that names them.  The reader is checked on a sequence that does."""
    touched = """
tiled:
	;;#ASMSTART
	global_load_dwordx4 v[72:75], v[2:3], off
	;;#ASMEND
	v_cndmask_b32_e64 v75, 0, v75, s[4:5]
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	s_endpgm
"""
    found = isa_scan.loads_touched_before_their_wait(touched)
    assert len(found) == 1 and "v_cndmask" in found[0][2]
    assert isa_scan.loads_touched_before_their_wait(touched.replace("v75, 0, v75", "v80, 0, v81")) == []
    text = assemblies["gemm_tiled_bf16"]
    assert text.count("global_load_dwordx4") > text.count(" nt") > 0       # asm loads are there
    assert "#ASMSTART" in text
    assert isa_scan.loads_touched_before_their_wait(text) == []
