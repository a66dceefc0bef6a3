"""The build's guard on the kernels that keep loads under way in registers (noeira_amd/build.py): the parser of the
compiler's resource remarks names exactly the guarded kernels that use scratch memory, and the guarded names exist in
the source they are listed under."""
import os

from noeira_amd import build as B

REMARKS = """a.hip:1:1: remark: Function Name: _ZN2nq22gemv_tile4_rows_kernelILi0ELb1ELi3EEE [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     VGPRs: 128 [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     ScratchSize [bytes/lane]: 80 [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     VGPRs Spill: 42 [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark: Function Name: _ZN2nq20gemm_tile4_mt_kernelILi0EEE [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     ScratchSize [bytes/lane]: 16 [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark: Function Name: _ZN2nq22gemv_tile8_rows_kernelILb0ELi4EEE [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     SGPRs Spill: 3 [-Rpass-analysis=kernel-resource-usage]
a.hip:1:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
"""


def test_spilling_kernels_names_the_guarded_ones_only():
    names = ("gemv_tile4_rows_kernel", "gemv_tile8_rows_kernel")
    assert B._spilling_kernels(REMARKS, names) == ["_ZN2nq22gemv_tile4_rows_kernelILi0ELb1ELi3EEE"]
    assert B._spilling_kernels(REMARKS, ("gemm_tile4_mt_kernel",)) == ["_ZN2nq20gemm_tile4_mt_kernelILi0EEE"]
    assert B._spilling_kernels("", names) == []


def test_guarded_kernels_exist_where_they_are_listed():
    for src, names in B.NO_SPILL.items():
        text = open(os.path.join(B.CSRC, src)).read()
        for n in names:
            assert f"void {n}(" in text, (src, n)
            # each of them waits by hand for loads written in inline assembly
        assert 'asm volatile("global_load_' in text and 's_waitcnt vmcnt(' in text


ASM = """\t.text
_ZN2nq4goodEv: ; @_ZN2nq4goodEv
\tglobal_load_dword v7, v[2:3], off ; pf
\tglobal_load_ushort v9, v[4:5], off ; pf
\tv_add_u32_e32 v1, s2, v0
\tglobal_load_dwordx4 v[10:13], v[2:3], off
\ts_waitcnt vmcnt(0) ; pfw
\tv_mov_b32_e32 v20, v7
.Lfunc_end0:
_ZN2nq3badEv: ; @_ZN2nq3badEv
\tglobal_load_dword v7, v[2:3], off ; pf
\tv_mov_b32_e32 v20, v7
\tscratch_store_dwordx2 off, v[6:7], off
\ts_waitcnt vmcnt(0) ; pfw
.Lfunc_end1:
_ZN2nq4wideEv: ; @_ZN2nq4wideEv
\tglobal_load_dwordx4 v[8:11], v[2:3], off ; pf
\tv_add_f32_e32 v1, v10, v0
\ts_waitcnt vmcnt(0) ; pfw
.Lfunc_end3:
_ZN2nq6nowaitEv: ; @_ZN2nq6nowaitEv
\tglobal_load_dword v7, v[2:3], off ; pf
\ts_endpgm
.Lfunc_end2:
"""


def test_a_prefetched_register_named_before_its_wait_is_reported():
    early = B._early_uses_of_prefetched(ASM)
    assert [k for k, _ in early] == ["_ZN2nq3badEv", "_ZN2nq3badEv", "_ZN2nq4wideEv", "_ZN2nq6nowaitEv"]
    assert "v_mov_b32_e32 v20, v7" in early[0][1] and "scratch_store" in early[1][1]
    for src in B.PREFETCH_MARKED:
        text = open(os.path.join(B.CSRC, src)).read()
        assert "; pf\"" in text and "; pfw\"" in text, src


LOOP_ASM = """\t.text
_ZN2nq4loopEv: ; @_ZN2nq4loopEv
\tglobal_load_dwordx4 v[0:3], v[8:9], off nt ; pf
\ts_branch .LBB0_2
.LBB0_1:
\ts_waitcnt vmcnt(1)
\t; pfh v[4:7]
\tv_mfma_f32_16x16x32_bf16 a[0:3], v[4:7], v[10:13], a[0:3]
\tglobal_load_dwordx4 v[0:3], v[8:9], off nt ; pf
.LBB0_2:
\tglobal_load_dwordx4 v[4:7], v[8:9], off nt ; pf
{extra}
\ts_waitcnt vmcnt(1)
\t; pfh v[0:3]
\tv_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[10:13], a[0:3]
\ts_cbranch_vccnz .LBB0_1
\ts_waitcnt vmcnt(0)
\t; pfh v[4:7]
\ts_endpgm
.Lfunc_end0:
"""


def test_inflight_check_follows_the_loop_and_catches_copies_and_spills():
    """Two slots in turn across a back edge: the second slot's load stands later in the text than its hand-over.  A
    clean loop passes; a move or a spill that takes a register of a slot in flight is named; a move of a slot that was
    handed over is not."""
    assert B._inflight_violations(LOOP_ASM.format(extra="\tv_add_u32_e32 v20, v21, v22")) == []
    bad = B._inflight_violations(LOOP_ASM.format(extra="\tv_mov_b32_e32 v20, v1"))
    assert [t for _, t in bad] == ["v_mov_b32_e32 v20, v1"]
    bad = B._inflight_violations(LOOP_ASM.format(extra="\tscratch_store_dwordx2 off, v[6:7], off"))
    assert [t for _, t in bad] == ["scratch_store_dwordx2 off, v[6:7], off"]
    # after its hand-over a slot's registers are ordinary values again
    ok = LOOP_ASM.format(extra="").replace("\ts_endpgm", "\tv_mov_b32_e32 v30, v5\n\ts_endpgm")
    assert B._inflight_violations(ok) == []


def test_inflight_marks_exist_in_the_sources_that_are_checked():
    for src in B.INFLIGHT_MARKED:
        text = open(os.path.join(B.CSRC, src)).read()
        assert text.count("; pf\"") >= 3 and text.count("; pfh ") >= 3, src
