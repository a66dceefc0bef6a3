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
        assert 'asm volatile("global_load_dwordx4' in text and 's_waitcnt vmcnt(' in text
