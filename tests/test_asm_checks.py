"""The build-time checks of the generated code of the list kernels (relax_amd/check_ring_asm.py), on small
hand-written listings: what they must accept and what they must refuse."""
from relax_amd import check_ring_asm as c

KERNEL = """
_ZN2wq4testEv:
\ts_load_dwordx2 s[0:1], s[4:5], 0x0
\t;;#ASMSTART
\tglobal_load_dwordx4 v[2:5], v6, s[0:1] nt
\t;;#ASMEND
{body}
\ts_endpgm
.Lfunc_end0:
"""


def _errors(body):
    return c.check(KERNEL.format(body=body))


def test_ring_registers_may_only_be_read_by_the_unpack_instructions():
    ok = "\t;;#ASMSTART\n\ts_waitcnt vmcnt(0)\n\t;;#ASMEND\n\t;;#ASMSTART\n\tv_and_or_b32 v7, v2, s2, v8\n\t;;#ASMEND\n\tv_add_u32_e32 v9, v7, v7"
    assert _errors(ok) == []
    assert _errors("\tv_mov_b32_e32 v9, v3") and "v_mov_b32_e32" in _errors("\tv_mov_b32_e32 v9, v3")[0]      # a copy
    assert _errors("\tscratch_store_dwordx4 off, v[2:5], off offset:16")                                            # a spill
    assert _errors("\tv_lshrrev_b32_e32 v9, 4, v2")                                                                 # another shift
    assert _errors("\tv_mov_b32_dpp v9, v2 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xf") == []                   # the lane exchange
    # a register the compiler reuses as a temporary after the slot was consumed is no longer a ring register
    assert _errors("\tv_mov_b32_e32 v2, 0\n\tv_add_u32_e32 v9, v2, v2") == []


def test_a_kernel_with_a_ring_must_not_spill_any_register():
    spill = "\tscratch_store_dword off, v40, off offset:84\n\tscratch_load_dword v40, off, off offset:84"
    errs = _errors(spill)
    assert errs and "scratch accesses" in errs[0]
    assert _errors("\tv_add_u32_e32 v40, v41, v42") == []


def test_a_file_without_ring_loads_is_refused():
    assert c.check("_ZN2wq4testEv:\n\tv_mov_b32_e32 v0, 0\n\ts_endpgm\n.Lfunc_end0:\n")


def _hazards(body):
    return c.check_asm_results(KERNEL.format(body=body))


def test_inline_assembly_results_must_not_reach_mfma_or_dpp_at_once():
    asm = "\t;;#ASMSTART\n\tv_pk_mul_f16 v10, v11, v12 op_sel_hi:[1,0]\n\t;;#ASMEND\n"
    mfma = "\tv_mfma_f32_16x16x32_f16 v[20:23], v[10:13], v[30:33], v[20:23]\n"
    filler = "\tv_add_u32_e32 v40, v41, v42\n"
    assert _hazards(asm + mfma)                                   # directly behind
    assert _hazards(asm + filler + mfma)                          # one instruction between
    assert _hazards(asm + filler + filler + filler + mfma) == []  # far enough
    assert _hazards("\tv_pk_mul_f16 v10, v11, v12\n" + mfma) == []  # the compiler's own instruction: its business
    # a statement that ends in its own s_nop is safe wherever it is placed
    own = "\t;;#ASMSTART\n\tv_mov_b32_dpp v10, v2 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t;;#ASMEND\n"
    dpp = "\tv_mov_b32_dpp v50, v10 row_ror:8 row_mask:0xf bank_mask:0xc\n"
    assert _hazards(own + dpp) == []
    bare = "\t;;#ASMSTART\n\tv_mov_b32_dpp v10, v2 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0xf\n\t;;#ASMEND\n"
    assert _hazards(bare + dpp)
    assert _hazards(bare + "\tv_mov_b32_dpp v10, v51 row_ror:8 row_mask:0xf bank_mask:0xc\n")  # the old value of a DPP destination counts
    # loads inside inline assembly are waited for by s_waitcnt, not by wait states
    assert _hazards("\t;;#ASMSTART\n\tglobal_load_dwordx4 v[10:13], v6, s[0:1] nt\n\t;;#ASMEND\n" + mfma) == []
