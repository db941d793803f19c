"""The build-time assembly check (mamba2d_amd/asmcheck.py) on hand-written listings."""
from mamba2d_amd import asmcheck

HEAD = "_ZN1k3fooEv:\n"


def listing(*insts):
    return HEAD + "".join("\t" + i + "\n" for i in insts)


def test_clean_sequence_passes():
    n, bad = asmcheck.check_text(listing(
        "v_exp_f32_e32 v1, v1", "v_exp_f32_e32 v2, v2", "v_mul_f32_e32 v9, v7, v8",
        "v_fmac_f32_dpp v9, v4, v1 row_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1"))
    assert n == 1 and bad == []


def test_transcendental_result_used_in_the_next_slot_is_reported():
    n, bad = asmcheck.check_text(listing(
        "v_exp_f32_e32 v1, v1",
        "v_fmac_f32_dpp v9, v4, v1 row_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1"))
    assert n == 1 and len(bad) == 1 and bad[0][0] == "_ZN1k3fooEv"
    # one instruction (or an s_nop) in between is enough
    assert asmcheck.check_text(listing("v_exp_f32_e32 v1, v1", "s_nop 0",
                                       "v_fmac_f32_dpp v9, v4, v1 row_shr:1"))[1] == []


def test_shifted_source_written_within_two_slots_is_reported():
    dpp = "v_mul_f32_dpp v9, v4, v1 row_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1"
    assert len(asmcheck.check_text(listing("v_mov_b32_e32 v4, v3", dpp))[1]) == 1
    assert len(asmcheck.check_text(listing("v_mov_b32_e32 v4, v3", "v_add_f32_e32 v20, v21, v22", dpp))[1]) == 1
    assert asmcheck.check_text(listing("v_mov_b32_e32 v4, v3", "s_nop 1", dpp))[1] == []
    assert asmcheck.check_text(listing("v_mov_b32_e32 v4, v3", "v_add_f32_e32 v20, v21, v22",
                                       "v_add_f32_e32 v23, v21, v22", dpp))[1] == []
    # a register range that covers the source counts as a write
    assert len(asmcheck.check_text(listing("v_pk_mov_b32 v[4:5], v[6:7], v[6:7]", dpp))[1]) == 1
    # the other operands of the DPP instruction are ordinary reads
    assert asmcheck.check_text(listing("v_mov_b32_e32 v1, v3", dpp))[1] == []


def test_histories_do_not_cross_kernels():
    text = listing("v_exp_f32_e32 v1, v1") + "_ZN1k3barEv:\n\tv_fmac_f32_dpp v9, v4, v1 row_shr:1\n"
    assert asmcheck.check_text(text)[1] == []


def test_kernels_that_ask_for_scratch_memory_are_listed():
    text = ("\t.amdhsa_kernel _ZN1k3fooEv\n\t\t.amdhsa_private_segment_fixed_size 0\n\t.end_amdhsa_kernel\n"
            "\t.amdhsa_kernel _ZN1k3barEv\n\t\t.amdhsa_private_segment_fixed_size 932\n\t.end_amdhsa_kernel\n")
    assert asmcheck.spilling_kernels(text) == [("_ZN1k3barEv", 932)]
