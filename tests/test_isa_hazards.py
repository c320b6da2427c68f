"""The compiled kernels must not read a scalar register in a memory instruction fewer than
5 wait states after a vector instruction wrote it (the compiler does not pad inline asm)."""

import shutil

import pytest


def test_scanner_flags_the_pattern_and_accepts_padding(ct):
    from causal_trainer_dev_amd import isa_hazards

    bad = """
kernel_a:
	v_readfirstlane_b32 s9, v5
	v_readfirstlane_b32 s8, v4
	global_store_dwordx2 v120, v[18:19], s[8:9] offset:0
"""
    assert len(isa_hazards.scan(bad)) == 1
    padded = bad.replace("\tglobal_store", "\ts_nop 4\n\tglobal_store")
    assert isa_hazards.scan(padded) == []
    scalar_alu = """
kernel_b:
	v_readfirstlane_b32 s0, v1
	s_ashr_i32 s1, s0, 31
	s_lshl_b64 s[0:1], s[0:1], 2
	s_add_u32 s0, s2, s0
	s_addc_u32 s1, s3, s1
	s_nop 0
	global_store_dwordx4 v252, v[2:5], s[0:1] offset:0
"""
    assert isa_hazards.scan(scalar_alu) == []
    two_short = """
kernel_c:
	v_readfirstlane_b32 s16, v4
	s_mov_b32 m0, s8
	s_nop 0
	global_load_lds_dwordx4 v52, s[16:17]
"""
    assert len(isa_hazards.scan(two_short)) == 1
    assert isa_hazards.scan("kernel_d:\n\tv_readfirstlane_b32 s16, v4\n\tglobal_load_dword v1, v[2:3], off\n") == []
    # a 16-byte store reads its data late: no vector write of the data registers for 2 wait states
    wide = """
kernel_e:
	global_store_dwordx4 v252, v[2:5], s[0:1] offset:0
	v_accvgpr_read_b32 v3, a17
"""
    assert len(isa_hazards.scan(wide)) == 1
    assert isa_hazards.scan(wide.replace("\tv_accvgpr", "\ts_nop 1\n\tv_accvgpr")) == []
    assert isa_hazards.scan(wide.replace("v3, a17", "v9, a17")) == []
    assert isa_hazards.scan(wide.replace("dwordx4 v252, v[2:5]", "dwordx2 v252, v[2:3]")) == []


def test_private_accumulator_check(ct):
    from causal_trainer_dev_amd import isa_hazards

    clean = """
_ZN2ct20attn_dkv_wide_kernelENS_10AttnParamsE:
	v_add_u32_e32 v1, v2, v3
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[0:15], v[4:7], v[8:11], a[0:15]
	;;#ASMEND
	s_endpgm
other_kernel:
	v_accvgpr_write_b32 a0, v1
"""
    assert isa_hazards.private_accumulators(clean, "attn_dkv_wide_kernel") == []
    parked = clean.replace("\tv_add_u32_e32 v1, v2, v3", "\tv_accvgpr_write_b32 a3, v1")
    assert len(isa_hazards.private_accumulators(parked, "attn_dkv_wide_kernel")) == 1
    spilled = clean.replace("\tv_add_u32_e32 v1, v2, v3", "\ts_barrier\n\tscratch_load_dword v1, off, off\n\ts_barrier")
    assert len(isa_hazards.private_accumulators(spilled, "attn_dkv_wide_kernel")) == 1
    outside = clean.replace("\tv_add_u32_e32 v1, v2, v3", "\ts_barrier\n\ts_barrier\n\tscratch_load_dword v1, off, off")
    assert isa_hazards.private_accumulators(outside, "attn_dkv_wide_kernel") == []
    assert len(isa_hazards.private_accumulators(clean, "missing_kernel")) == 1


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_library_sources_have_no_scalar_base_hazard(ct):
    from causal_trainer_dev_amd import isa_hazards

    findings = isa_hazards.scan_library()
    assert findings and all(not problems for problems in findings.values()), findings


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_steady_state_paths_keep_their_instruction_budget(ct):
    """Vector ALU instructions per MFMA on the paths an all-allowed key tile takes, read off the
    compiled head-dimension-128 kernels. What the arithmetic alone needs per score is fma + exp2 + add
    (+ half a max3 and half a bf16 packing) in the forward, fma, exp2, sub, mul (+ half a packing)
    in dQ, and mul, exp2, mul (+ a packing each for P and dS; the sums with the per-row terms come
    out of the matrix pipe) in dK/dV: 4.0, 3.0 and 2.0 per MFMA. The kernels with two
    wavefronts per SIMD add the rebuilding of their swizzled fragment addresses per tile (their 16
    pointers do not fit beside the accumulators), which is the rest. The bounds hold these paths
    where they are; masked tiles and the per-item prologue and epilogue come on top (measured
    averages over whole kernels at short packed segments: forward 6.7, dK/dV 4.6; at long
    segments: forward 4.7, dQ 4.4)."""

    from causal_trainer_dev_amd import build as recipe
    from causal_trainer_dev_amd import isa_hazards

    assembly = isa_hazards.device_assembly(recipe.CSRC / "ct_attn.hip", recipe.HIP_FLAGS)

    # forward: the step of a tile inside a stretch that needs no decisions is two blocks, the
    # statement with the first 8 MFMAs, the step's four copies and the maximum, then (the running
    # maximum did not move) the two statements with the other 24 MFMAs and the 32 exponentials
    forward = isa_hazards.block_mix(assembly, "attn_fwd_kernelILi128ELi4E")
    first_part = [b for b in forward if b["mfma"] == 8 and b["max3"] >= 15 and b["vmem"] == 4]
    second_part = [b for b in forward if b["mfma"] == 24 and b["exp"] == 32]
    assert first_part and second_part
    assert all(b["vmem"] == 0 for b in second_part)                 # no spill traffic on this path
    valu = max(b["valu"] for b in first_part) + max(b["valu"] for b in second_part)
    # (the general step's statements sit in blocks of the same shape with its decisions around
    # them: the leanest blocks are the stretch's; one s_waitcnt per MFMA, for its fragment read, is
    # part of the count)
    scalar = min(b["salu"] for b in first_part) + min(b["salu"] for b in second_part)
    assert valu / 32 <= 4.6, valu
    assert scalar / 32 <= 1.7, scalar

    # dQ and dK/dV: the blocks of the key-tile loop that hold the MFMA sequences also hold the
    # exponent / dS arithmetic of an all-allowed tile (masking sits in blocks of its own)
    def loop_ratio(kernel, mfmas_per_step, stores_per_block=0):
        blocks = [b for b in isa_hazards.block_mix(assembly, kernel) if b["mfma"]]
        assert blocks and sum(b["mfma"] for b in blocks) % mfmas_per_step == 0
        assert all(b["vmem"] <= stores_per_block for b in blocks)      # no spill traffic on these paths
        return (sum(b["valu"] for b in blocks) / sum(b["mfma"] for b in blocks),
                sum(b["salu"] for b in blocks) / sum(b["mfma"] for b in blocks))

    dq_valu, dq_salu = loop_ratio("attn_dq_kernelILi128ELi4E", 48)
    dkv_valu, dkv_salu = loop_ratio("attn_dkv_kernelILi128ELb0E", 32)
    stored_valu, _ = loop_ratio("attn_dkv_kernelILi128ELb1E", 32, stores_per_block=2)   # + the dS store
    assert dq_valu <= 4.0 and dkv_valu <= 4.1 and stored_valu <= 4.2, (dq_valu, dkv_valu, stored_valu)
    # scalar instructions of those blocks: bounds, branches, copy bookkeeping
    assert dq_salu <= 2.0 and dkv_salu <= 2.0, (dq_salu, dkv_salu)
