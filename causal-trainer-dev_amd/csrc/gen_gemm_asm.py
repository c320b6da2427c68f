"""Generates ct_gemm_asm.inc: the hand-scheduled main loop of the 256 x 256 GEMM tile.

One wavefront runs on each SIMD, so whatever the wavefront issues between two MFMAs must fit
into the 32 cycles the matrix pipe is busy with the first of them, or the pipe drains. A
global -> LDS copy costs about 23 cycles to issue and an LDS fragment read 4 to 8; issued in
bursts (as the compiler schedules them) they stall the MFMA stream for hundreds of cycles per
k-step. The sequence below fixes the order: at most one copy or two fragment reads behind any
MFMA, nothing else.

Loop structure (operand A: m-contiguous tile read with transposed LDS reads, operand B:
k-contiguous tile read with ds_read_b128; ring of 4 LDS stages of 32 KB, stage = A tile then B
tile; the body is unrolled over the 4 stages so that every LDS offset is an immediate):

  step k, stage s = k % 4
    MFMA  0..15  use fragments f0 = (stage s, contraction 0..15), read during step k-1
    MFMA 16..31  use fragments f1 = (stage s, contraction 16..31), read behind MFMA 0..7
    copies of step k+3 -> stage (s+3) % 4 (read during step k-1, free since the barrier of
      that step): A tile behind MFMA 1, 5, 8, 10, B tile behind MFMA 19, 22, 25, 28
    behind MFMA 12: wait until this wavefront's copies of step k+1 have landed
      (vmcnt(12): step k+2 and the A half of step k+3 may stay in flight) and its reads of
      stage s have returned, barrier; then f0 of step k+1 is read behind MFMA 12..17, each
      read into registers whose last MFMA has been issued.
  Copies are issued for every step, including the last three whose data nobody reads: their
  source is clamped to the last valid step, which keeps the loop free of branches and the
  vmcnt arithmetic uniform.

Fixed registers (declared as clobbers): v[176:239] fragments, v[240:249] fragment addresses
+ 64 KB, s[40:41] / s[42:43] copy sources of A / B, s44 step counter, s45-s46 temporaries.

Run ``python gen_gemm_asm.py > ct_gemm_asm.inc`` after editing; the output is committed.
"""

STAGE = 32768
F0A, F0B, F1A, F1B, HI = 176, 192, 208, 224, 240
ACC = lambda i, j: "%%%d" % (4 * i + j)
PTR_A, PTR_B, STRIDE_A, STEPS, LDS_WAVE = "%16", "%17", "%18", "%19", "%20"
ADDR_A = lambda second, i: 21 + 4 * second + i
ADDR_B = lambda ks: 29 + ks
VOFF = lambda operand, n: "%%%d" % (31 + 4 * operand + n)


def addr(operand_index, stage, offset):
    """register and immediate of an LDS read at (address operand) + stage * STAGE + offset"""
    if stage < 2:
        return "%%%d" % operand_index, stage * STAGE + offset
    return "v%d" % (HI + operand_index - 21), (stage - 2) * STAGE + offset


def frag_reads(stage, ks):
    """the 12 reads of the fragments (stage, ks), keyed by the fragment they fill"""
    fa, fb = (F0A, F0B) if ks == 0 else (F1A, F1B)
    out = {}
    for i in range(4):
        reads = []
        for second in range(2):
            reg, imm = addr(ADDR_A(second, i), stage, ks * 8192)
            lo = fa + 4 * i + 2 * second
            reads.append("ds_read_b64_tr_b16 v[%d:%d], %s offset:%d" % (lo, lo + 1, reg, imm))
        out["a%d" % i] = reads
    for j in range(4):
        reg, imm = addr(ADDR_B(ks), stage, j * 2048)
        lo = fb + 4 * j
        out["b%d" % j] = ["ds_read_b128 v[%d:%d], %s offset:%d" % (lo, lo + 3, reg, imm)]
    return out


def mfma(m):
    ks, r = divmod(m, 16)
    i, j = divmod(r, 4)
    fa, fb = (F0A, F0B) if ks == 0 else (F1A, F1B)
    return "v_mfma_f32_32x32x16_bf16 %s, v[%d:%d], v[%d:%d], %s" % (
        ACC(i, j), fa + 4 * i, fa + 4 * i + 3, fb + 4 * j, fb + 4 * j + 3, ACC(i, j))


def copy(operand, n, stage):
    dst = stage * STAGE + operand * 16384 + n * 4096
    src = "s[40:41]" if operand == 0 else "s[42:43]"
    return ["s_add_u32 m0, %s, %d" % (LDS_WAVE, dst), "s_nop 0",
            "global_load_lds_dwordx4 %s, %s" % (VOFF(operand, n), src)]


ADVANCE = [
    "s_cmp_lt_u32 s44, " + STEPS,
    "s_cselect_b32 s45, %s, 0" % STRIDE_A,
    "s_cselect_b32 s46, 64, 0",
    "s_add_u32 s40, s40, s45",
    "s_addc_u32 s41, s41, 0",
    "s_add_u32 s42, s42, s46",
    "s_addc_u32 s43, s43, 0",
    "s_add_u32 s44, s44, 1",
]


def step(u):
    stage, nxt, dst = u, (u + 1) & 3, (u + 3) & 3
    f1 = frag_reads(stage, 1)
    f0n = frag_reads(nxt, 0)
    behind = {m: [] for m in range(32)}
    # f1 of this stage: all of its registers are free (their MFMAs belong to the last step)
    for m, keys in {0: ["a0"], 2: ["b0", "b1"], 3: ["b2", "b3"], 4: ["a1"], 6: ["a2"], 7: ["a3"]}.items():
        for key in keys:
            behind[m] += f1[key]
    for m, n in {1: 0, 5: 1, 8: 2, 10: 3}.items():
        behind[m] += copy(0, n, dst)
    behind[12] += ["s_waitcnt vmcnt(12)", "s_waitcnt lgkmcnt(0)", "s_barrier"]
    # f0 of the next step: a0..a2 are free after MFMA 11, b_j after MFMA 12 + j, a3 after MFMA 15
    for m, keys in {12: ["a0"], 13: ["a1"], 14: ["a2"], 15: ["b0", "b1"], 16: ["b2", "b3"], 17: ["a3"]}.items():
        for key in keys:
            behind[m] += f0n[key]
    for m, n in {19: 0, 22: 1, 25: 2, 28: 3}.items():
        behind[m] += copy(1, n, dst)
    behind[29] += ADVANCE
    lines = ["s_waitcnt lgkmcnt(0)"]
    for m in range(32):
        lines.append(mfma(m))
        lines += behind[m]
    return lines


def gemm_loop():
    lines = ["s_mov_b64 s[40:41], " + PTR_A, "s_mov_b64 s[42:43], " + PTR_B, "s_mov_b32 s44, 4"]
    for k in range(10):
        lines.append("v_add_u32 v%d, 0x10000, %%%d" % (HI + k, 21 + k))
    first = frag_reads(0, 0)
    for key in ["a0", "b0", "b1", "b2", "b3", "a1", "a2", "a3"]:
        lines += first[key]
    lines.append("ct_gemm_loop_%=:")
    for u in range(4):
        lines += step(u)
    lines += ["s_sub_u32 s45, s44, 4", "s_cmp_lt_u32 s45, " + STEPS, "s_cbranch_scc1 ct_gemm_loop_%="]
    # drain: nothing in flight, every wavefront done with the LDS tiles, MFMA results readable
    lines += ["s_waitcnt vmcnt(0)", "s_waitcnt lgkmcnt(0)", "s_barrier", "s_nop 15", "s_nop 7"]
    return lines


def emit(lines, name):
    body = " \\\n".join('  "%s\\n\\t"' % ln for ln in lines)
    return "#define %s \\\n%s\n" % (name, body)


def clobbers():
    regs = ["v%d" % r for r in range(F0A, HI + 10)] + ["s%d" % r for r in range(40, 47)]
    return ", ".join('"%s"' % r for r in regs)


if __name__ == "__main__":
    print("// Generated by gen_gemm_asm.py -- do not edit by hand.")
    print(emit(gemm_loop(), "CT_GEMM_LOOP"))
    print("#define CT_GEMM_LOOP_CLOBBERS %s" % clobbers())
