"""Generates ct_attn_asm.inc: hand-scheduled MFMA sequences of the attention kernels (D = 128).

The compiler's scheduler places every LDS fragment read directly in front of the MFMA that
consumes it once register pressure is high, so each MFMA pays the full LDS latency. These
sequences pin the order instead: fragment reads run AHEAD fragments in front of their MFMA,
into fixed scratch registers v[240:255] (declared as clobbers), and s_waitcnt lgkmcnt(n) is
exact because nothing else of the wavefront is counted by lgkmcnt while a sequence runs (each
starts with lgkmcnt(0)).

Run ``python gen_attn_asm.py > ct_attn_asm.inc`` after editing; the output is committed.
"""

SCRATCH0 = 240
# The compiler cannot see the MFMAs inside an asm statement, so it will not insert the wait
# states that a vector ALU read of a fresh MFMA result needs; the sequences end with them.
TAIL = ["s_nop 15", "s_nop 7"]
# dK/dV: the wavefront drops to issue priority 0 for a sequence and returns to 1 after it, so
# that the other wavefront of the SIMD, when it is in its exponent / dS arithmetic, issues
# first: an MFMA sequence issues one instruction every 32 cycles and loses nothing by waiting a
# few, while the arithmetic phase is issue-bound (measured: dK/dV kernel 3 % faster; the same
# in the forward sequences, or with the levels swapped, is slower or neutral).
DKV_HEAD = ["s_waitcnt lgkmcnt(0)", "s_setprio 0"]
DKV_TAIL = ["s_setprio 1"] + TAIL


def slot_regs(slot):
    lo = SCRATCH0 + 4 * slot
    return lo, lo + 3


def emit(lines, name):
    body = "\n".join('  "%s\\n\\t"' % ln for ln in lines)
    return "#define %s \\\n%s\n" % (name, body.replace("\n", " \\\n"))


def pv_sequence(ahead, slots):
    """O^T[db] += V^T frag(step, db) * P^T[step]: 16 MFMAs, each fragment = 2 ds_read_b64_tr_b16.

    operands: %0-%3 accumulators, %4-%7 lo pointers (column block db), %8-%11 hi pointers,
    %12-%15 probability fragments (k-step), %16 byte offset of the V tile.
    """
    n = 16
    lines = ["s_waitcnt lgkmcnt(0)"]

    def load(i):
        step, db = divmod(i, 4)
        lo, _ = slot_regs(i % slots)
        off = "%%16+%d" % (step * 4096)
        return ["ds_read_b64_tr_b16 v[%d:%d], %%%d offset:%s" % (lo, lo + 1, 4 + db, off),
                "ds_read_b64_tr_b16 v[%d:%d], %%%d offset:%s" % (lo + 2, lo + 3, 8 + db, off)]

    for i in range(min(ahead, n)):
        lines += load(i)
    for i in range(n):
        later = min(ahead - 1, n - 1 - i)
        lines.append("s_waitcnt lgkmcnt(%d)" % (2 * later))
        step, db = divmod(i, 4)
        lo, hi = slot_regs(i % slots)
        lines.append("v_mfma_f32_32x32x16_bf16 %%%d, v[%d:%d], %%%d, %%%d" % (db, lo, hi, 12 + step, db))
        if i + ahead < n:
            lines += load(i + ahead)
    return lines + TAIL


def qk_sequence(ahead, slots):
    """S^T[kb] = K frag(kb, ks) * Q^T[ks]: 16 MFMAs, each fragment = 1 ds_read_b128.

    operands: %0-%1 score accumulators (written), %2-%9 fragment pointers (k-step ks),
    %10-%17 query fragments (k-step), %18 byte offset of the K tile.
    """
    n = 16
    lines = ["s_waitcnt lgkmcnt(0)"]

    def load(i):
        ks, kb = divmod(i, 2)
        lo, hi = slot_regs(i % slots)
        return ["ds_read_b128 v[%d:%d], %%%d offset:%%18+%d" % (lo, hi, 2 + ks, kb * 8192)]

    for i in range(min(ahead, n)):
        lines += load(i)
    for i in range(n):
        later = min(ahead - 1, n - 1 - i)
        lines.append("s_waitcnt lgkmcnt(%d)" % later)
        ks, kb = divmod(i, 2)
        lo, hi = slot_regs(i % slots)
        src_c = "0" if ks == 0 else "%%%d" % kb
        lines.append("v_mfma_f32_32x32x16_bf16 %%%d, v[%d:%d], %%%d, %s" % (kb, lo, hi, 10 + ks, src_c))
        if i + ahead < n:
            lines += load(i + ahead)
    return lines + TAIL


DKV_SLOTS = 5
DKV_SCRATCH0 = 256 - 4 * DKV_SLOTS - 1  # one address temporary, then the fragment slots


def dkv_slot(slot):
    lo = DKV_SCRATCH0 + 1 + 4 * slot
    return lo, lo + 3


def dkv_sdp_sequence():
    """S = Q K^T and dP = dO V^T of one (32 query rows x 32 keys) block, interleaved: per k-step
    one MFMA of each chain. The fragment reads (Q, dO, V per k-step) run through a ring of
    DKV_SLOTS registers quads: a read is issued as soon as the MFMA that used its slot has been
    issued, so reads stay DKV_SLOTS fragments in front of their MFMAs.

    operands: %0 S, %1 dP (written), %2-%9 row-fragment pointers (k-step), %10-%17 K fragments
    (registers), %18 byte offset of this wavefront's V rows (scalar), %19 byte offset of the
    stage (Q tile; the dO tile follows 8192 bytes later).
    """
    steps = 8
    total = 3 * steps  # read r = 3 ks + which; which: 0 Q, 1 dO, 2 V
    lines = list(DKV_HEAD)
    state = {"issued": 0}

    def load_next():
        r = state["issued"]
        if r >= total:
            return []
        state["issued"] += 1
        ks, which = divmod(r, 3)
        lo, hi = dkv_slot(r % DKV_SLOTS)
        if which == 2:
            return ["v_add_u32_e32 v%d, %%18, %%%d" % (DKV_SCRATCH0, 2 + ks),
                    "ds_read_b128 v[%d:%d], v%d" % (lo, hi, DKV_SCRATCH0)]
        return ["ds_read_b128 v[%d:%d], %%%d offset:%%19+%d" % (lo, hi, 2 + ks, which * 8192)]

    for _ in range(DKV_SLOTS):
        lines += load_next()
    for ks in range(steps):
        q_slot = dkv_slot((3 * ks) % DKV_SLOTS)
        do_slot = dkv_slot((3 * ks + 1) % DKV_SLOTS)
        v_slot = dkv_slot((3 * ks + 2) % DKV_SLOTS)
        lines.append("s_waitcnt lgkmcnt(%d)" % (state["issued"] - (3 * ks + 1)))
        lines.append("v_mfma_f32_32x32x16_bf16 %%0, v[%d:%d], %%%d, %s" % (q_slot[0], q_slot[1], 10 + ks,
                                                                        "0" if ks == 0 else "%0"))
        lines += load_next()
        lines.append("s_waitcnt lgkmcnt(%d)" % (state["issued"] - (3 * ks + 3)))
        lines.append("v_mfma_f32_32x32x16_bf16 %%1, v[%d:%d], v[%d:%d], %s" % (do_slot[0], do_slot[1], v_slot[0],
                                                                              v_slot[1], "0" if ks == 0 else "%1"))
        lines += load_next()
        lines += load_next()
    return lines + DKV_TAIL


def dkv_acc_sequence(ahead=DKV_SLOTS, slots=DKV_SLOTS):
    """dV[db] += P^T[step] dO(step, db) and dK[db] += dS^T[step] Q(step, db), interleaved: 16
    MFMAs, each with one transposed fragment (2 ds_read_b64_tr_b16) read `ahead` fragments in
    front of it.

    operands: %0-%3 dV accumulators, %4-%7 dK accumulators, %8-%11 lo pointers (column block db),
    %12-%15 hi pointers, %16-%17 P^T (k-step), %18-%19 dS^T (k-step), %20 byte offset of the
    stage (Q tile; the dO tile follows 8192 bytes later).
    """
    order = [(step, db, which) for step in range(2) for db in range(4) for which in range(2)]  # which: 0 dV, 1 dK
    n = len(order)
    lines = list(DKV_HEAD)

    def load(i):
        step, db, which = order[i]
        lo, _ = dkv_slot(i % slots)
        off = "%%20+%d" % (step * 4096 + (8192 if which == 0 else 0))
        return ["ds_read_b64_tr_b16 v[%d:%d], %%%d offset:%s" % (lo, lo + 1, 8 + db, off),
                "ds_read_b64_tr_b16 v[%d:%d], %%%d offset:%s" % (lo + 2, lo + 3, 12 + db, off)]

    for i in range(min(ahead, n)):
        lines += load(i)
    for i in range(n):
        later = min(ahead - 1, n - 1 - i)
        lines.append("s_waitcnt lgkmcnt(%d)" % (2 * later))
        step, db, which = order[i]
        lo, hi = dkv_slot(i % slots)
        acc = db if which == 0 else 4 + db
        aop = (16 if which == 0 else 18) + step
        lines.append("v_mfma_f32_32x32x16_bf16 %%%d, %%%d, v[%d:%d], %%%d" % (acc, aop, lo, hi, acc))
        if i + ahead < n:
            lines += load(i + ahead)
    return lines + DKV_TAIL


# (Dropping the issue priority for these sequences, as the dK/dV ones do, measured neutral here.)
DQ_HEAD = ["s_waitcnt lgkmcnt(0)"]
DQ_TAIL = TAIL


def dq_sdp_half_sequence(ahead=4, slots=4):
    """dQ kernel, one 32-key half of a key tile: S^T = K_half Q^T and dP^T = V_half dO^T, the two
    chains alternating (16 MFMAs, one ds_read_b128 fragment each, read `ahead` fragments in front).

    operands: %0 S^T, %1 dP^T (written), %2-%9 row-fragment pointers (k-step), %10-%17 Q fragments,
    %18-%25 dO fragments, %26 byte offset of the half's K rows, %27 that of its V rows.
    """
    n = 16
    lines = list(DQ_HEAD)

    def load(i):
        ks, which = divmod(i, 2)
        lo, hi = slot_regs(i % slots)
        return ["ds_read_b128 v[%d:%d], %%%d offset:%%%d" % (lo, hi, 2 + ks, 26 + which)]

    for i in range(min(ahead, n)):
        lines += load(i)
    for i in range(n):
        later = min(ahead - 1, n - 1 - i)
        lines.append("s_waitcnt lgkmcnt(%d)" % later)
        ks, which = divmod(i, 2)
        lo, hi = slot_regs(i % slots)
        src_c = "0" if ks == 0 else "%%%d" % which
        lines.append("v_mfma_f32_32x32x16_bf16 %%%d, v[%d:%d], %%%d, %s" % (which, lo, hi, (18 if which else 10) + ks, src_c))
        if i + ahead < n:
            lines += load(i + ahead)
    return lines + DQ_TAIL


def dq_acc_half_sequence(ahead=4, slots=4):
    """dQ kernel, one 32-key half: dQ^T[db] += K_half^T frag(step, db) * dS^T[step], 8 MFMAs, each
    fragment = 2 ds_read_b64_tr_b16.

    operands: %0-%3 accumulators, %4-%7 lo pointers (column block db), %8-%11 hi pointers,
    %12-%13 dS fragments (k-step), %14 byte offset of the half's K rows.
    """
    n = 8
    lines = list(DQ_HEAD)

    def load(i):
        step, db = divmod(i, 4)
        lo, _ = slot_regs(i % slots)
        off = "%%14+%d" % (step * 4096)
        return ["ds_read_b64_tr_b16 v[%d:%d], %%%d offset:%s" % (lo, lo + 1, 4 + db, off),
                "ds_read_b64_tr_b16 v[%d:%d], %%%d offset:%s" % (lo + 2, lo + 3, 8 + db, off)]

    for i in range(min(ahead, n)):
        lines += load(i)
    for i in range(n):
        later = min(ahead - 1, n - 1 - i)
        lines.append("s_waitcnt lgkmcnt(%d)" % (2 * later))
        step, db = divmod(i, 4)
        lo, hi = slot_regs(i % slots)
        lines.append("v_mfma_f32_32x32x16_bf16 %%%d, v[%d:%d], %%%d, %%%d" % (db, lo, hi, 12 + step, db))
        if i + ahead < n:
            lines += load(i + ahead)
    return lines + DQ_TAIL


def clobbers():
    regs = ", ".join('"v%d"' % r for r in range(SCRATCH0, SCRATCH0 + 16))
    dkv = ", ".join('"v%d"' % r for r in range(DKV_SCRATCH0, 256))
    return "#define CT_ATTN_ASM_SCRATCH %s\n\n#define CT_DKV_ASM_SCRATCH %s\n" % (regs, dkv)


if __name__ == "__main__":
    print("// Generated by gen_attn_asm.py -- do not edit by hand.")
    print(emit(pv_sequence(4, 4), "CT_ATTN_PV_SEQUENCE"))
    print(emit(qk_sequence(4, 4), "CT_ATTN_QK_SEQUENCE"))
    print(emit(dq_sdp_half_sequence(), "CT_DQ_SDP_HALF_SEQUENCE"))
    print(emit(dq_acc_half_sequence(), "CT_DQ_ACC_HALF_SEQUENCE"))
    print(emit(dkv_sdp_sequence(), "CT_DKV_SDP_SEQUENCE"))
    print(emit(dkv_acc_sequence(), "CT_DKV_ACC_SEQUENCE"))
    print(clobbers())
