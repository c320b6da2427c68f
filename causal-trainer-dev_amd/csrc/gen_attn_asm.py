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


# ---------------------------------------------------------------------------
# Forward, interleaved form. A wavefront that runs its softmax arithmetic and its MFMAs in
# separate stretches leaves the matrix pipe idle during the first and the vector ALU idle during
# the second; the other wavefront of the SIMD fills only part of that. Here the arithmetic of key
# tile t sits between the MFMAs of O += V(t-1)^T P(t-1)^T and S(t+1)^T = K(t+1) Q^T of the same
# wavefront: about five vector instructions fit behind an MFMA without delaying the next one.
#
# The scores live in two buffers of 32 registers that only these statements name, v[176:207] ("a")
# and v[208:239] ("b"); the compiler is kept out of v[176:255] (clobbers on every statement, and a
# static check of the compiled kernel). The scores of tile t are in buffer a when t counts even
# from the first tile of the query tile, else in b; S(t+1) is written to the other buffer while
# the exponentials of tile t are taken in place. The bf16 pairs of P(t) go into the first 16
# registers of the buffer they came from (pair p reads scores 2p, 2p+1 and writes register p, which
# an earlier pair has already read), where the PV product of the next step finds them; by the time
# S(t+2) is written over them that product has been issued.
#
# Per key tile, when the tile before and the tile after are there too (FWD_* statements):
#   max:   first half of the PV product (k-steps 0, 1)   | maximum of S(t)
#   exp_a: second half of the PV product (k-steps 2, 3)  | exponentials of scores 0..FWD_SPLIT-1
#   exp_b: S(t+1)                                        | exponentials of the other scores
# (an asm statement takes at most 30 operands, and the decision to move the running maximum sits
# between the first two). Otherwise the same arithmetic and the same products as statements of
# their own (FWD_*_ONLY, FWD_QK, FWD_PV, FWD_PV_LATE), which give the same bits.
# ---------------------------------------------------------------------------
FWD_S = {"a": 112, "b": 144}
FWD_FIRST_PRIVATE = 112
FWD_RING0 = 176          # four fragment slots of four registers
FWD_LAST_PRIVATE = 191
FWD_SPLIT = 10


def other(cur):
    return "b" if cur == "a" else "a"


def fwd_slot(slot):
    lo = FWD_RING0 + 4 * slot
    return lo, lo + 3


def fwd_acc(db):
    return "a[%d:%d]" % (16 * db, 16 * db + 15)


def weave(groups, valu, lead=0):
    """MFMA groups (wait, MFMA, the fragment reads behind it) with the vector instructions spread
    evenly behind them; `lead` of them go in front of the first group, under the first reads."""
    out = list(valu[:lead])
    rest = valu[lead:]
    pos = 0
    for gi, group in enumerate(groups):
        out += group
        want = (len(rest) * (gi + 1)) // len(groups)
        out += rest[pos:want]
        pos = want
    return out


def fwd_pf(cur, step):
    """P^T fragment of k-step `step` of the tile before the one in buffer `cur`."""
    lo = FWD_S[other(cur)] + 4 * step
    return "v[%d:%d]" % (lo, lo + 3)


def fwd_pv_groups(cur, steps):
    """MFMA groups of O^T[db] += V^T frag(step, db) * P^T[step] for the given k-steps; returns
    (head reads, groups). Operands by name: lo0-3, hi0-3, voff."""
    order = [(step, db) for step in steps for db in range(4)]
    n, ahead, slots = len(order), 4, 4

    def load(i):
        step, db = order[i]
        lo, _ = fwd_slot(i % slots)
        o = "%%[voff]+%d" % (step * 4096)
        return ["ds_read_b64_tr_b16 v[%d:%d], %%[lo%d] offset:%s" % (lo, lo + 1, db, o),
                "ds_read_b64_tr_b16 v[%d:%d], %%[hi%d] offset:%s" % (lo + 2, lo + 3, db, o)]

    head = ["s_waitcnt lgkmcnt(0)"]
    for i in range(min(ahead, n)):
        head += load(i)
    groups = []
    for i in range(n):
        later = min(ahead - 1, n - 1 - i)
        step, db = order[i]
        lo, hi = fwd_slot(i % slots)
        g = ["s_waitcnt lgkmcnt(%d)" % (2 * later),
             "v_mfma_f32_32x32x16_bf16 %s, v[%d:%d], %s, %s" % (fwd_acc(db), lo, hi, fwd_pf(cur, step), fwd_acc(db))]
        if i + ahead < n:
            g += load(i + ahead)
        groups.append(g)
    return head, groups


def fwd_qk_groups(cur):
    """MFMA groups of S(t+1)^T = K Q^T into the buffer other than `cur`. Operands by name: rp0-7
    fragment pointers (k-step), q0-7 query fragments, koff."""
    nxt = FWD_S[other(cur)]
    n, ahead, slots = 16, 4, 4

    def load(i):
        ks, kb = divmod(i, 2)
        lo, hi = fwd_slot(i % slots)
        return ["ds_read_b128 v[%d:%d], %%[rp%d] offset:%%[koff]+%d" % (lo, hi, ks, kb * 8192)]

    head = ["s_waitcnt lgkmcnt(0)"]
    for i in range(ahead):
        head += load(i)
    groups = []
    for i in range(n):
        later = min(ahead - 1, n - 1 - i)
        ks, kb = divmod(i, 2)
        lo, hi = fwd_slot(i % slots)
        dst = "v[%d:%d]" % (nxt + 16 * kb, nxt + 16 * kb + 15)
        g = ["s_waitcnt lgkmcnt(%d)" % later,
             "v_mfma_f32_32x32x16_bf16 %s, v[%d:%d], %%[q%d], %s" % (dst, lo, hi, ks, "0" if ks == 0 else dst)]
        if i + ahead < n:
            g += load(i + ahead)
        groups.append(g)
    return head, groups


def fwd_exp_ops(cur, lo, hi):
    """P = exp2(S c - m) in place for scores lo..hi-1 of buffer `cur` (lo, hi even), the running
    sum in score order, and the bf16 pairs; ordered so that nothing reads the result of the
    transcendental instruction directly in front of it. Operands: %[m] the reference, %[psum] the
    sum, %[c] log2 e (scalar)."""
    s0 = FWD_S[cur]
    ops = []
    for k in range(lo, hi + 2):
        if k < hi:
            ops.append("v_fma_f32 v%d, v%d, %%[c], -%%[m]" % (s0 + k, s0 + k))
        if lo <= k - 1 < hi:
            ops.append("v_exp_f32_e32 v%d, v%d" % (s0 + k - 1, s0 + k - 1))
        if lo <= k - 2 < hi:
            i = k - 2
            ops.append("v_add_f32_e32 %%[psum], %%[psum], v%d" % (s0 + i))
            if i % 2 == 1:
                ops.append("v_cvt_pk_bf16_f32 v%d, v%d, v%d" % (s0 + i // 2, s0 + i - 1, s0 + i))
    return ops


def fwd_max_ops(cur):
    """%[mx] = log2 e times the maximum of the lane pair's scores in buffer `cur`; %[tmp] scratch."""
    s0 = FWD_S[cur]
    ops = ["v_max3_f32 %%[mx], v%d, v%d, v%d" % (s0, s0 + 1, s0 + 2)]
    for j in range(3, 31, 2):
        ops.append("v_max3_f32 %%[mx], %%[mx], v%d, v%d" % (s0 + j, s0 + j + 1))
    ops.append("v_max_f32_e32 %%[mx], %%[mx], v%d" % (s0 + 31))
    ops += ["v_mov_b32_e32 %[tmp], %[mx]", "s_nop 1", "v_permlane32_swap_b32 %[mx], %[tmp]",
            "v_max_f32_e32 %[mx], %[mx], %[tmp]", "v_mul_f32_e32 %[mx], %[c], %[mx]"]
    return ops


def flatten(head, groups):
    return head + [ln for g in groups for ln in g]


def fwd_statements(cur):
    head_pv01, pv01 = fwd_pv_groups(cur, (0, 1))
    head_pv23, pv23 = fwd_pv_groups(cur, (2, 3))
    head_pv, pv = fwd_pv_groups(cur, (0, 1, 2, 3))
    head_qk, qk = fwd_qk_groups(cur)
    key_offset = lambda i: 32 * (i // 16) + 8 * ((i % 16) // 4) + (i % 16) % 4
    s0 = FWD_S[cur]
    causal = []
    for i in range(32):
        causal += ["v_cmp_le_i32_e32 vcc, %d, %%[rel]" % key_offset(i),
                   "v_cndmask_b32_e32 v%d, %%[ninf], v%d, vcc" % (s0 + i, s0 + i)]
    # ids: the tile's 64 key ids sit in LDS in key order; %[idp] is this lane's address of key
    # 4 * (lane / 32), so the quad of registers 4 q .. 4 q + 3 of block kb is the 16 bytes at
    # offset 4 * (32 kb + 8 q). Quads go through the fragment ring (four in flight).
    ids = ["s_waitcnt lgkmcnt(0)"]
    quad_regs = lambda q: FWD_RING0 + 4 * (q % 4)
    quad_read = lambda q: "ds_read_b128 v[%d:%d], %%[idp] offset:%d" % (
        quad_regs(q), quad_regs(q) + 3, 4 * (32 * (q // 4) + 8 * (q % 4)))
    ids += [quad_read(q) for q in range(4)]
    for q in range(8):
        ids.append("s_waitcnt lgkmcnt(%d)" % min(3, 7 - q))
        for e in range(4):
            i = 4 * q + e
            ids += ["v_cmp_eq_u32_e32 vcc, %%[segq], v%d" % (quad_regs(q) + e),
                    "v_cndmask_b32_e32 v%d, %%[ninf], v%d, vcc" % (s0 + i, s0 + i)]
        if q + 4 < 8:
            ids.append(quad_read(q + 4))
    return {
        # the three interleaved statements
        "MAX": head_pv01 + weave(fwd_with_copies(pv01, 2), fwd_max_ops(cur)),
        "EXP_A": head_pv23 + weave(pv23, fwd_exp_ops(cur, 0, FWD_SPLIT)),
        "EXP_B": head_qk + weave(qk, fwd_exp_ops(cur, FWD_SPLIT, 32), lead=6) + TAIL,
        # the same pieces on their own
        "MAX_ONLY": fwd_max_ops(cur),
        "EXP_ONLY": fwd_exp_ops(cur, 0, 32),
        "PV": flatten(head_pv, pv) + TAIL,
        "PV_LATE": flatten(head_pv23, pv23) + TAIL,
        "QK": flatten(head_qk, qk) + TAIL,
        # the first scores of a query tile, with the clearing of the output accumulator behind the MFMAs
        "QK_ZERO": head_qk + weave(qk, fwd_accumulator_statements()["ZERO"]) + TAIL,
        # masks: scores of pairs that are not allowed become -inf. CAUSAL: allowed = key offset in the
        # tile <= %[rel] (per lane)
        "MASK_CAUSAL": causal,
        # IDS: the key's id (read here from the id ring in LDS) differs from %[segq] (per lane)
        "MASK_IDS": ids,
    }


def fwd_with_copies(groups, passes):
    """The step's global -> LDS copies of this wavefront (V rows of this tile, then K rows of the
    tile after next: `passes` pieces of 1 KB each) placed behind the MFMAs: their issue then costs
    the matrix pipe nothing. Copy g: m0 = %[d<g>] (LDS destination, scalar), source = scalar base
    %[vsrc] (g < passes) or %[ksrc] plus the lane's byte offset %[off<g % passes>]. m0 is set one
    MFMA ahead of its copy; the last copy closes the statement."""
    out = [list(g) for g in groups]
    n = 2 * passes
    assert n <= len(groups)
    for g in range(n):
        load = "global_load_lds_dwordx4 %%[off%d], %%[%s]" % (g % passes, "vsrc" if g < passes else "ksrc")
        out[g].append("s_mov_b32 m0, %%[d%d]" % g)
        if g + 1 < len(groups):
            out[g + 1] = out[g + 1][:2] + [load] + out[g + 1][2:]
        else:
            out.append([load])
    return out


def fwd_accumulator_statements():
    """The output accumulator O^T (128 x 32 queries) lives in a[0:63], which only these statements
    and the PV products name. ZERO; SCALE: every element times %[alpha] (per lane: the row's
    factor), eight elements in flight through the fragment ring; the read-out uses CT_DKVW_READ."""
    zero = ["v_accvgpr_write_b32 a%d, 0" % r for r in range(64)]
    scale = []
    ring = list(range(FWD_RING0, FWD_RING0 + 8))
    for base in range(0, 64, 8):
        scale += ["v_accvgpr_read_b32 v%d, a%d" % (ring[e], base + e) for e in range(8)]
        scale += ["v_mul_f32_e32 v%d, %%[alpha], v%d" % (ring[e], ring[e]) for e in range(8)]
        scale += ["v_accvgpr_write_b32 a%d, v%d" % (base + e, ring[e]) for e in range(8)]
    return {"ZERO": zero, "SCALE": scale + ["s_nop 1"]}


def fwd_private_clobbers():
    return ", ".join(['"v%d"' % r for r in range(FWD_FIRST_PRIVATE, FWD_LAST_PRIVATE + 1)] +
                     ['"a%d"' % r for r in range(64)])


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

    operands: %0 S, %1 dP (read and written: the chains start from what the caller put there, the
    per-row terms -lse / scale and -delta), %2-%9 row-fragment pointers (k-step), %10-%17 K
    fragments (registers), %18 byte offset of this wavefront's V rows (scalar), %19 byte offset of
    the stage (Q tile; the dO tile follows 8192 bytes later).
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
        lines.append("v_mfma_f32_32x32x16_bf16 %%0, v[%d:%d], %%%d, %%0" % (q_slot[0], q_slot[1], 10 + ks))
        lines += load_next()
        lines.append("s_waitcnt lgkmcnt(%d)" % (state["issued"] - (3 * ks + 3)))
        lines.append("v_mfma_f32_32x32x16_bf16 %%1, v[%d:%d], v[%d:%d], %%1" % (do_slot[0], do_slot[1], v_slot[0],
                                                                               v_slot[1]))
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


# ---------------------------------------------------------------------------
# dK/dV, wide form: one wavefront per SIMD owns 64 keys (two 32-key blocks) and runs a whole
# (head, query block) step as one instruction stream. With nothing else resident on the SIMD the
# wavefront's exponent / dS arithmetic has to sit between its own MFMAs: the arithmetic of key
# block 0 is placed under the S / dP MFMAs of key block 1, that of key block 1 under the dV / dK
# MFMAs of key block 0.
#
# Fixed registers (declared as clobbers): a ring of 5 fragment slots, the score / dP blocks of
# both key blocks (their first 8 registers later hold the bf16 P and dS fragments) and the 16
# lse2 / delta values of this lane's query rows.
# ---------------------------------------------------------------------------
W_SLOTS = 5
W_RING0 = 256 - 4 * W_SLOTS
W_S = (W_RING0 - 64, W_RING0 - 32)      # S^T accumulators of key block 0 / 1 (16 registers each)
W_DP = (W_RING0 - 48, W_RING0 - 16)     # dP accumulators
W_ADDR = W_RING0 - 65                   # address of a V fragment
W_FIRST = W_ADDR


class Stream:
    """Instruction list with in-order tracking of the LDS reads in flight (lgkmcnt)."""

    def __init__(self):
        self.lines = ["s_waitcnt lgkmcnt(0)"]
        self.pending = []

    def lds(self, text, tag):
        self.lines.append(text)
        self.pending.append(tag)
        assert len(self.pending) <= 15, "lgkmcnt holds at most 15"

    def wait(self, tag):
        if tag not in self.pending:
            return
        i = len(self.pending) - 1 - self.pending[::-1].index(tag)
        self.lines.append("s_waitcnt lgkmcnt(%d)" % (len(self.pending) - 1 - i))
        self.pending = self.pending[i + 1:]

    def emit(self, text):
        self.lines.append(text)


def w_acc(i):
    """Accumulator i of the wide kernel: 0-3 dV of key block 0 (column block db), 4-7 dV of key
    block 1, 8-11 dK of key block 0, 12-15 dK of key block 1. They live in fixed accumulation
    registers for the whole kernel and are never handed to the compiler."""
    return "a[%d:%d]" % (16 * i, 16 * i + 15)


class WideOperands:
    """Names of the asm operands of one stream (strings such as "%12")."""

    def __init__(self, first_input, masked):
        n = first_input
        self.k = [["%%%d" % (n + 8 * kb + ks) for ks in range(8)] for kb in range(2)]   # K fragments [kb][ks]
        self.rp = ["%%%d" % (n + 16 + ks) for ks in range(8)]                          # row-fragment pointers
        self.tlo = ["%%%d" % (n + 24 + db) for db in range(4)]                         # transposed fragments, lo
        self.thi = ["%%%d" % (n + 28 + db) for db in range(4)]                         # ... hi
        self.stat = "%%%d" % (n + 32)      # pointer of this lane's statistics (LDS base + 16 * (lane / 32))
        self.scale = "%%%d" % (n + 33)     # scale * log2(e), scalar
        self.voff = "%%%d" % (n + 34)      # byte offset of this wavefront's V rows, scalar
        self.src = ["%%%d" % (n + 35 + i) for i in range(4)]   # Q rows, dO rows, two statistics arrays (scalar pairs)
        self.tile_base = "%%%d" % (n + 39)  # LDS address of this wavefront's first slot of a Q tile at stage offset 0
        self.stat_base = "%%%d" % (n + 40)  # LDS address of its first statistics array at stage offset 0
        self.count = n + 41
        if masked:
            self.sinit = ["%%%d" % (n + 41), "%%%d" % (n + 42)]
            self.count = n + 43


def dkvw_stream(o, stage, other, loff, lane16, masked=False):
    """One (head, query block) step of the wide dK/dV kernel for both key blocks.

    `stage` / `other`: byte offsets (operand names or numbers) of the stage that is read (Q tile, dO
    tile 8192 later, -lse / scale at 16384, -delta at 16512) and of the stage the next item is
    copied into; `loff` the four registers with this thread's source offsets of a 32 x 128 tile,
    `lane16` the register with 16 * lane.

    The copies of the next item (its Q and dO rows and statistics) are issued from inside the
    stream, one behind each of the first ten MFMAs.

    The S blocks start from -lse / scale of their query rows (read from the stage) and the dP
    blocks from -delta. With `masked`, the starting values of the two S blocks come in registers
    instead (o.sinit): the caller has put -inf where a pair is not allowed, and the sum, the
    probability and dS of such a pair are then -inf, 0 and 0 without any instruction here knowing
    about masks.
    """
    st = Stream()

    def stats(kb):
        # The S and dP blocks start from the per-row terms instead of 0: -lse / scale and -delta of
        # the block's 16 query rows (4 consecutive rows per read, the accumulator's own order).
        for qd in range(0 if masked else 4):
            st.lds("ds_read_b128 v[%d:%d], %s offset:%s+%d" % (W_S[kb] + 4 * qd, W_S[kb] + 4 * qd + 3, o.stat, stage,
                                                                16384 + 32 * qd), "stat%d" % kb)
        for qd in range(4):
            st.lds("ds_read_b128 v[%d:%d], %s offset:%s+%d" % (W_DP[kb] + 4 * qd, W_DP[kb] + 4 * qd + 3, o.stat, stage,
                                                                16512 + 32 * qd), "stat%d" % kb)

    stats(0)

    def acc16(base):
        return "v[%d:%d]" % (base, base + 15)

    def slot(r):
        lo = W_RING0 + 4 * (r % W_SLOTS)
        return lo, "v[%d:%d]" % (lo, lo + 3)

    # ---- the reads (in issue order) and the MFMAs (in issue order, each naming the reads it needs)
    reads, mfmas = [], []
    for kb in range(2):
        for ks in range(8):
            base = len(reads)
            reads.append(["ds_read_b128 {v4}, %s offset:%s" % (o.rp[ks], stage)])                   # Q
            reads.append(["ds_read_b128 {v4}, %s offset:%s+8192" % (o.rp[ks], stage)])              # dO
            reads.append(["v_add_u32_e32 v%d, %s, %s" % (W_ADDR, o.voff, o.rp[ks]),                  # V
                          "ds_read_b128 {v4}, v%d offset:%d" % (W_ADDR, 8192 * kb)])
            c_s = o.sinit[kb] if (masked and ks == 0) else acc16(W_S[kb])
            mfmas.append(("v_mfma_f32_32x32x16_bf16 %s, {r0}, %s, %s" % (acc16(W_S[kb]), o.k[kb][ks], c_s), [base]))
            mfmas.append(("v_mfma_f32_32x32x16_bf16 %s, {r0}, {r1}, %s" % (acc16(W_DP[kb]), acc16(W_DP[kb])), [base + 1, base + 2]))
    for kb in range(2):
        for step in range(2):
            for db in range(4):
                for which in range(2):  # 0: dV (P^T, dO), 1: dK (dS^T, Q)
                    off = "%s+%d" % (stage, step * 4096 + (8192 if which == 0 else 0))
                    reads.append(["ds_read_b64_tr_b16 {v2lo}, %s offset:%s" % (o.tlo[db], off),
                                  "ds_read_b64_tr_b16 {v2hi}, %s offset:%s" % (o.thi[db], off)])
                    acc = w_acc((0 if which == 0 else 8) + 4 * kb + db)
                    src = (W_S if which == 0 else W_DP)[kb] + 4 * step
                    mfmas.append(("v_mfma_f32_32x32x16_bf16 %s, v[%d:%d], {r0}, %s" % (acc, src, src + 3, acc),
                                  [len(reads) - 1]))
    assert len(mfmas) == 64

    # ---- the arithmetic, attached to MFMA slots. Element e of key block kb starts under MFMA
    # 16 + 16 kb + 11 e / 8: elements 0-7 are packed before the block's first dV / dK MFMA (32 + 16
    # kb) needs them, elements 8-15 before its ninth does, and no MFMA has much more than one
    # element behind it.
    fill = [[] for _ in range(len(mfmas) + 1)]
    for kb in range(2):
        S, DP = W_S[kb], W_DP[kb]
        done = {}
        for e in range(16):
            t = 16 + 16 * kb + (11 * e) // 8
            fill[t] += ["v_mul_f32_e32 v%d, %s, v%d" % (S + e, o.scale, S + e),
                        "v_exp_f32_e32 v%d, v%d" % (S + e, S + e)]
            # the dP block is first read two MFMAs later: its last MFMA has long retired by then
            fill[t + 2] += ["v_mul_f32_e32 v%d, v%d, v%d" % (DP + e, S + e, DP + e)]
            done[e] = t + 2
            if e % 2 == 1:
                k = e // 2
                fill[t + 2] += ["v_cvt_pk_bf16_f32 v%d, v%d, v%d" % (S + k, S + 2 * k, S + 2 * k + 1),
                                "v_cvt_pk_bf16_f32 v%d, v%d, v%d" % (DP + k, DP + 2 * k, DP + 2 * k + 1)]
        assert done[7] < 32 + 16 * kb and done[15] < 40 + 16 * kb

    # ---- emission: reads run ahead of their MFMAs as far as the ring allows
    state = {"issued": 0}
    consumed = [False] * len(reads)

    def issue_reads():
        while state["issued"] < len(reads):
            r = state["issued"]
            if r >= W_SLOTS and not consumed[r - W_SLOTS]:
                break
            lo, v4 = slot(r)
            for text in reads[r]:
                text = text.format(v4=v4, v2lo="v[%d:%d]" % (lo, lo + 1), v2hi="v[%d:%d]" % (lo + 2, lo + 3))
                if text.startswith("ds_"):
                    st.lds(text, r)
                else:
                    st.emit(text)
            state["issued"] += 1

    # the copies: (instructions in front of the MFMA, instructions behind it)
    copies = []
    for which in range(2):
        for n in range(4):
            copies.append((["s_add_u32 m0, %s, %s+%d" % (o.tile_base, other, 8192 * which + 2048 * n)],
                           ["global_load_lds_dwordx4 %s, %s" % (loff[n], o.src[which])]))
    for which in range(2):
        copies.append((["s_add_u32 m0, %s, %s+%d" % (o.stat_base, other, 128 * which)],
                       ["s_mov_b64 exec, 0xff", "global_load_lds_dwordx4 %s, %s" % (lane16, o.src[2 + which]),
                        "s_mov_b64 exec, -1"]))

    issue_reads()
    for i, (text, needs) in enumerate(mfmas):
        st.wait(needs[-1])
        if i < len(copies):
            for line in copies[i][0]:
                st.emit(line)
        names = {"r%d" % n: slot(r)[1] for n, r in enumerate(needs)}
        st.emit(text.format(**names))
        if i < len(copies):
            for line in copies[i][1]:
                st.emit(line)
        for r in needs:
            consumed[r] = True
        if i == 3:
            stats(1)   # (the registers are free: their last readers were the previous step's MFMAs)
        issue_reads()
        for line in fill[i]:
            st.emit(line)
    assert not fill[64] and state["issued"] == len(reads)
    return st.lines


def dkvw_step_sequence(masked=False):
    """A single step. operands: %0-%40 as WideOperands(0) lays them out, %41 / %42 the S starting
    values (masked form only), then the stage offset, the other stage's offset (immediates), the four
    source offsets of this thread and 16 * lane."""
    o = WideOperands(0, masked)
    n = o.count
    stage, other = "%%%d" % n, "%%%d" % (n + 1)
    loff = ["%%%d" % (n + 2 + i) for i in range(4)]
    return dkvw_stream(o, stage, other, loff, "%%%d" % (n + 6), masked) + TAIL


def dkvw_run_sequence():
    """A run of all-allowed steps over consecutive query blocks of one head: the stream of the
    stage the run starts on, then the stream of the other stage, and so on, each followed by the
    wait for the copies it issued and the workgroup barrier; the source offsets advance by one
    query block per step.

    operands: %0 steps left (scalar, counted down to 0); %1-%4 this thread's source offsets and %5
    16 * lane (advanced); %6-%46 as WideOperands(6) lays them out; %47 bytes between the Q rows of
    consecutive query blocks (scalar); %48 / %49 byte offsets of the stage the run starts on and of
    the other one.
    """
    o = WideOperands(6, False)
    assert o.count == 47
    loff, lane16 = ["%1", "%2", "%3", "%4"], "%5"
    close = ["s_waitcnt vmcnt(0)", "s_barrier"] + ["v_add_u32_e32 %s, %%47, %s" % (r, r) for r in loff] + [
        "v_add_u32_e32 %s, 0x80, %s" % (lane16, lane16), "s_sub_u32 %0, %0, 1", "s_cmp_eq_u32 %0, 0"]
    lines = ["dkvw_run_%=:"]
    lines += dkvw_stream(o, "%48", "%49", loff, lane16) + close + ["s_cbranch_scc1 dkvw_run_end_%="]
    lines += dkvw_stream(o, "%49", "%48", loff, lane16) + close + ["s_cbranch_scc0 dkvw_run_%="]
    lines += ["dkvw_run_end_%=:"]
    return lines + TAIL


def dkvw_zero():
    return ["v_accvgpr_write_b32 a%d, 0" % r for r in range(256)]


def dkvw_read():
    """operands: %0-%15 the 16 values of one accumulator, %16 its first register number."""
    return ["v_accvgpr_read_b32 %%%d, a[%%16+%d]" % (e, e) for e in range(16)]


def clobbers():
    regs = ", ".join('"v%d"' % r for r in range(SCRATCH0, SCRATCH0 + 16))
    dkv = ", ".join('"v%d"' % r for r in range(DKV_SCRATCH0, 256))
    wide = ", ".join('"v%d"' % r for r in range(W_FIRST, 256))
    accs = ", ".join('"a%d"' % r for r in range(256))
    return ("#define CT_ATTN_ASM_SCRATCH %s\n\n#define CT_DKV_ASM_SCRATCH %s\n\n#define CT_DKVW_ASM_SCRATCH %s\n\n"
            "#define CT_DKVW_ACCUMULATORS %s\n\n#define CT_FWD_PRIVATE %s\n" % (regs, dkv, wide, accs,
                                                                             fwd_private_clobbers()))


if __name__ == "__main__":
    print("// Generated by gen_attn_asm.py -- do not edit by hand.")
    print(emit(pv_sequence(4, 4), "CT_ATTN_PV_SEQUENCE"))
    print(emit(qk_sequence(4, 4), "CT_ATTN_QK_SEQUENCE"))
    for cur in ("a", "b"):
        for name, lines in fwd_statements(cur).items():
            print(emit(lines, "CT_FWD_%s_%s" % (name, cur.upper())))
    for name, lines in fwd_accumulator_statements().items():
        print(emit(lines, "CT_FWD_ACC_%s" % name))
    print(emit(dq_sdp_half_sequence(), "CT_DQ_SDP_HALF_SEQUENCE"))
    print(emit(dq_acc_half_sequence(), "CT_DQ_ACC_HALF_SEQUENCE"))
    print(emit(dkv_sdp_sequence(), "CT_DKV_SDP_SEQUENCE"))
    print(emit(dkv_acc_sequence(), "CT_DKV_ACC_SEQUENCE"))
    print(emit(dkvw_step_sequence(), "CT_DKVW_FAST_SEQUENCE"))
    print(emit(dkvw_step_sequence(masked=True), "CT_DKVW_MASKED_SEQUENCE"))
    print(emit(dkvw_run_sequence(), "CT_DKVW_RUN_SEQUENCE"))
    print(emit(dkvw_zero(), "CT_DKVW_ZERO"))
    print(emit(dkvw_read(), "CT_DKVW_READ"))
    print(clobbers())
