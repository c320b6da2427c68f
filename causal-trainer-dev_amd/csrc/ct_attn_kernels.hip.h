// Attention kernels for gfx950: forward and delta (shared pieces for dQ too).
//
// Common structure. A workgroup is 4 wavefronts. In the forward and dQ
// kernels every wavefront owns 32 query rows of one query head (a "row
// block") and walks the 64-key tiles its rows can see; K and V tiles are
// staged through LDS (double buffered, one barrier per tile) and shared by
// the 4 wavefronts. With GQA the 4 wavefronts of a workgroup are HS query
// heads of the same KV head times 4/HS consecutive row blocks, so one K/V
// tile feeds HS heads.
//
// Scores are produced transposed, S^T = K Q^T, so that in the MFMA
// accumulator layout one lane holds 16 keys of a single query: row max / row
// sum are in-lane reductions plus one exchange with lane^32, and the
// probabilities can be fed straight back as the B operand of O^T = V^T P^T
// (V^T fetched with transposed LDS reads).
//
// Numerics follow the reference kernel (src/kernels/efficient_attention.py):
// the softmax scale is rounded to bf16 and multiplied into q in bf16
// (:906-907), scores and softmax statistics are f32 (:586-616), rows without
// a visible key give O = 0 and LSE = 0 (:746-760). Probabilities are rounded
// to bf16 for the PV product as in vanilla_attention
// (src/modeling/attention.py:138).
#pragma once

#include <type_traits>

#include "ct_attn_asm.inc"
#include "ct_attn_meta.hip.h"
#include "ct_common.hip.h"

namespace ct {

constexpr int kKeyTile = 64;
constexpr float kNegInf = -__builtin_inff();

struct AttnParams {
  const bf16* q;
  const bf16* k;
  const bf16* v;
  const int* seg;
  const int* end;   // may be null
  const int* meta;  // [B][nrb][kMetaW]
  const int* sched; // [B][schedule_ints(nrb)]
  bf16* out;        // forward: written; backward: forward output
  float* lse;
  const bf16* dout;
  float* delta;     // backward: rowsum(out * dout), head-major [B, Hq, S] (written by dQ, read by dK/dV)
  float* lse2;      // backward: -lse / scale, head-major [B, Hq, S] (written by dQ, read by dK/dV)
  bf16* dq;
  bf16* dk;
  bf16* dv;
  int B, S, Hq, Hkv;
  float scale;      // already rounded to bf16
  // dK/dV work list (backward only)
  int* dkv_header;
  int2* dkv_entries;
  int* dq_counters;  // kDqCounters ints, zeroed by the work-list kernel of the same call
  float* dkv_partials;
  int dkv_max_entries, dkv_max_partials;
  // KV heads [kvh_base, kvh_base + kvh_count) are what a backward launch works on (all of them
  // unless dS goes through the workspace, which bounds that region by running the heads in passes)
  int kvh_base, kvh_count;
  char* ds;              // dS region of the pass, null when dQ recomputes S and dP
  size_t ds_row_blocks;  // dS blocks reserved per (query head, batch row)
};

// ---------------------------------------------------------------------------
// K/V tile staging: global -> registers -> swizzled LDS.
// LDS stage layout: K tile, V tile (64 x D bf16 each), 64 segment ids.
// ---------------------------------------------------------------------------
template <int D>
struct KvStage {
  static constexpr int kTileBytes = kKeyTile * D * 2;
  static constexpr int kK = 0;
  static constexpr int kV = kTileBytes;
  static constexpr int kSeg = 2 * kTileBytes;
  static constexpr int kBytes = 2 * kTileBytes + kKeyTile * 4;
};

// Asynchronous fetch of key tile `tile` (K rows, V rows, segment ids) into an LDS stage.
template <int D>
struct KvFetcher {
  TileDma<kKeyTile, D / 8> dma;
  const char* kbase;
  const char* vbase;
  const int* segb;
  size_t row_stride_bytes;
  CT_DEVICE KvFetcher(const bf16* k, const bf16* v, const int* seg, size_t row_stride_elems)
      : dma(row_stride_elems * 2), kbase(reinterpret_cast<const char*>(k)),
        vbase(reinterpret_cast<const char*>(v)), segb(seg), row_stride_bytes(row_stride_elems * 2) {}
  CT_DEVICE void issue(int tile, lds_addr stage) const {
    const size_t origin = (size_t)tile * kKeyTile * row_stride_bytes;
    dma.issue(kbase + origin, stage + KvStage<D>::kK);
    dma.issue(vbase + origin, stage + KvStage<D>::kV);
    if (threadIdx.x < 16)  // 64 ids = 16 lanes x 16 bytes, linear layout
      dma16_s(segb + tile * kKeyTile, threadIdx.x * 16, stage + KvStage<D>::kSeg);
  }
};

// Decoded position of a workgroup / wavefront in the (batch, head, row block)
// space. Hardware workgroup ids run over (rank, group): the group (batch,
// head slice, KV head) is the fast index, so a group always lands on the same
// XCD (ids are dealt round robin to the 8 XCDs) and keeps its K/V in that L2;
// the rank is the position in the batch row's work-sorted schedule, longest
// tiles first.
template <int HS, int NW = 4>
struct QueryWork {
  static constexpr int PB = NW / HS;  // row blocks per workgroup
  int b, h, kvh, qt, rb;
  CT_DEVICE QueryWork(const AttnParams& p) {
    const int nrb = p.S / 32;
    const int g = p.Hq / p.Hkv;
    const int slices = g / HS;
    const int groups = p.B * slices * p.Hkv;
    const int group = blockIdx.x % groups, rank = blockIdx.x / groups;
    kvh = group % p.Hkv;
    const int rest = group / p.Hkv;
    const int slice = rest % slices;
    b = rest / slices;
    const int* sched = p.sched + (size_t)b * schedule_ints(nrb) + query_schedule_offset(nrb, PB);
    qt = uniform(sched[rank]);
    const int w = threadIdx.x >> 6;
    h = kvh * g + slice * HS + (w % HS);
    rb = qt * PB + (w / HS);
  }
  // explicit coordinates: batch row, KV head, head slice of the group, query tile
  CT_DEVICE QueryWork(const AttnParams& p, int b_, int kvh_, int slice, int qt_)
      : b(b_), kvh(kvh_), qt(qt_) {
    // (wave-uniform, and said so: head and row block are then scalars that cost nothing to keep
    // or to form again, instead of per-lane values hoisted out of the caller's loop)
    const int w = uniform(threadIdx.x >> 6);
    h = kvh * (p.Hq / p.Hkv) + slice * HS + (w % HS);
    rb = qt * PB + (w / HS);
  }
};

// S^T (two 32-key blocks) = K_tile Q^T for this wavefront's 32 queries.
// `tile_off` is the tile's byte offset from the LDS base the offsets were built on.
template <int D, class RowFrags>
CT_DEVICE void scores_t(int tile_off, const RowFrags& ro, const bf16x8* qf, f32x16* s) {
  s[0] = zero16();
  s[1] = zero16();
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) s[kb] = mfma32(ro.load(tile_off, kb, ks), qf[ks], s[kb]);
  }
}

// Sets the scores of disallowed (query, key) pairs of a transposed score tile to -inf.
// The pair rule is seg_k == seg_q != 0 and key <= end_q (src/modeling/attention.py:67-97);
// each half is only evaluated where the tile's summaries do not already prove it:
//   SEG     the key tile or the query block mixes segment ids
//   CAUSAL  the tile's last key lies beyond the smallest visible end of the block
// `seg_q_or_never` is the query's id, or -1 for a padding query (ids are >= 0, so -1 never
// matches); `last_rel` is end_q - first key of the tile - 4 * (lane / 32), which makes the
// key offset of accumulator register r of block kb the lane-independent constant
// 32 kb + 8 (r / 4) + r % 4.
template <bool SEG, bool CAUSAL>
CT_DEVICE void mask_block_t(lds_addr segk, int seg_q_or_never, int last_rel, int kb, f32x16& s) {
  // (opaque, so that the lane's share of the addresses below is recomputed here rather than
  // kept in a register across the caller's loop, where it ends up spilled)
  int lane = lane_id();
  asm volatile("" : "+v"(lane));
  const int half = lane >> 5;
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {
    i32x4 sk = {0, 0, 0, 0};
    if constexpr (SEG) sk = lds_load<i32x4>(segk + (kb * 32 + 8 * qd + 4 * half) * 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      bool ok = true;
      if constexpr (SEG) ok = sk[e] == seg_q_or_never;
      if constexpr (CAUSAL) ok = ok && (kb * 32 + 8 * qd + e <= last_rel);
      s[4 * qd + e] = ok ? s[4 * qd + e] : kNegInf;
    }
  }
}
template <bool SEG, bool CAUSAL>
CT_DEVICE void mask_scores_t(lds_addr segk, int seg_q_or_never, int last_rel, f32x16* s) {
  mask_block_t<SEG, CAUSAL>(segk, seg_q_or_never, last_rel, 0, s[0]);
  mask_block_t<SEG, CAUSAL>(segk, seg_q_or_never, last_rel, 1, s[1]);
}

// acc (D x 32 queries, transposed) += X^T W^T where X is a 64-row LDS tile read
// transposed and W^T are the accumulator-layout weights wt[2].
template <int D, class TrFrags>
CT_DEVICE void accumulate_t(int tile_off, const TrFrags& to, const f32x16* wt, f32x16* acc) {
#pragma unroll
  for (int step = 0; step < 4; ++step) {
    const bf16x8 bop = pack_acc8(wt[step >> 1], step & 1);
#pragma unroll
    for (int db = 0; db < D / 32; ++db) acc[db] = mfma32(to.load(tile_off, step, db), bop, acc[db]);
  }
}

// Write a transposed accumulator (D x 32 rows) as bf16 rows of D elements to
// global memory, staged through this wavefront's private LDS patch so that
// the global stores are 16 bytes per lane and contiguous per row.
template <int D>
CT_DEVICE void store_rows_t(const f32x16* acc, float row_scale, lds_addr patch, bf16* gbase,
                            size_t row_stride) {
  constexpr int CPR = D / 8;
  int l = lane_id();
  // The 16 patch addresses below depend on the lane only. Hoisted out of a caller's loop they
  // would be 16 registers held for the whole kernel (and, once spilled, 16 scratch reloads
  // with a full memory wait each per call), so the lane id is made opaque here and the
  // addresses are recomputed where they are used.
  asm volatile("" : "+v"(l));
  const int j = l & 31, half = l >> 5;
  using Patch = PatchRows<D>;
  const lds_addr store_base = Patch::store_base(patch, j, half);
  const unsigned row_swizzle = Patch::row_swizzle(j);
  auto block = [&](auto db_tag) {
    constexpr int db = decltype(db_tag)::value;
    auto quad = [&](auto qd_tag) {
      constexpr int qd = decltype(qd_tag)::value;
      bf16x4 pk;
#pragma unroll
      for (int e = 0; e < 4; ++e) pk[e] = (bf16)(acc[db][4 * qd + e] * row_scale);
      lds_store<bf16x4>(store_base + Patch::template chunk_term<db * 4 + qd>(row_swizzle), pk);
    };
    quad(std::integral_constant<int, 0>{});
    quad(std::integral_constant<int, 1>{});
    quad(std::integral_constant<int, 2>{});
    quad(std::integral_constant<int, 3>{});
  };
  block(std::integral_constant<int, 0>{});
  block(std::integral_constant<int, 1>{});
  if constexpr (D > 64) {
    block(std::integral_constant<int, 2>{});
    block(std::integral_constant<int, 3>{});
  }
  static_assert(D == 64 || D == 128, "two or four 32-column blocks");
  (void)CPR;
  __builtin_amdgcn_wave_barrier();
  Patch::to_global(patch, l, gbase, row_stride);
}

// Shared prologue of the forward and dQ kernels.
template <int D, int HS, int NW = 4>
struct QueryTileContext {
  static constexpr int PB = NW / HS;
  QueryWork<HS, NW> work;
  const int* meta_b;
  QueryBlockBounds mine;
  int first, last;
  int pos, seg_q, end_q;
  bool active;  // false for the row blocks past the end of a partial last tile
  size_t q_off, stat_off;
  const bf16* kbase;
  const bf16* vbase;
  const int* segb;
  CT_DEVICE explicit QueryTileContext(const AttnParams& p) : work(p) { init(p); }
  CT_DEVICE QueryTileContext(const AttnParams& p, int b, int kvh, int slice, int qt)
      : work(p, b, kvh, slice, qt) {
    init(p);
  }
  CT_DEVICE void init(const AttnParams& p) {
    const int nrb = p.S / 32;
    derive(p);
    mine = query_block_bounds(meta_b, work.rb);
    if (!active) mine.min_nz = 0;    // interacts with nothing
    first = INT_MAX;
    last = -1;
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      if (work.qt * PB + i >= nrb) break;
      const MetaPtr m = meta_const(meta_b + (work.qt * PB + i) * kMetaW);
      first = min(first, uniform(m[kKvFirst]));
      last = max(last, uniform(m[kKvLast]));
    }
    seg_q = p.seg[(size_t)work.b * p.S + pos];
    end_q = p.end ? p.end[(size_t)work.b * p.S + pos] : pos;
  }
  // everything that follows from the coordinates by arithmetic
  CT_DEVICE void derive(const AttnParams& p) {
    const int nrb = p.S / 32;
    meta_b = p.meta + (size_t)work.b * nrb * kMetaW;
    active = work.rb < nrb;
    if (!active) work.rb = nrb - 1;  // keeps every address below in range
    pos = work.rb * 32 + (lane_id_here() & 31);
    q_off = (((size_t)work.b * p.S + pos) * p.Hq + work.h) * D;
    stat_off = ((size_t)work.b * p.S + pos) * p.Hq + work.h;
    kbase = p.k + ((size_t)work.b * p.S * p.Hkv + work.kvh) * D;
    vbase = p.v + ((size_t)work.b * p.S * p.Hkv + work.kvh) * D;
    segb = p.seg + (size_t)work.b * p.S;
  }

  // The same context from values read earlier: the bounds (scalar loads, so that waiting for
  // them is no wait for vector memory) and the row's id and visible end.
  struct TileBounds {
    // as loaded: nothing is computed from them where they are requested, so nothing waits there
    QueryBlockBounds mine;
    int kv_first[PB], kv_last[PB];
  };
  CT_DEVICE static TileBounds tile_bounds(const AttnParams& p, const QueryWork<HS, NW>& work) {
    const int nrb = p.S / 32;
    const int* meta = p.meta + (size_t)work.b * nrb * kMetaW;
    TileBounds t;
    t.mine = query_block_bounds(meta, min(work.rb, nrb - 1));
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      const MetaPtr m = meta_const(meta + min(work.qt * PB + i, nrb - 1) * kMetaW);
      t.kv_first[i] = m[kKvFirst];
      t.kv_last[i] = m[kKvLast];
    }
    return t;
  }
  CT_DEVICE QueryTileContext(const AttnParams& p, int b, int kvh, int slice, int qt, const TileBounds& t,
                             int seg_q_, int end_q_)
      : work(p, b, kvh, slice, qt) {
    const int nrb = p.S / 32;
    derive(p);
    mine = t.mine;
    if (!active) mine.min_nz = 0;
    first = INT_MAX;
    last = -1;
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      if (work.qt * PB + i >= nrb) break;
      first = min(first, uniform(t.kv_first[i]));
      last = max(last, uniform(t.kv_last[i]));
    }
    seg_q = seg_q_;
    end_q = p.end ? end_q_ : pos;
  }
  CT_DEVICE bool row_valid() const { return seg_q != 0; }
  // does this wavefront's row block have anything in key tile t (bounds kb)?
  CT_DEVICE bool wave_visits(const KeyTileBounds& kb, int t) const {
    return blocks_interact(mine.min_nz, mine.max_id, mine.end_max, uniform(kb.min_nz),
                           uniform(kb.max_id), t * kKeyTile);
  }
  CT_DEVICE bool interior(const KeyTileBounds& kb, int t) const {
    return tile_is_interior(mine.uniform, mine.end_min, uniform(kb.uniform),
                            t * kKeyTile + kKeyTile - 1);
  }
};

// Hand-scheduled MFMA sequences for D = 128 (see gen_attn_asm.py). TILE_OFF is the byte
// offset of the operand tile from the LDS base the fragment pointers were built on.
template <int TILE_OFF>
CT_DEVICE void pv_sequence_128(const TrFragOffsets<16, KSlots::kAccum>& to, const bf16x8* pf,
                               f32x16* oacc) {
  asm volatile(CT_ATTN_PV_SEQUENCE
               : "+v"(oacc[0]), "+v"(oacc[1]), "+v"(oacc[2]), "+v"(oacc[3])
               : "v"(to.ptr[0][0]), "v"(to.ptr[0][1]), "v"(to.ptr[0][2]), "v"(to.ptr[0][3]),
                 "v"(to.ptr[1][0]), "v"(to.ptr[1][1]), "v"(to.ptr[1][2]), "v"(to.ptr[1][3]),
                 "v"(pf[0]), "v"(pf[1]), "v"(pf[2]), "v"(pf[3]), "i"(TILE_OFF)
               : "memory", CT_ATTN_ASM_SCRATCH);
}
template <int TILE_OFF>
CT_DEVICE void qk_sequence_128(const RowFragOffsets<16>& ro, const bf16x8* qf, f32x16* s) {
  asm volatile(CT_ATTN_QK_SEQUENCE
               : "=&v"(s[0]), "=&v"(s[1])
               : "v"(ro.ptr[0]), "v"(ro.ptr[1]), "v"(ro.ptr[2]), "v"(ro.ptr[3]), "v"(ro.ptr[4]),
                 "v"(ro.ptr[5]), "v"(ro.ptr[6]), "v"(ro.ptr[7]), "v"(qf[0]), "v"(qf[1]), "v"(qf[2]),
                 "v"(qf[3]), "v"(qf[4]), "v"(qf[5]), "v"(qf[6]), "v"(qf[7]), "i"(TILE_OFF)
               : "memory", CT_ATTN_ASM_SCRATCH);
}

// Forward, interleaved form (see gen_attn_asm.py): statements on registers that only they name:
// the score buffers v[112:143] ("a") and v[144:175] ("b"), a fragment ring v[176:191] and the
// output accumulator O^T in a[0:63]. NAME = a: the scores of the current key tile are in a, P^T of
// the tile before in the first half of b, and the next tile's scores go to b; NAME = b the other
// way round. Every statement lists all of these registers as clobbered, so the compiler keeps no
// value of its own there across one, and a static check of the compiled kernel
// (isa_hazards.private_registers) proves that it uses none of them between statements either.
// A wavefront's share of a step's global -> LDS copies, for the statement that issues them: the
// sources (wave-uniform addresses of the V tile and the K tile), this thread's two byte offsets
// into a tile (a tile is two pieces of 1 KB per wavefront), and the LDS destinations (the V
// pieces, then the K pieces).
struct FwdCopies {
  unsigned long long v_source, k_source;
  unsigned lane_off[2];
  unsigned dst[4];
};
#define CT_FWD_TR_PTRS(to)                                                                              \
  [lo0] "v"(to.ptr[0][0]), [lo1] "v"(to.ptr[0][1]), [lo2] "v"(to.ptr[0][2]), [lo3] "v"(to.ptr[0][3]), \
      [hi0] "v"(to.ptr[1][0]), [hi1] "v"(to.ptr[1][1]), [hi2] "v"(to.ptr[1][2]), [hi3] "v"(to.ptr[1][3])
#define CT_FWD_ROW_PTRS(ro, qf)                                                                          \
  [rp0] "v"(ro.ptr[0]), [rp1] "v"(ro.ptr[1]), [rp2] "v"(ro.ptr[2]), [rp3] "v"(ro.ptr[3]),               \
      [rp4] "v"(ro.ptr[4]), [rp5] "v"(ro.ptr[5]), [rp6] "v"(ro.ptr[6]), [rp7] "v"(ro.ptr[7]),           \
      [q0] "v"(qf[0]), [q1] "v"(qf[1]), [q2] "v"(qf[2]), [q3] "v"(qf[3]), [q4] "v"(qf[4]), [q5] "v"(qf[5]), \
      [q6] "v"(qf[6]), [q7] "v"(qf[7])
#define CT_FWD_STATEMENTS(NAME, UPPER)                                                                        \
  /* first half of the PV product | maximum of the scores (times log2 e, over the lane pair) */              \
  template <int V_OFF>                                                                                        \
  CT_DEVICE float fwd_max_##NAME(const TrFragOffsets<16, KSlots::kAccum>& to, const FwdCopies& cp) {         \
    float mx, tmp;                                                                                            \
    asm volatile(CT_FWD_MAX_##UPPER                                                                           \
                 : [mx] "=&v"(mx), [tmp] "=&v"(tmp)                                                           \
                 : CT_FWD_TR_PTRS(to), [c] "s"(kLog2e), [voff] "i"(V_OFF), [vsrc] "s"(cp.v_source),           \
                   [ksrc] "s"(cp.k_source), [off0] "v"(cp.lane_off[0]), [off1] "v"(cp.lane_off[1]),           \
                   [d0] "s"(cp.dst[0]), [d1] "s"(cp.dst[1]), [d2] "s"(cp.dst[2]), [d3] "s"(cp.dst[3])          \
                 : "memory", "m0", CT_FWD_PRIVATE);                                                           \
    return mx;                                                                                                \
  }                                                                                                           \
  /* second half of the PV product | first exponentials */                                                    \
  template <int V_OFF>                                                                                        \
  CT_DEVICE void fwd_exp_a_##NAME(const TrFragOffsets<16, KSlots::kAccum>& to, float m, float& psum) {       \
    asm volatile(CT_FWD_EXP_A_##UPPER                                                                         \
                 : [psum] "+v"(psum)                                                                          \
                 : CT_FWD_TR_PTRS(to), [m] "v"(m), [c] "s"(kLog2e), [voff] "i"(V_OFF)                         \
                 : "memory", CT_FWD_PRIVATE);                                                                 \
  }                                                                                                           \
  /* scores of the next tile | the other exponentials */                                                      \
  template <int K_OFF>                                                                                        \
  CT_DEVICE void fwd_exp_b_##NAME(const RowFragOffsets<16>& ro, const bf16x8* qf, float m, float& psum) {    \
    asm volatile(CT_FWD_EXP_B_##UPPER                                                                         \
                 : [psum] "+v"(psum)                                                                          \
                 : CT_FWD_ROW_PTRS(ro, qf), [m] "v"(m), [c] "s"(kLog2e), [koff] "i"(K_OFF)                    \
                 : "memory", CT_FWD_PRIVATE);                                                                 \
  }                                                                                                           \
  CT_DEVICE float fwd_max_only_##NAME() {                                                                     \
    float mx, tmp;                                                                                            \
    asm volatile(CT_FWD_MAX_ONLY_##UPPER                                                                      \
                 : [mx] "=&v"(mx), [tmp] "=&v"(tmp)                                                           \
                 : [c] "s"(kLog2e)                                                                            \
                 : "memory", CT_FWD_PRIVATE);                                                                 \
    return mx;                                                                                                \
  }                                                                                                           \
  CT_DEVICE void fwd_exp_only_##NAME(float m, float& psum) {                                                  \
    asm volatile(CT_FWD_EXP_ONLY_##UPPER                                                                      \
                 : [psum] "+v"(psum)                                                                          \
                 : [m] "v"(m), [c] "s"(kLog2e)                                                                \
                 : "memory", CT_FWD_PRIVATE);                                                                 \
  }                                                                                                           \
  template <int V_OFF>                                                                                        \
  CT_DEVICE void fwd_pv_##NAME(const TrFragOffsets<16, KSlots::kAccum>& to) {                                \
    asm volatile(CT_FWD_PV_##UPPER : : CT_FWD_TR_PTRS(to), [voff] "i"(V_OFF) : "memory", CT_FWD_PRIVATE);     \
  }                                                                                                           \
  template <int V_OFF>                                                                                        \
  CT_DEVICE void fwd_pv_late_##NAME(const TrFragOffsets<16, KSlots::kAccum>& to) {                           \
    asm volatile(CT_FWD_PV_LATE_##UPPER : : CT_FWD_TR_PTRS(to), [voff] "i"(V_OFF) : "memory", CT_FWD_PRIVATE); \
  }                                                                                                           \
  /* scores of the next tile into the other buffer */                                                         \
  template <int K_OFF>                                                                                        \
  CT_DEVICE void fwd_qk_##NAME(const RowFragOffsets<16>& ro, const bf16x8* qf) {                             \
    asm volatile(CT_FWD_QK_##UPPER : : CT_FWD_ROW_PTRS(ro, qf), [koff] "i"(K_OFF) : "memory", CT_FWD_PRIVATE); \
  }                                                                                                           \
  /* the same with the output accumulator cleared behind the MFMAs (a query tile's first scores) */          \
  template <int K_OFF>                                                                                        \
  CT_DEVICE void fwd_qk_zero_##NAME(const RowFragOffsets<16>& ro, const bf16x8* qf) {                        \
    asm volatile(CT_FWD_QK_ZERO_##UPPER : : CT_FWD_ROW_PTRS(ro, qf), [koff] "i"(K_OFF) : "memory", CT_FWD_PRIVATE); \
  }                                                                                                           \
  /* -inf where the key's offset in the tile exceeds rel (per lane) */                                        \
  CT_DEVICE void fwd_mask_causal_##NAME(int rel) {                                                            \
    asm volatile(CT_FWD_MASK_CAUSAL_##UPPER                                                                   \
                 :                                                                                            \
                 : [rel] "v"(rel), [ninf] "v"(kNegInf)                                                        \
                 : "memory", "vcc", CT_FWD_PRIVATE);                                                          \
  }                                                                                                           \
  /* -inf where the key's id differs from seg (per lane); ids: the lane's address of the id of key */        \
  /* 4 * (lane / 32) of the tile in the id ring                                                      */        \
  CT_DEVICE void fwd_mask_ids_##NAME(lds_addr ids, int seg) {                                                 \
    asm volatile(CT_FWD_MASK_IDS_##UPPER                                                                      \
                 :                                                                                            \
                 : [idp] "v"(ids), [segq] "v"(seg), [ninf] "v"(kNegInf)                                       \
                 : "memory", "vcc", CT_FWD_PRIVATE);                                                          \
  }
CT_FWD_STATEMENTS(a, A)
CT_FWD_STATEMENTS(b, B)

// The output accumulator in a[0:63]: cleared, multiplied by the row's factor (one per lane), and
// read out as the four 32-column blocks of O^T.
CT_DEVICE void fwd_acc_zero() { asm volatile(CT_FWD_ACC_ZERO : : : "memory", CT_FWD_PRIVATE); }
CT_DEVICE void fwd_acc_scale(float alpha) {
  asm volatile(CT_FWD_ACC_SCALE : : [alpha] "v"(alpha) : "memory", CT_FWD_PRIVATE);
}
template <int INDEX>
CT_DEVICE f32x16 fwd_acc_read() {
  float v[16];
  asm volatile(CT_DKVW_READ
               : "=v"(v[0]), "=v"(v[1]), "=v"(v[2]), "=v"(v[3]), "=v"(v[4]), "=v"(v[5]), "=v"(v[6]), "=v"(v[7]),
                 "=v"(v[8]), "=v"(v[9]), "=v"(v[10]), "=v"(v[11]), "=v"(v[12]), "=v"(v[13]), "=v"(v[14]), "=v"(v[15])
               : "i"(16 * INDEX)
               : "memory");
  f32x16 out;
#pragma unroll
  for (int e = 0; e < 16; ++e) out[e] = v[e];
  return out;
}

// dQ kernel, one 32-key half of a key tile (see gen_attn_asm.py): S^T and dP^T of the half, and
// the half's contribution to dQ^T. K_OFF / V_OFF are the byte offsets of the half's K and V rows.
template <int K_OFF, int V_OFF>
CT_DEVICE void dq_sdp_half_128(const RowFragOffsets<16>& ro, const bf16x8* qf, const bf16x8* dof, f32x16& s,
                               f32x16& dp) {
  asm volatile(CT_DQ_SDP_HALF_SEQUENCE
               : "=&v"(s), "=&v"(dp)
               : "v"(ro.ptr[0]), "v"(ro.ptr[1]), "v"(ro.ptr[2]), "v"(ro.ptr[3]), "v"(ro.ptr[4]),
                 "v"(ro.ptr[5]), "v"(ro.ptr[6]), "v"(ro.ptr[7]), "v"(qf[0]), "v"(qf[1]), "v"(qf[2]),
                 "v"(qf[3]), "v"(qf[4]), "v"(qf[5]), "v"(qf[6]), "v"(qf[7]), "v"(dof[0]), "v"(dof[1]),
                 "v"(dof[2]), "v"(dof[3]), "v"(dof[4]), "v"(dof[5]), "v"(dof[6]), "v"(dof[7]), "i"(K_OFF),
                 "i"(V_OFF)
               : "memory", CT_ATTN_ASM_SCRATCH);
}
template <int K_OFF>
CT_DEVICE void dq_acc_half_128(const TrFragOffsets<16, KSlots::kAccum>& to, bf16x8 p0, bf16x8 p1, f32x16* acc) {
  asm volatile(CT_DQ_ACC_HALF_SEQUENCE
               : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3])
               : "v"(to.ptr[0][0]), "v"(to.ptr[0][1]), "v"(to.ptr[0][2]), "v"(to.ptr[0][3]),
                 "v"(to.ptr[1][0]), "v"(to.ptr[1][1]), "v"(to.ptr[1][2]), "v"(to.ptr[1][3]), "v"(p0), "v"(p1),
                 "i"(K_OFF)
               : "memory", CT_ATTN_ASM_SCRATCH);
}

// ---------------------------------------------------------------------------
// Forward
//
// One workgroup of 8 wavefronts per compute unit (wavefronts w and w + 4 share a SIMD), each with
// 32 query rows of one head. Two forms of the key-tile loop:
//
// D = 128, interleaved (attn_fwd_item). Per key tile t a wavefront has three pieces of work: the
// softmax arithmetic of tile t (vector ALU), O += V(t-1)^T P(t-1)^T and S(t+1)^T = K(t+1) Q^T
// (32 MFMAs). They are independent of each other, so the arithmetic is issued between the MFMAs
// of the same wavefront (three asm statements per tile, see gen_attn_asm.py): about five vector
// instructions fit behind an MFMA without delaying the next one, and the matrix pipe does not
// wait for a separate arithmetic phase. The first and the last tile of a query tile, tiles that a
// wavefront's rows do not see, and tiles on which the running maximum has to move take the same
// pieces one after the other (same instructions on the same registers: same bits). The scores
// never leave the registers that those statements name.
// LDS holds 2 stages; stage s = V rows of tile s and K rows of tile s + 2, exactly what the step
// of tile s + 1 reads. The copies for stage t are issued at the start of the step of tile t, into
// the buffer that the step before has finished with, and awaited at its end, in front of the one
// workgroup barrier per step. Segment ids of the key tiles go through a ring of 4 slots (tile t
// in slot t % 4, copied together with its K rows, read in the step of tile t).
//
// Other head sizes, phased (attn_fwd_item_phased):
// One workgroup of 8 wavefronts per compute unit: wavefronts w and w + 4 share
// a SIMD. Per key tile a wavefront alternates between a VALU phase (softmax of
// the tile's scores) and an MFMA phase (O += V^T P of this tile, then the
// scores of the next tile). Wavefronts 4..7 (the "late" group) run half a step
// behind wavefronts 0..3 (they pass one extra barrier before the loop, the
// others one after it), and a workgroup barrier closes every phase, so on each
// SIMD one wavefront is in its VALU phase while the other one is in its MFMA
// phase and the two pipes overlap.
//
// Global phase numbering: the early group runs VALU phase t in phase 2t and
// MFMA phase t in phase 2t + 1; the late group one phase later. LDS holds 2
// stages; stage s = V rows of tile s and K rows of tile s + 1, exactly the
// operands of MFMA phase s, read in phases 2s + 1 and 2s + 2. The copies for
// stage t + 1 replace stage t - 1 and are issued at the start of phase 2t + 1
// (early group: on entering MFMA phase t; late group: on entering VALU phase
// t) and awaited at the end of phase 2t + 2, one barrier before the first read.
// Segment ids of the key tiles go through a ring of 4 slots (tile t in slot
// t % 4, copied together with stage t - 1, read in phases 2t and 2t + 1).
// ---------------------------------------------------------------------------
constexpr int kFwdWaves = 8;
constexpr float kRescaleSlack = 8.f;

template <int D>
struct VkStage {
  static constexpr int kTileBytes = kKeyTile * D * 2;
  static constexpr int kV = 0;
  static constexpr int kK = kTileBytes;
  static constexpr int kBytes = 2 * kTileBytes;
  static constexpr int kSegRing = 2 * kBytes;  // after both stages
  static constexpr int kSegSlotBytes = kKeyTile * 4;
  // behind the id ring: per wavefront, the patch through which its O rows go to memory (a place of
  // its own, so that the next query tile's first copies can be on their way meanwhile)
  static constexpr int kStorePatches = kSegRing + 4 * kSegSlotBytes;
  static constexpr int kStorePatchBytes = 32 * D * 2;
  static constexpr int kTotalBytes = kStorePatches + kFwdWaves * kStorePatchBytes;
  // offset of the slot that holds the ids of key tile t
  static CT_DEVICE int seg_slot(int t) { return kSegRing + (t & 3) * kSegSlotBytes; }
};

template <int D>
struct VkFetcher {
  TileDma<kKeyTile, D / 8, kFwdWaves * 64> dma;
  const char* kbase;
  const char* vbase;
  const int* segb;
  size_t row_stride_bytes;
  CT_DEVICE VkFetcher(const bf16* k, const bf16* v, const int* seg, size_t row_stride_elems)
      : dma(row_stride_elems * 2), kbase(reinterpret_cast<const char*>(k)),
        vbase(reinterpret_cast<const char*>(v)), segb(seg), row_stride_bytes(row_stride_elems * 2) {}
  CT_DEVICE void issue_v(int tile, lds_addr stage) const {
    dma.issue(vbase + (size_t)tile * kKeyTile * row_stride_bytes, stage + VkStage<D>::kV);
  }
  // K rows of `tile` into `stage`, its segment ids into the ring (lds0 = start of LDS)
  CT_DEVICE void issue_k(int tile, lds_addr stage, lds_addr lds0) const {
    dma.issue(kbase + (size_t)tile * kKeyTile * row_stride_bytes, stage + VkStage<D>::kK);
    if (threadIdx.x < 16)  // 64 ids = 16 lanes x 16 bytes, linear layout
      dma16_s(segb + tile * kKeyTile, threadIdx.x * 16, lds0 + VkStage<D>::seg_slot(tile));
  }
  // stage s: V(s), K(s + 1); tiles past `last` are skipped
  CT_DEVICE void issue_stage(int s, int last, lds_addr stage, lds_addr lds0) const {
    if (s <= last) issue_v(s, stage);
    if (s + 1 <= last) issue_k(s + 1, stage, lds0);
  }
  // Stage s = V(s), K(s + 2) as the operands of a statement that issues this wavefront's copies
  // itself. A K tile past `last` is replaced by tile `last` (copied to where nothing reads it):
  // the statement has no branches.
  static constexpr int kPasses = decltype(dma)::kPasses;
  // this thread's offsets and this wavefront's LDS destinations for copies into `stage`
  CT_DEVICE FwdCopies stage_destinations(lds_addr stage) const {
    static_assert(kPasses == 2, "two pieces per tile and wavefront");
    const int wave = uniform(threadIdx.x >> 6);
    FwdCopies c;
#pragma unroll
    for (int n = 0; n < kPasses; ++n) {
      c.lane_off[n] = dma.lane_off[n];
      c.dst[n] = uniform((int)(unsigned)(uintptr_t)(stage + VkStage<D>::kV + (n * kFwdWaves * 64 + wave * 64) * 16));
      c.dst[kPasses + n] =
          uniform((int)(unsigned)(uintptr_t)(stage + VkStage<D>::kK + (n * kFwdWaves * 64 + wave * 64) * 16));
    }
    return c;
  }
  CT_DEVICE FwdCopies stage_copies(int s, int last, lds_addr stage) const {
    const auto scalar64 = [](const char* ptr) {
      const unsigned long long b = (unsigned long long)(uintptr_t)ptr;
      const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)b);
      const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
      return ((unsigned long long)hi << 32) | (unsigned long long)lo;
    };
    FwdCopies c = stage_destinations(stage);
    c.v_source = scalar64(vbase + (size_t)s * kKeyTile * row_stride_bytes);
    c.k_source = scalar64(kbase + (size_t)min(s + 2, last) * kKeyTile * row_stride_bytes);
    return c;
  }
  // the segment ids that go with the K rows of tile s + 2
  CT_DEVICE void issue_ids_two_ahead(int s, int last, lds_addr lds0) const {
    if (s + 2 <= last && threadIdx.x < 16)
      dma16_s(segb + (s + 2) * kKeyTile, threadIdx.x * 16, lds0 + VkStage<D>::seg_slot(s + 2));
  }
};

// What a query tile reads from memory before its first key tile can be fetched, read ahead by the
// tile before it (one workgroup owns the compute unit: nothing else would hide these round
// trips). The bounds are requested at the start of the previous tile, as scalar loads that
// complete with that tile's own; the rows (id, visible end, Q) behind its last key tile.
template <int D, int HS>
struct FwdAhead {
  using Context = QueryTileContext<D, HS, kFwdWaves>;
  int b, qt;
  typename Context::TileBounds bounds;
  int seg_q, end_q;
  RowBlockLoader<D> q_rows;  // whole rows per instruction; they become fragments in the tile's prologue
  // the K rows of the tile's first two key tiles are on their way to the two stages, the V rows of
  // its first key tile to stage 0 (the tile before issued them behind its last key tile)
  bool first_copies_issued = false;
  // key tiles of tile (b, qt), from the bounds
  CT_DEVICE void key_range(const AttnParams& p, int& first, int& last) const {
    constexpr int PB = Context::PB;
    const int nrb = p.S / 32;
    first = INT_MAX;
    last = -1;
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      if (qt * PB + i >= nrb) break;
      first = min(first, uniform(bounds.kv_first[i]));
      last = max(last, uniform(bounds.kv_last[i]));
    }
  }
  CT_DEVICE void request_bounds(const AttnParams& p, int b_, int kvh, int slice, int qt_) {
    b = b_;
    qt = qt_;
    bounds = Context::tile_bounds(p, QueryWork<HS, kFwdWaves>(p, b, kvh, slice, qt));
  }
  // rows of tile (b, qt), as set by request_bounds
  CT_DEVICE void request_rows(const AttnParams& p, int kvh, int slice) {
    const QueryWork<HS, kFwdWaves> work(p, b, kvh, slice, qt);
    // (lane id made opaque: the lane's share of the addresses is rebuilt here instead of being
    // kept in registers across the whole kernel)
    const int l = lane_id_here();
    const size_t position = (size_t)b * p.S + min(work.rb, p.S / 32 - 1) * 32 + (l & 31);
    seg_q = p.seg[position];
    // (always a load: a value formed here instead would first have to wait for the load before
    // it, which may still own the register; the context ignores it without visible ends)
    end_q = (p.end ? p.end : p.seg)[position];
    const size_t first = (size_t)b * p.S + min(work.rb, p.S / 32 - 1) * 32;
    q_rows.request(p.q + (first * p.Hq + work.h) * D, (size_t)p.Hq * D);
  }
};

// One query tile (kFwdWaves / HS row blocks x HS heads of one KV head), start to finish. `ahead`
// holds what this tile read ahead on entry and what tile (batch row next_b, tile next_qt) did on
// return. The request is unconditional (the last tile of a workgroup names itself again): a
// conditional one would keep the old Q registers alive through the whole tile.
template <int D, int HS>
CT_DEVICE void attn_fwd_item_phased(const AttnParams& p, FwdAhead<D, HS>& ahead, int next_b,
                             int next_qt, int kvh, int slice, const lds_addr lds0,
                             const RowFragOffsets<D / 8>& ro,
                             const TrFragOffsets<D / 8, KSlots::kAccum>& to) {
  constexpr int kStage = VkStage<D>::kBytes;
  const QueryTileContext<D, HS, kFwdWaves> ctx(p, ahead.b, kvh, slice, ahead.qt, ahead.bounds, ahead.seg_q,
                                                ahead.end_q);

  const int l = lane_id(), half = l >> 5, w = threadIdx.x >> 6;
  const bool late = uniform(w) >= kFwdWaves / 2;
  const size_t q_row_stride = (size_t)p.Hq * D;
  const size_t kv_row_stride = (size_t)p.Hkv * D;


  f32x16 oacc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db) oacc[db] = zero16();
  float m_run = kNegInf;  // softmax reference (a recent running max), log2 domain
  float l_run = 0.f;      // this lane's share of the running sum (f32: the LSE is held to 1e-3)

  const VkFetcher<D> fetch(ctx.kbase, ctx.vbase, ctx.segb, kv_row_stride);
  int t = ctx.first;
  const int last = ctx.last;
  KeyTileBounds kb = {0, 0, 0}, nb = {0, 0, 0};  // bounds of tiles t and t + 1
  f32x16 s[2];
  bool visit = false;
  if (t <= last) {
    fetch.issue_k(t, lds0 + kStage, lds0);  // stage first - 1 (buffer 1): only its K half
    fetch.issue_stage(t, last, lds0, lds0);  // stage first -> buffer 0
    kb = key_tile_bounds(ctx.meta_b, t);
    if (t + 1 <= last) nb = key_tile_bounds(ctx.meta_b, t + 1);
    visit = ctx.wave_visits(kb, t);
  }
  // the next tile's bounds: scalar loads behind this tile's first copies; nothing here uses them
  ahead.request_bounds(p, next_b, kvh, slice, next_qt);
  // (the Q rows are touched only now: the first copies above needed nothing but the bounds)
  bf16x8 qf[D / 16];
  ahead.q_rows.to_fragments(lds0 + (VkStage<D>::kStorePatches + w * VkStage<D>::kStorePatchBytes), qf);
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) qf[ks] = scale_bf16x8(qf[ks], p.scale);
  dma_wait_all();
  __syncthreads();
  if (visit) scores_t<D>(kStage + VkStage<D>::kK, ro, qf, s);
  if (late) __builtin_amdgcn_s_barrier();

  // The VALU phase of tile t: masks, running maximum and sum, probabilities as bf16 fragments.
  auto softmax_phase = [&](bf16x8* pf) {
    if (visit) {
      float mx = kNegInf;
      {
        // What the summaries leave open for this tile. A key tile with one shared id X turns
        // the id test into a per-query predicate (seg_q == X), which folds into the visible-end
        // bound; only a key tile that mixes ids needs the per-key comparison.
        const int k_uniform = uniform(kb.uniform);
        const bool mixed_keys = k_uniform == 0;
        const bool need_seg = ctx.mine.uniform == 0 || ctx.mine.uniform != k_uniform;
        const bool need_causal = t * kKeyTile + kKeyTile - 1 > ctx.mine.end_min;
        if (need_seg || need_causal) {
          const int seg_cmp = ctx.row_valid() ? ctx.seg_q : -1;
          int last_rel = ctx.end_q - t * kKeyTile - 4 * half;
          if (mixed_keys) {
            mask_scores_t<true, true>(lds0 + VkStage<D>::seg_slot(t), seg_cmp, last_rel, s);
          } else {
            if (seg_cmp != k_uniform) last_rel = -1;  // no key of this tile is visible
            mask_scores_t<false, true>(lds0, seg_cmp, last_rel, s);
          }
        }
      }
#pragma unroll
      for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kbk][r]);
      mx = pair_max(mx) * kLog2e;
      // The running reference m_run only follows the true maximum when that has grown by
      // more than kRescaleSlack (log2 units): probabilities are then at most 2^slack, well
      // inside bf16 / f32 range, the normalisation by the row sum is unchanged, and the
      // accumulator is rescaled on few tiles instead of most.
      if (__any(mx > m_run + kRescaleSlack)) {
        const float m_new = fmaxf(m_run, mx);
        const float m_use = (m_new == kNegInf) ? 0.f : m_new;
        const float alpha = exp2_fast(m_run - m_use);  // m_run = -inf -> 0
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
        m_run = m_new;
      }
      const float m_use = (m_run == kNegInf) ? 0.f : m_run;
      float psum = 0.f;
#pragma unroll
      for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          s[kbk][r] = exp2_fast(fmaf(s[kbk][r], kLog2e, -m_use));
          psum += s[kbk][r];
        }
      l_run += psum;
#pragma unroll
      for (int step4 = 0; step4 < 4; ++step4) pf[step4] = pack_acc8(s[step4 >> 1], step4 & 1);
    }
  };
  // O^T += V^T P^T for the tile in buffer CUR
  auto pv_phase = [&](auto stage_tag, const bf16x8* pf) {
    constexpr int CUR = decltype(stage_tag)::value;
    if constexpr (D == 128) {
      pv_sequence_128<CUR * kStage + VkStage<D>::kV>(to, pf, oacc);
    } else {
#pragma unroll
      for (int step4 = 0; step4 < 4; ++step4)
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
          oacc[db] = mfma32(to.load(CUR * kStage + VkStage<D>::kV, step4, db), pf[step4], oacc[db]);
    }
  };

  // One step = VALU phase + MFMA phase of tile t < last; CUR is the buffer of stage t.
  auto step = [&](auto stage_tag) {
    constexpr int CUR = decltype(stage_tag)::value;
    const lds_addr next_stage = lds0 + (CUR ^ 1) * kStage;
    // ---- VALU phase ----
    if (late) fetch.issue_stage(t + 1, last, next_stage, lds0);
    // bounds of tile t + 2: requested now, first needed one step from now
    KeyTileBounds nnb = nb;
    if (t + 2 <= last) nnb = key_tile_bounds(ctx.meta_b, t + 2);
    bf16x8 pf[4];
    softmax_phase(pf);
    if (!late) dma_wait_all();  // stage t, issued one step ago
    __builtin_amdgcn_s_barrier();
    // ---- MFMA phase ----
    if (!late) fetch.issue_stage(t + 1, last, next_stage, lds0);
    const bool visit_next = ctx.wave_visits(nb, t + 1);
    if (visit) pv_phase(stage_tag, pf);
    if constexpr (D == 128) {
      if (visit_next) qk_sequence_128<CUR * kStage + VkStage<D>::kK>(ro, qf, s);
    } else {
      if (visit_next) scores_t<D>(CUR * kStage + VkStage<D>::kK, ro, qf, s);
    }
    if (late) dma_wait_all();  // stage t + 1, issued at the start of this step
    __builtin_amdgcn_s_barrier();
    visit = visit_next;
    kb = nb;
    nb = nnb;
    ++t;
  };
  const bool any_tile = t <= last;
  while (t < last) {
    step(std::integral_constant<int, 0>{});
    if (t >= last) break;
    step(std::integral_constant<int, 1>{});
  }
  // The step of the last tile: nothing to fetch and no scores to form, so the Q registers are
  // free, and no later wait of this tile is a wait for memory: the next tile's rows are requested
  // behind the last such wait and land under the PV product, the stores of O and the next
  // tile's first copies. (One call site for every path: several would meet in register copies
  // that wait for the loads.)
  bf16x8 pf[4];
  if (any_tile) {
    softmax_phase(pf);
    if (!late) dma_wait_all();  // stage t, issued one step ago
    __builtin_amdgcn_s_barrier();
  }
  ahead.request_rows(p, kvh, slice);
  if (any_tile) {
    if (visit) {
      if (((last - ctx.first) & 1) == 0)
        pv_phase(std::integral_constant<int, 0>{}, pf);
      else
        pv_phase(std::integral_constant<int, 1>{}, pf);
    }
    __builtin_amdgcn_s_barrier();
  }
  if (!late) __builtin_amdgcn_s_barrier();
  // Every copy of this tile has been waited for by the wavefronts that issued it, so only LDS
  // traffic has to settle before the stages become store patches (a wait for memory here would
  // wait for the next tile's loads).
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();

  const float l_tot = pair_sum(l_run);
  const bool has = l_tot > 0.f;
  const float inv = has ? 1.f / l_tot : 0.f;
  if (ctx.active) {
    const int le = lane_id_here();
    const size_t stat = ((size_t)ctx.work.b * p.S + ctx.work.rb * 32 + (le & 31)) * p.Hq + ctx.work.h;
    if (le < 32) p.lse[stat] = has ? (__logf(l_tot) + m_run * kLn2) : 0.f;
    const lds_addr patch = lds0 + w * 32 * D * 2;
    bf16* obase = p.out + (((size_t)ctx.work.b * p.S + ctx.work.rb * 32) * p.Hq + ctx.work.h) * D;
    store_rows_t<D>(oacc, inv, patch, obase, q_row_stride);
  }
  // The store patches overlap the stages of the next item: its copies may start once every
  // wavefront has read its patch back (LDS reads only; the global stores stay in flight).
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();
}

// store_rows_t for the accumulator in a[0:63] (D = 128), one 32-column block in registers at a time.
CT_DEVICE void fwd_store_rows(float row_scale, lds_addr patch, bf16* gbase, size_t row_stride) {
  constexpr int D = 128, CPR = D / 8;
  int l = lane_id();
  asm volatile("" : "+v"(l));  // (as in store_rows_t: the patch addresses are formed here)
  const int j = l & 31, half = l >> 5;
  using Patch = PatchRows<D>;
  const lds_addr store_base = Patch::store_base(patch, j, half);
  const unsigned row_swizzle = Patch::row_swizzle(j);
  auto block = [&](auto db_tag) {
    constexpr int db = decltype(db_tag)::value;
    const f32x16 acc = fwd_acc_read<db>();
    auto quad = [&](auto qd_tag) {
      constexpr int qd = decltype(qd_tag)::value;
      bf16x4 pk;
#pragma unroll
      for (int e = 0; e < 4; ++e) pk[e] = (bf16)(acc[4 * qd + e] * row_scale);
      lds_store<bf16x4>(store_base + Patch::template chunk_term<db * 4 + qd>(row_swizzle), pk);
    };
    quad(std::integral_constant<int, 0>{});
    quad(std::integral_constant<int, 1>{});
    quad(std::integral_constant<int, 2>{});
    quad(std::integral_constant<int, 3>{});
  };
  block(std::integral_constant<int, 0>{});
  block(std::integral_constant<int, 1>{});
  block(std::integral_constant<int, 2>{});
  block(std::integral_constant<int, 3>{});
  (void)CPR;
  __builtin_amdgcn_wave_barrier();
  Patch::to_global(patch, l, gbase, row_stride);
}

// One query tile, interleaved form (D = 128). Arguments as attn_fwd_item_phased.
template <int D, int HS>
CT_DEVICE void attn_fwd_item(const AttnParams& p, FwdAhead<D, HS>& ahead, int next_b,
                             int next_qt, bool more, int kvh, int slice, const lds_addr lds0,
                             const RowFragOffsets<D / 8>& ro,
                             const TrFragOffsets<D / 8, KSlots::kAccum>& to) {
  static_assert(D == 128, "the interleaved statements are written for D = 128");
  constexpr int kStage = VkStage<D>::kBytes;
  constexpr int kV = VkStage<D>::kV, kK = VkStage<D>::kK;
  const QueryTileContext<D, HS, kFwdWaves> ctx(p, ahead.b, kvh, slice, ahead.qt, ahead.bounds, ahead.seg_q,
                                                ahead.end_q);

  const int w = threadIdx.x >> 6;
  const size_t q_row_stride = (size_t)p.Hq * D;
  const size_t kv_row_stride = (size_t)p.Hkv * D;

  float m_run = kNegInf;  // softmax reference (a recent running max), log2 domain
  float l_run = 0.f;      // this lane's share of the running sum (f32: the LSE is held to 1e-3)

  const VkFetcher<D> fetch(ctx.kbase, ctx.vbase, ctx.segb, kv_row_stride);
  int t = ctx.first;
  const int last = ctx.last;
  const bool any_tile = t <= last;
  const bool k_rows_on_their_way = ahead.first_copies_issued;
  KeyTileBounds kb = {0, 0, 0}, nb = {0, 0, 0};  // bounds of tiles t and t + 1
  bool visit = false;       // does this wavefront see tile t (its scores are in the buffer of t)
  bool visit_prev = false;  // ... tile t - 1 (P^T in the other buffer, PV product still to do)
  if (any_tile) {
    // K rows of the first two tiles (they belong to stages first - 2 and first - 1), and the V rows
    // of the first: its place in stage `first` is free already, only the K half of that stage has
    // to wait until K(first) has been read
    // (a query tile that follows another in this workgroup had its K rows copied by that one)
    if (!k_rows_on_their_way) {
      fetch.issue_k(t, lds0, lds0);
      if (t + 1 <= last) fetch.issue_k(t + 1, lds0 + kStage, lds0);
      fetch.issue_v(t, lds0);
    }
    kb = key_tile_bounds(ctx.meta_b, t);
    if (t + 1 <= last) nb = key_tile_bounds(ctx.meta_b, t + 1);
    visit = ctx.wave_visits(kb, t);
  }
  // Which of the 64 tiles from `chart_base` on this wavefront sees (bit j of `seen`: tile
  // chart_base + j) and sees in full, without a mask (`plain`): lane j looks at tile chart_base + j.
  int chart_base = 0;
  unsigned long long seen = 0, plain = 0;
  auto chart = [&](int base) {
    chart_base = base;
    const int tj = base + lane_id_here();
    bool sees = false, full = false;
    if (tj >= ctx.first && tj <= last) {
      const int* a = ctx.meta_b + (size_t)(2 * tj) * kMetaW;
      const int* c = a + kMetaW;
      const int a_min = a[kMinNz], c_min = c[kMinNz];
      const int k_min = a_min == 0 ? c_min : (c_min == 0 ? a_min : min(a_min, c_min));
      const int k_max = max(a[kMaxId], c[kMaxId]);
      const int k_uniform = (a[kUniform] == c[kUniform]) ? a[kUniform] : 0;
      sees = blocks_interact(ctx.mine.min_nz, ctx.mine.max_id, ctx.mine.end_max, k_min, k_max, tj * kKeyTile);
      const bool need_seg = ctx.mine.uniform == 0 || ctx.mine.uniform != k_uniform;
      const bool need_causal = tj * kKeyTile + kKeyTile - 1 > ctx.mine.end_min;
      full = sees && !need_seg && !need_causal;
    }
    seen = __ballot(sees);
    plain = __ballot(full);
  };
  // (charted here: its loads travel with the first copies)
  if (any_tile) chart(t - 1);
  // the next tile's bounds: scalar loads behind this tile's first copies; nothing here uses them
  ahead.request_bounds(p, next_b, kvh, slice, next_qt);
  // (the Q rows are touched only now: the first copies above needed nothing but the bounds)
  bf16x8 qf[D / 16];
  ahead.q_rows.to_fragments(lds0 + (VkStage<D>::kStorePatches + w * VkStage<D>::kStorePatchBytes), qf);
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) qf[ks] = scale_bf16x8(qf[ks], p.scale);
  dma_wait_all();
  __syncthreads();
  // Every wavefront is past the last PV product of the query tile before: the V rows of this one's
  // first key tile may take their place (first read one step from now, behind that step's wait).
  if (any_tile && k_rows_on_their_way) fetch.issue_v(t, lds0);
  // (statement "b" writes buffer a: the first tile counts even; the output accumulator is cleared
  // behind its MFMAs, or on its own where this wavefront does not see the first tile)
  if (visit) fwd_qk_zero_b<kK>(ro, qf);
  else fwd_acc_zero();
  // every wavefront has read K(first): the first step's copies may replace it
  __builtin_amdgcn_s_barrier();

  // The running reference m_run only follows the true maximum when that has grown by more than
  // kRescaleSlack (log2 units): probabilities are then at most 2^slack, well inside bf16 / f32
  // range, the normalisation by the row sum is unchanged, and the accumulator is rescaled on few
  // tiles instead of most.
  auto must_rescale = [&](float mx) { return __any(mx > m_run + kRescaleSlack) != 0; };
  auto rescale = [&](float mx) {
    const float m_new = fmaxf(m_run, mx);
    const float m_use = (m_new == kNegInf) ? 0.f : m_new;
    const float alpha = exp2_fast(m_run - m_use);  // m_run = -inf -> 0
    l_run *= alpha;
    // (rows without a finite reference have seen no key yet: their sums are still zero, and on a
    // query tile's first key tile that is every row)
    if (__any(m_run != kNegInf)) fwd_acc_scale(alpha);
    m_run = m_new;
  };

  // The step of tile t. PARITY = (t - first) & 1: the scores of tile t are in buffer a (0) or b
  // (1), stage t - 1 (V(t - 1), K(t + 1)) is in LDS buffer 1 - PARITY, stage t goes to PARITY.
  auto step = [&](auto parity_tag) {
    constexpr int PARITY = decltype(parity_tag)::value;
    constexpr int V_OFF = (1 - PARITY) * kStage + kV, K_OFF = (1 - PARITY) * kStage + kK;
    const bool visit_next = t < last && ctx.wave_visits(nb, t + 1);
    // the copies of stage t: inside the first statement where the step runs the interleaved ones
    const bool interleaved = visit_prev && visit && visit_next;
    if (interleaved) {
      fetch.issue_ids_two_ahead(t, last, lds0);
    } else {
      if (t != ctx.first) fetch.issue_v(t, lds0 + PARITY * kStage);  // (V(first) went with the first copies)
      if (t + 2 <= last) fetch.issue_k(t + 2, lds0 + PARITY * kStage, lds0);
    }

    if (visit) {
      // Masks: what the summaries leave open for this tile. A key tile with one shared id X turns
      // the id test into a per-query predicate (seg_q == X), which folds into the visible-end
      // bound; only a key tile that mixes ids needs the per-key comparison.
      const int k_uniform = uniform(kb.uniform);
      const bool need_seg = ctx.mine.uniform == 0 || ctx.mine.uniform != k_uniform;
      const bool need_causal = t * kKeyTile + kKeyTile - 1 > ctx.mine.end_min;
      if (need_seg || need_causal) {
        const int seg_cmp = ctx.row_valid() ? ctx.seg_q : -1;
        if (k_uniform == 0) {
          // the ids of the tile's keys against the row's (-1 for a padding row matches none), then,
          // where the tile reaches past the smallest visible end, the keys' offsets against the row's end
          const int half = lane_id_here() >> 5;
          const lds_addr ids = lds0 + (VkStage<D>::seg_slot(t) + 16 * half);
          if constexpr (PARITY == 0) fwd_mask_ids_a(ids, seg_cmp);
          else fwd_mask_ids_b(ids, seg_cmp);
          if (need_causal) {
            const int rel = ctx.end_q - t * kKeyTile - 4 * half;
            if constexpr (PARITY == 0) fwd_mask_causal_a(rel);
            else fwd_mask_causal_b(rel);
          }
        } else {
          // (no key of this tile is visible to a query of another id)
          const int rel = seg_cmp != k_uniform ? -1 : ctx.end_q - t * kKeyTile - 4 * (lane_id_here() >> 5);
          if constexpr (PARITY == 0) fwd_mask_causal_a(rel);
          else fwd_mask_causal_b(rel);
        }
      }
    }

    if (interleaved) {
      const auto copies = fetch.stage_copies(t, last, lds0 + PARITY * kStage);
      float mx;
      if constexpr (PARITY == 0) mx = fwd_max_a<V_OFF>(to, copies);
      else mx = fwd_max_b<V_OFF>(to, copies);
      if (must_rescale(mx)) {
        if constexpr (PARITY == 0) fwd_pv_late_a<V_OFF>(to);
        else fwd_pv_late_b<V_OFF>(to);
        rescale(mx);
        const float m_use = (m_run == kNegInf) ? 0.f : m_run;
        float psum = 0.f;
        if constexpr (PARITY == 0) {
          fwd_exp_only_a(m_use, psum);
          fwd_qk_a<K_OFF>(ro, qf);
        } else {
          fwd_exp_only_b(m_use, psum);
          fwd_qk_b<K_OFF>(ro, qf);
        }
        l_run += psum;
      } else {
        const float m_use = (m_run == kNegInf) ? 0.f : m_run;
        float psum = 0.f;
        if constexpr (PARITY == 0) {
          fwd_exp_a_a<V_OFF>(to, m_use, psum);
          fwd_exp_b_a<K_OFF>(ro, qf, m_use, psum);
        } else {
          fwd_exp_a_b<V_OFF>(to, m_use, psum);
          fwd_exp_b_b<K_OFF>(ro, qf, m_use, psum);
        }
        l_run += psum;
      }
    } else {
      if (visit_prev) {
        if constexpr (PARITY == 0) fwd_pv_a<V_OFF>(to);
        else fwd_pv_b<V_OFF>(to);
      }
      if (visit) {
        float mx;
        if constexpr (PARITY == 0) mx = fwd_max_only_a();
        else mx = fwd_max_only_b();
        if (must_rescale(mx)) rescale(mx);
        const float m_use = (m_run == kNegInf) ? 0.f : m_run;
        float psum = 0.f;
        if constexpr (PARITY == 0) fwd_exp_only_a(m_use, psum);
        else fwd_exp_only_b(m_use, psum);
        l_run += psum;
      }
      if (visit_next) {
        if constexpr (PARITY == 0) fwd_qk_a<K_OFF>(ro, qf);
        else fwd_qk_b<K_OFF>(ro, qf);
      }
    }
    // bounds of tile t + 2, first needed one step from now: requested here, as loaded, so that the
    // scalar loads complete under the two waits below instead of in front of the next statement
    // (every statement starts by waiting for the wavefront's LDS and scalar loads)
    KeyTileWords ahead_words = key_tile_words_request(ctx.meta_b, min(t + 2, last));
    dma_wait_all();  // stage t
    __builtin_amdgcn_s_barrier();
    key_tile_words_wait(ahead_words);
    visit_prev = visit;
    visit = visit_next;
    kb = nb;
    nb = key_tile_bounds(ahead_words);
    ++t;
  };
  // A step without decisions, for a stretch of tiles that this wavefront sees in full (no masks)
  // between two tiles that it sees: what step() works out per tile (bounds, who sees what, which
  // masks) is known for the whole stretch, and its scalar work, about 150 instructions that both
  // wavefronts of a SIMD run at the same time while the matrix pipe waits, shrinks to the copy
  // sources and the loop count.
  unsigned long long v_source = 0, k_source = 0;  // sources of the copies of the plain step of tile t
  const unsigned long long tile_bytes = (unsigned long long)kKeyTile * kv_row_stride * 2;
  auto plain_step = [&](auto parity_tag) {
    constexpr int PARITY = decltype(parity_tag)::value;
    constexpr int V_OFF = (1 - PARITY) * kStage + kV, K_OFF = (1 - PARITY) * kStage + kK;
    fetch.issue_ids_two_ahead(t, last, lds0);
    auto copies = fetch.stage_destinations(lds0 + PARITY * kStage);
    copies.v_source = v_source;
    copies.k_source = k_source;
    float mx;
    if constexpr (PARITY == 0) mx = fwd_max_a<V_OFF>(to, copies);
    else mx = fwd_max_b<V_OFF>(to, copies);
    if (must_rescale(mx)) {
      if constexpr (PARITY == 0) fwd_pv_late_a<V_OFF>(to);
      else fwd_pv_late_b<V_OFF>(to);
      rescale(mx);
      const float m_use = (m_run == kNegInf) ? 0.f : m_run;
      float psum = 0.f;
      if constexpr (PARITY == 0) {
        fwd_exp_only_a(m_use, psum);
        fwd_qk_a<K_OFF>(ro, qf);
      } else {
        fwd_exp_only_b(m_use, psum);
        fwd_qk_b<K_OFF>(ro, qf);
      }
      l_run += psum;
    } else {
      const float m_use = (m_run == kNegInf) ? 0.f : m_run;
      float psum = 0.f;
      if constexpr (PARITY == 0) {
        fwd_exp_a_a<V_OFF>(to, m_use, psum);
        fwd_exp_b_a<K_OFF>(ro, qf, m_use, psum);
      } else {
        fwd_exp_a_b<V_OFF>(to, m_use, psum);
        fwd_exp_b_b<K_OFF>(ro, qf, m_use, psum);
      }
      l_run += psum;
    }
    v_source += tile_bytes;
    if (t + 3 <= last) k_source += tile_bytes;  // (the K tile two ahead of the next step, held at `last`)
    dma_wait_all();  // stage t
    __builtin_amdgcn_s_barrier();
    ++t;
  };


  while (t <= last) {
    // a stretch of plain steps from tile t on: tiles u with u - 1 seen, u plain, u + 1 seen
    if (t - chart_base >= 63) chart(t - 1);
    const unsigned long long stretch = ((seen << 1) & plain & (seen >> 1)) >> (t - chart_base);
    int n = (int)__builtin_ctzll(~stretch);
    if (n > 0) {
      v_source = (unsigned long long)(uintptr_t)(fetch.vbase + (size_t)t * tile_bytes);
      k_source = (unsigned long long)(uintptr_t)(fetch.kbase + (size_t)min(t + 2, last) * tile_bytes);
      if (((t - ctx.first) & 1) != 0) {
        plain_step(std::integral_constant<int, 1>{});
        --n;
      }
      for (; n >= 2; n -= 2) {
        plain_step(std::integral_constant<int, 0>{});
        plain_step(std::integral_constant<int, 1>{});
      }
      if (n != 0) plain_step(std::integral_constant<int, 0>{});
      // back to the general step: tile t - 1 and tile t are seen, and their bounds are read again
      visit_prev = true;
      visit = true;
      kb = key_tile_bounds(ctx.meta_b, t);
      nb = key_tile_bounds(ctx.meta_b, min(t + 1, last));
      continue;
    }
    if (((t - ctx.first) & 1) == 0) step(std::integral_constant<int, 0>{});
    else step(std::integral_constant<int, 1>{});
  }
  // What is left is the PV product of the last tile, and no later wait of this query tile is a
  // wait for memory. Every wavefront is past its last read of K rows, so the next query tile's
  // first two K tiles can take their places in the stages now, and its rows are requested behind
  // them: all of that lands under the last product and the stores of O. (`ahead` names the next
  // tile since the prologue. Its V rows wait for the barrier in its own prologue: until then a
  // wavefront may still read this tile's.)
  ahead.first_copies_issued = false;
  if (more) {
    int next_first, next_last;
    ahead.key_range(p, next_first, next_last);
    if (next_first <= next_last) {
      VkFetcher<D> next_fetch = fetch;
      next_fetch.kbase = reinterpret_cast<const char*>(p.k + ((size_t)ahead.b * p.S * p.Hkv + kvh) * D);
      next_fetch.segb = p.seg + (size_t)ahead.b * p.S;
      next_fetch.issue_k(next_first, lds0, lds0);
      if (next_first + 1 <= next_last) next_fetch.issue_k(next_first + 1, lds0 + kStage, lds0);
      ahead.first_copies_issued = true;
    }
  }
  ahead.request_rows(p, kvh, slice);
  if (any_tile && visit_prev) {
    // stage `last` is in LDS buffer (last - first) & 1, P^T(last) in the score buffer of that
    // parity: the statement that reads it is the one of the opposite name
    if (((last - ctx.first) & 1) == 0) fwd_pv_b<kV>(to);
    else fwd_pv_a<kStage + kV>(to);
  }

  const float l_tot = pair_sum(l_run);
  const bool has = l_tot > 0.f;
  const float inv = has ? 1.f / l_tot : 0.f;
  if (ctx.active) {
    const int le = lane_id_here();
    const size_t stat = ((size_t)ctx.work.b * p.S + ctx.work.rb * 32 + (le & 31)) * p.Hq + ctx.work.h;
    if (le < 32) p.lse[stat] = has ? (__logf(l_tot) + m_run * kLn2) : 0.f;
    // (the patch is this wavefront's alone: its next use, one query tile on, follows these reads
    // in the wavefront's own order, so no barrier closes the tile)
    const lds_addr patch = lds0 + (VkStage<D>::kStorePatches + w * VkStage<D>::kStorePatchBytes);
    bf16* obase = p.out + (((size_t)ctx.work.b * p.S + ctx.work.rb * 32) * p.Hq + ctx.work.h) * D;
    fwd_store_rows(inv, patch, obase, q_row_stride);
  }
}

// Workgroup (group, bin): walks the query tiles of one work bin for one
// (head slice, KV head) group. The group is the fast index, so with 8 groups a
// group stays on one XCD (workgroup ids are dealt round robin to the 8 XCDs)
// and its K/V rows stay in that XCD's L2.
template <int D, int HS>
__global__ __launch_bounds__(kFwdWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void
attn_fwd_kernel(AttnParams p) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr lds0 = lds_address_of(smem_raw);
  constexpr int PB = kFwdWaves / HS;
  const RowFragOffsets<D / 8> ro(lds0);
  const TrFragOffsets<D / 8, KSlots::kAccum> to(lds0);
  const int nrb = p.S / 32;
  const int slices = (p.Hq / p.Hkv) / HS;
  const int groups = slices * p.Hkv;
  const int group = blockIdx.x % groups, bin = blockIdx.x / groups;
  const int kvh = group % p.Hkv, slice = group / p.Hkv;
  const MetaPtr region = meta_const(p.meta + bin_region_offset(p.B, nrb, PB));
  const int tpr = bin_tiles_per_row(nrb, PB);
  const int it_end = uniform(region[bin + 1]);
  int it = uniform(region[bin]);
  if (it >= it_end) return;
  FwdAhead<D, HS> ahead;
  {
    const int item = uniform(region[kBins + 1 + it]);
    ahead.request_bounds(p, item / tpr, kvh, slice, item % tpr);
    ahead.request_rows(p, kvh, slice);
  }
  for (; it < it_end; ++it) {
    const int next_item = uniform(region[kBins + 1 + min(it + 1, it_end - 1)]);
    if constexpr (D == 128)
      attn_fwd_item<D, HS>(p, ahead, next_item / tpr, next_item % tpr, it + 1 < it_end, kvh, slice, lds0, ro, to);
    else
      attn_fwd_item_phased<D, HS>(p, ahead, next_item / tpr, next_item % tpr, kvh, slice, lds0, ro, to);
  }
}

// ---------------------------------------------------------------------------
// delta[row] = sum_d f32(out[row, d]) * f32(dout[row, d])      (HBM bound)
// One 16-byte load per lane per tensor; D/8 lanes share a row; rows are (b, s, h) flattened.
// The backward does not launch this kernel: its dQ kernel computes delta for the rows of each
// query tile from the dO fragments it loads anyway (one read of `out` instead of a pass over
// `out` and `dout`). This is the pass on its own, behind ct_attn_delta.
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_delta_kernel(const bf16* out, const bf16* dout,
                                                         float* delta, long rows) {
  // A workgroup walks tiles of kUnroll x 256 sixteen-byte chunks with a grid stride; a thread
  // issues the 2 x kUnroll loads of its chunks before it touches any of them, so that every
  // wavefront keeps 8 KB in flight (a pass that streams from HBM is bound by bytes in flight,
  // not by arithmetic). The operands are read once: loaded with the non-temporal hint.
  constexpr int LPR = D / 8;     // lanes per row
  constexpr int kUnroll = 4;
  const long chunks = rows * LPR;
  const long tile = 256L * kUnroll;
  for (long base = (long)blockIdx.x * tile; base < chunks; base += (long)gridDim.x * tile) {
    u32x4 a[kUnroll], g[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const long chunk = base + k * 256 + threadIdx.x;
      if (chunk < chunks) {
        a[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(out) + chunk);
        g[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(dout) + chunk);
      } else {
        a[k] = u32x4{0u, 0u, 0u, 0u};
        g[k] = u32x4{0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const long chunk = base + k * 256 + threadIdx.x;
      const bf16x8 av = as_bf16x8(a[k]), gv = as_bf16x8(g[k]);
      float acc = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += (float)av[e] * (float)gv[e];
#pragma unroll
      for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
      if (chunk < chunks && chunk % LPR == 0) delta[chunk / LPR] = acc;
    }
  }
}

// The same pass in the form the backward needs when its dK/dV kernel runs first: -delta and
// -lse / scale, both head-major [B, Hq, S] (the dK/dV kernels add them to their dP and S blocks).
// A workgroup takes 4 x (256 / lanes per row) consecutive positions of one head; consecutive
// workgroups take the heads of the same positions, so the rows in flight at a time are one
// contiguous stretch of `out` and `dout`.
template <int D>
__global__ __launch_bounds__(256) void attn_bwd_stats_kernel(const bf16* out, const bf16* dout,
                                                             const float* lse, float* neg_delta,
                                                             float* neg_lse_scaled, int B, int S,
                                                             int Hq, float exponent_scale) {
  constexpr int LPR = D / 8;          // lanes per row
  constexpr int RPP = 256 / LPR;      // rows per pass of the workgroup
  constexpr int kUnroll = 4;
  constexpr int kTile = kUnroll * RPP;  // 64 (D = 128) or 128 (D = 64) positions: divides S
  const int tiles_per_row = S / kTile;
  const long tiles = (long)B * tiles_per_row * Hq;
  const int r0 = threadIdx.x / LPR, chunk = threadIdx.x % LPR;
  for (long tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int h = (int)(tile % Hq);
    const long rest = tile / Hq;
    const int st = (int)(rest % tiles_per_row), b = (int)(rest / tiles_per_row);
    u32x4 a[kUnroll], g[kUnroll];
    float row_lse[kUnroll];
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const size_t row = ((size_t)b * S + st * kTile + r0 + k * RPP) * Hq + h;
      a[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(out) + row * LPR + chunk);
      g[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(dout) + row * LPR + chunk);
      row_lse[k] = lse[row];
    }
#pragma unroll
    for (int k = 0; k < kUnroll; ++k) {
      const bf16x8 av = as_bf16x8(a[k]), gv = as_bf16x8(g[k]);
      float acc = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += (float)av[e] * (float)gv[e];
#pragma unroll
      for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
      if (chunk == 0) {
        const size_t stat = ((size_t)b * Hq + h) * S + st * kTile + r0 + k * RPP;
        neg_delta[stat] = -acc;
        neg_lse_scaled[stat] = -row_lse[k] / exponent_scale;
      }
    }
  }
}

}  // namespace ct
