// Attention backward kernels for gfx950.
//
// dQ kernel: same walk as the forward (a wavefront owns 32 query rows and
// visits the 64-key tiles they can see). Per tile, transposed:
//   S^T = K Q^T, P^T = exp(S^T - lse), dP^T = V dO^T, dS^T = P^T (dP^T - delta),
//   dQ^T += K^T dS^T                      (src/kernels/efficient_attention.py:1015-1048)
// dK/dV kernel: a workgroup owns 128 keys of one KV head (32 per wavefront,
// K and V fragments held in registers) and walks every (query head of the
// group, 32-row query block) that can see them; Q (pre-scaled, bf16) and dO
// are staged through LDS. Per block:
//   S = Q K^T, P = exp(S - lse), dP = dO V^T, dS = P (dP - delta),
//   dV += P^T dO, dK += dS^T Q_scaled      (:1294-1343)
// Every output tile has a single owner: no atomics, fixed summation order.
#pragma once

#include "ct_attn_kernels.hip.h"

namespace ct {

// ---------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------
// Fragment address structures of the backward kernels: the register-lean ones where the tile
// is wide enough for them (both kernels are at the register limit).
template <int D>
using LeanRowFrags = std::conditional_t<(D / 8 >= 16), RowFragCompact<D / 8>, RowFragOffsets<D / 8>>;
template <int D>
using LeanTrFrags = std::conditional_t<(D / 8 >= 16), TrFragCompact<D / 8, KSlots::kAccum>,
                                       TrFragOffsets<D / 8, KSlots::kAccum>>;

// The dK/dV kernels work on unscaled Q K^T and put the softmax scale into the exponent. Any finite
// scale is legal (the operator only asks for a finite one): a scale too small for lse / scale to
// stay finite (|scale| < 1e-30, zero included) is replaced there by 1e-30, for which scale * S
// vanishes against lse in f32 all the same (dK is still multiplied by the true scale), and a
// masked pair is marked by the infinity that the sign of the exponent's scale turns into -inf.
__host__ __device__ inline float exponent_scale(float scale) {
  return (scale < 1e-30f && scale > -1e-30f) ? 1e-30f : scale;
}
CT_DEVICE float masked_score(float scale) { return exponent_scale(scale) < 0.f ? -kNegInf : kNegInf; }

// P = exp2(S log2e - lse2), dS = P (dP - delta) for one 32-key block, in place in s.
CT_DEVICE void dq_arith(f32x16& s, const f32x16& dp, float lse2, float delta_q) {
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float prob = exp2_fast(fmaf(s[r], kLog2e, -lse2));
    s[r] = prob * (dp[r] - delta_q);
  }
}

// One query tile (4 / HS row blocks x HS heads of one KV head), start to finish.
template <int D, int HS>
CT_DEVICE void attn_dq_item(const AttnParams& p, int b, int kvh, int slice, int qt, const lds_addr lds_base) {
  constexpr int kStage = KvStage<D>::kBytes;
  // (the fragment pointers are rebuilt per item from an opaque base: kept across the item loop
  // they end up spilled and reloaded in the key-tile loop)
  lds_addr lds0 = lds_base;
  asm volatile("" : "+v"(lds0));
  const LeanRowFrags<D> ro(lds0);
  const LeanTrFrags<D> to(lds0);

  const QueryTileContext<D, HS> ctx(p, b, kvh, slice, qt);
  const int l = lane_id(), half = l >> 5, w = threadIdx.x >> 6;
  const size_t q_row_stride = (size_t)p.Hq * D;
  const size_t kv_row_stride = (size_t)p.Hkv * D;
  const size_t stat_t = ((size_t)ctx.work.b * p.Hq + ctx.work.h) * p.S + ctx.pos;  // head-major
  const float lse2 = p.lse[ctx.stat_off] * kLog2e;

  // The first key tile's copies go first (stage 0), the rows of Q, dO and O behind them; their
  // way into fragments leads through this wavefront's patch in stage 1, which nothing uses yet.
  const KvFetcher<D> fetch(ctx.kbase, ctx.vbase, ctx.segb, kv_row_stride);
  int t = ctx.first;
  KeyTileBounds kb = {0, 0, 0};
  if (t <= ctx.last) {
    fetch.issue(t, lds0);
    kb = key_tile_bounds(ctx.meta_b, t);
  }
  bf16x8 qf[D / 16], dof[D / 16];
  u32x4 of[D / 16];  // this row's half of `out`, for delta
  {
    const size_t block_off = (((size_t)ctx.work.b * p.S + ctx.work.rb * 32) * p.Hq + ctx.work.h) * D;
    const lds_addr patch = lds0 + kStage + uniform(w) * 32 * D * 2;
    RowBlockLoader<D> q_rows, do_rows, o_rows;
    q_rows.request(p.q + block_off, q_row_stride);
    do_rows.request(p.dout + block_off, q_row_stride);
    o_rows.request(p.out + block_off, q_row_stride);
    q_rows.to_fragments(patch, qf);
    do_rows.to_fragments(patch, dof);
    o_rows.to_fragments(patch, of);
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) qf[ks] = scale_bf16x8(qf[ks], p.scale);
  }
  f32x16 dqacc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db) dqacc[db] = zero16();
  dma_wait_all();
  __syncthreads();

  // delta = sum_d out[row, d] * dout[row, d], after the wait above so that the first key tile's
  // copies are not held back behind these loads; the dK/dV kernel, launched after this one, reads
  // delta and lse * log2(e) head-major
  float delta_part = 0.f;
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    u32x4 o_bits = of[ks];
    asm volatile("" : "+v"(o_bits));
    const u32x4 do_bits = __builtin_bit_cast(u32x4, dof[ks]);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      delta_part = fmaf(__uint_as_float(o_bits[e] << 16), __uint_as_float(do_bits[e] << 16), delta_part);
      delta_part = fmaf(__uint_as_float(o_bits[e] & 0xffff0000u), __uint_as_float(do_bits[e] & 0xffff0000u),
                        delta_part);
    }
  }
  const float delta_q = pair_sum(delta_part);
  if (ctx.active && half == 0) {
    // for the dK/dV kernel: the values it adds to its S and dP blocks, P = exp2((S - lse / scale) *
    // scale * log2(e)) and dS = P (dP - delta)
    p.delta[stat_t] = -delta_q;
    p.lse2[stat_t] = -p.lse[ctx.stat_off] / exponent_scale(p.scale);
  }

  auto step = [&](auto stage_tag) {
    constexpr int CUR = decltype(stage_tag)::value;
    const lds_addr stage = lds0 + CUR * kStage;
    const bool more = t + 1 <= ctx.last;
    KeyTileBounds nb = kb;
    if (more) {
      fetch.issue(t + 1, lds0 + (CUR ^ 1) * kStage);
      nb = key_tile_bounds(ctx.meta_b, t + 1);
    }
    if (ctx.wave_visits(kb, t)) {
      // Same specialisation as the forward: masked scores become -inf, so their
      // probability exp2(-inf) is exactly 0 and so is dS.
      const int k_uniform = uniform(kb.uniform);
      const bool need_seg = ctx.mine.uniform == 0 || ctx.mine.uniform != k_uniform;
      const bool need_causal = t * kKeyTile + kKeyTile - 1 > ctx.mine.end_min;
      const int seg_cmp = ctx.row_valid() ? ctx.seg_q : -1;
      int last_rel = ctx.end_q - t * kKeyTile - 4 * half;
      if (k_uniform != 0 && seg_cmp != k_uniform) last_rel = -1;
      constexpr int kOff = CUR * kStage + KvStage<D>::kK, vOff = CUR * kStage + KvStage<D>::kV;
      if constexpr (D == 128) {
        // The tile is worked in its two 32-key halves, each start to finish (S and dP, the
        // arithmetic, the half's share of dQ): 32 score registers are live at a time instead of
        // 64, which is what leaves room for the fragment ring of the hand-scheduled sequences
        // without spilling registers inside this loop.
        const RowFragOffsets<16> rp = RowFragOffsets<16>::expand(ro);
        const TrFragOffsets<16, KSlots::kAccum> tp =
            TrFragOffsets<16, KSlots::kAccum>::expand(TrFragCompact<16, KSlots::kAccum>(lds_base, lane_id_here()));
        auto half_tile = [&](auto kb_tag) {
          constexpr int KB = decltype(kb_tag)::value;
          f32x16 s, dp;
          dq_sdp_half_128<kOff + KB * 8192, vOff + KB * 8192>(rp, qf, dof, s, dp);
          if (need_seg || need_causal) {
            if (k_uniform == 0) mask_block_t<true, true>(stage + KvStage<D>::kSeg, seg_cmp, last_rel, KB, s);
            else mask_block_t<false, true>(stage, seg_cmp, last_rel, KB, s);
          }
          dq_arith(s, dp, lse2, delta_q);
          dq_acc_half_128<kOff + KB * 8192>(tp, pack_acc8(s, 0), pack_acc8(s, 1), dqacc);
        };
        half_tile(std::integral_constant<int, 0>{});
        half_tile(std::integral_constant<int, 1>{});
      } else {
        f32x16 s[2], dp[2];
        scores_t<D>(kOff, ro, qf, s);
        scores_t<D>(vOff, ro, dof, dp);
        if (need_seg || need_causal) {
          if (k_uniform == 0) mask_scores_t<true, true>(stage + KvStage<D>::kSeg, seg_cmp, last_rel, s);
          else mask_scores_t<false, true>(stage, seg_cmp, last_rel, s);
        }
        dq_arith(s[0], dp[0], lse2, delta_q);
        dq_arith(s[1], dp[1], lse2, delta_q);
        accumulate_t<D>(kOff, LeanTrFrags<D>::fresh(lds_base), s, dqacc);
      }
    }
    dma_wait_all();
    __syncthreads();
    kb = nb;
    ++t;
  };
  while (t <= ctx.last) {
    step(std::integral_constant<int, 0>{});
    if (t > ctx.last) break;
    step(std::integral_constant<int, 1>{});
  }

  if (ctx.active) {
    const lds_addr patch = lds0 + w * 32 * D * 2;
    bf16* gbase = p.dq + (((size_t)ctx.work.b * p.S + ctx.work.rb * 32) * p.Hq + ctx.work.h) * D;
    store_rows_t<D>(dqacc, p.scale, patch, gbase, q_row_stride);
  }
  // the store patches overlap the stages of the next item: its copies may start once every
  // wavefront has read its patch back
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __syncthreads();
}

// Workgroups of one (head slice, KV head) group share a work counter and pull query tiles of PB
// row blocks from the work-sorted schedules of the batch rows (tile `rank` of row b at pull
// B * rank + b: heaviest tiles first), so a workgroup that drew light tiles simply draws more of
// them. (Static bins left 15 % of the workgroup slots idle at the end of the launch: the time
// of a tile depends on its mix of masked and unmasked key tiles, not just on their number.)
// The group is the fast index of blockIdx: a group stays on one XCD and its K / V rows in that
// XCD's L2. With more groups than counters (kDqCounters) the tiles are dealt round robin.
template <int D, int HS>
__global__ __launch_bounds__(256, 2) void attn_dq_kernel(AttnParams p) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr lds0 = lds_address_of(smem_raw);
  __shared__ int next_pull;
  constexpr int PB = 4 / HS;
  const int nrb = p.S / 32;
  const int slices = (p.Hq / p.Hkv) / HS;
  const int groups = slices * p.kvh_count;
  const int group = blockIdx.x % groups, member = blockIdx.x / groups, members = gridDim.x / groups;
  const int kvh = p.kvh_base + group % p.kvh_count, slice = group / p.kvh_count;
  const int tpr = bin_tiles_per_row(nrb, PB);
  const int total = p.B * tpr;
  const MetaPtr sched = meta_const(p.sched + query_schedule_offset(nrb, PB));
  const bool dynamic = slices * p.Hkv <= kDqCounters;
  for (int pull = member;; pull += members) {
    if (dynamic) {
      if (threadIdx.x == 0) next_pull = atomicAdd(&p.dq_counters[slice * p.Hkv + kvh], 1);
      __syncthreads();
      pull = uniform(next_pull);
      __syncthreads();
    }
    if (pull >= total) break;
    const int b = pull % p.B, rank = pull / p.B;
    const int qt = uniform(sched[(size_t)b * schedule_ints(nrb) + rank]);
    attn_dq_item<D, HS>(p, b, kvh, slice, qt, lds0);
  }
}

// ---------------------------------------------------------------------------
// dK / dV
// ---------------------------------------------------------------------------
constexpr int kQueryTile = 32;

// LDS stage: Q tile, dO tile (32 x D bf16 each), then lse2 / delta (f32) and
// seg / end (i32), 32 entries each.
template <int D>
struct QdoStage {
  static constexpr int kTileBytes = kQueryTile * D * 2;
  static constexpr int kQ = 0;
  static constexpr int kDo = kTileBytes;
  static constexpr int kLse = 2 * kTileBytes;
  static constexpr int kDelta = kLse + kQueryTile * 4;
  static constexpr int kSeg = kDelta + kQueryTile * 4;
  static constexpr int kEnd = kSeg + kQueryTile * 4;
  static constexpr int kBytes = kEnd + kQueryTile * 4;
  static constexpr int kPatchBytes = 4 * 32 * D * 2;
  // resident V rows of the workgroup's 128 keys (32 per wavefront), after the two stages
  static constexpr int kVResident = 2 * kBytes;
  static constexpr int kTotalBytes = 2 * kBytes + kPatchBytes;
};

// Starts the asynchronous copy of query block qb of head h into `stage`: Q and dO rows, and
// the per-row statistics. The four statistics arrays (lse2, delta: head-major f32; segment ids,
// visible ends: i32) are 128 contiguous bytes each for the 32 rows and sit in the stage in that
// order; wavefront w fetches array w with its first 8 lanes (one copy instruction, the source
// chosen with scalar selects), so no wavefront carries a divergent address computation.
// Without visible ends (plain causal) wavefront 3 has nothing to fetch.
template <int D>
CT_DEVICE void qdo_fetch(const TileDma<kQueryTile, D / 8>& dma, const AttnParams& p, int b, int h,
                         int qb, lds_addr stage) {
  const size_t origin = (((size_t)b * p.S + qb * kQueryTile) * p.Hq + h) * D;
  dma.issue(reinterpret_cast<const char*>(p.q + origin), stage + QdoStage<D>::kQ);
  dma.issue(reinterpret_cast<const char*>(p.dout + origin), stage + QdoStage<D>::kDo);
  const int which = uniform(threadIdx.x >> 6);
  if (which < (p.end ? 4 : 3)) {
    const size_t head_major = ((size_t)b * p.Hq + h) * p.S + qb * kQueryTile;
    const size_t row_major = (size_t)b * p.S + qb * kQueryTile;
    const char* src = which == 0   ? reinterpret_cast<const char*>(p.lse2 + head_major)
                      : which == 1 ? reinterpret_cast<const char*>(p.delta + head_major)
                      : which == 2 ? reinterpret_cast<const char*>(p.seg + row_major)
                                   : reinterpret_cast<const char*>(p.end + row_major);
    const unsigned lane = threadIdx.x & 63;
    if (lane < 8) dma16_s(src, lane * 16, stage + QdoStage<D>::kLse + which * (kQueryTile * 4));
  }
}

// Fragment address structures of the dK/dV kernel: the register-lean ones where the tile is
// wide enough for them (the kernel is at the register limit).
template <int D>
using DkvRowFrags = std::conditional_t<(D / 8 >= 16), RowFragCompact<D / 8>, RowFragOffsets<D / 8>>;
template <int D>
using DkvTrFrags = std::conditional_t<(D / 8 >= 16), TrFragCompact<D / 8, KSlots::kAccum>,
                                      TrFragOffsets<D / 8, KSlots::kAccum>>;

// X (32 rows of an LDS tile) times register fragments: C[row, key] = sum_d X[row, d] F[key, d].
template <int D>
CT_DEVICE f32x16 rows_times_frags(int tile_off, const DkvRowFrags<D>& ro, const bf16x8* frags,
                                  f32x16 c = zero16()) {
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) c = mfma32(ro.load(tile_off, 0, ks), frags[ks], c);
  return c;
}

// Hand-scheduled MFMA sequences of the dK/dV kernel for D = 128 (gen_attn_asm.py): the
// compiler's own schedule issues each LDS fragment read directly in front of the MFMA that
// consumes it, so with two wavefronts per SIMD every MFMA pays most of the LDS latency.
// STAGE_OFF is the byte offset of the stage (Q tile, then dO tile) from the LDS base the
// pointers were built on; v_off the byte offset of this wavefront's V rows.
template <int STAGE_OFF>
CT_DEVICE void dkv_sdp_sequence_128(const RowFragOffsets<16>& ro, const bf16x8* kf, unsigned v_off,
                                    f32x16& s, f32x16& dp) {
  asm volatile(CT_DKV_SDP_SEQUENCE
               : "+v"(s), "+v"(dp)
               : "v"(ro.ptr[0]), "v"(ro.ptr[1]), "v"(ro.ptr[2]), "v"(ro.ptr[3]), "v"(ro.ptr[4]),
                 "v"(ro.ptr[5]), "v"(ro.ptr[6]), "v"(ro.ptr[7]), "v"(kf[0]), "v"(kf[1]), "v"(kf[2]),
                 "v"(kf[3]), "v"(kf[4]), "v"(kf[5]), "v"(kf[6]), "v"(kf[7]), "s"(v_off), "i"(STAGE_OFF)
               : "memory", CT_DKV_ASM_SCRATCH);
}
template <int STAGE_OFF>
CT_DEVICE void dkv_acc_sequence_128(const TrFragOffsets<16, KSlots::kAccum>& to, const f32x16& prob,
                                    const f32x16& ds, f32x16* dvacc, f32x16* dkacc) {
  const bf16x8 p0 = pack_acc8(prob, 0), p1 = pack_acc8(prob, 1);
  const bf16x8 d0 = pack_acc8(ds, 0), d1 = pack_acc8(ds, 1);
  asm volatile(CT_DKV_ACC_SEQUENCE
               : "+v"(dvacc[0]), "+v"(dvacc[1]), "+v"(dvacc[2]), "+v"(dvacc[3]), "+v"(dkacc[0]),
                 "+v"(dkacc[1]), "+v"(dkacc[2]), "+v"(dkacc[3])
               : "v"(to.ptr[0][0]), "v"(to.ptr[0][1]), "v"(to.ptr[0][2]), "v"(to.ptr[0][3]),
                 "v"(to.ptr[1][0]), "v"(to.ptr[1][1]), "v"(to.ptr[1][2]), "v"(to.ptr[1][3]), "v"(p0),
                 "v"(p1), "v"(d0), "v"(d1), "i"(STAGE_OFF)
               : "memory", CT_DKV_ASM_SCRATCH);
}

// acc (32 keys x D) += W^T X, W in accumulator layout (rows = the 32 tile rows,
// cols = keys), X the 32-row LDS tile read transposed.
template <int D>
CT_DEVICE void accumulate_keys(int tile_off, const DkvTrFrags<D>& to, const f32x16& wt,
                               f32x16* acc) {
#pragma unroll
  for (int step = 0; step < 2; ++step) {
    const bf16x8 aop = pack_acc8(wt, step);
#pragma unroll
    for (int db = 0; db < D / 32; ++db) acc[db] = mfma32(aop, to.load(tile_off, step, db), acc[db]);
  }
}

// Store a (32 rows x D) accumulator (lanes along D) as bf16 rows via an LDS patch.
template <int D>
CT_DEVICE void store_rows(const f32x16* acc, lds_addr patch, bf16* gbase, size_t row_stride) {
  constexpr int CPR = D / 8;
  const int l = lane_id(), j = l & 31, half = l >> 5;
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
    const int col = db * 32 + j;
#pragma unroll
    for (int r = 0; r < 16; ++r)
      lds_store<bf16>(patch + tile_byte_offset<CPR>(acc_row(r, half), col >> 3) + (col & 7) * 2,
                      (bf16)acc[db][r]);
  }
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int n = 0; n < 32 * CPR / 64; ++n) {
    const int e = l + 64 * n;
    const int row = e / CPR, c = e % CPR;
    const u32x4 val = lds_load<u32x4>(patch + tile_byte_offset<CPR>(row, c));
    store_global16(gbase + (size_t)row * row_stride + c * 8, val);
  }
}


// Number of (head, query block) items of 128-key tile `tile` (= batch row * tiles per row + kt).
CT_DEVICE int dkv_tile_items(const int* meta, int nrb, int tile, int g, int* q_lo_out = nullptr) {
  const int nt = nrb / 4;
  const int* m = meta + ((size_t)(tile / nt) * nrb + (size_t)(tile % nt) * 4) * kMetaW;
  int q_lo = INT_MAX, q_hi = -1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    q_lo = min(q_lo, m[i * kMetaW + kQFirst]);
    q_hi = max(q_hi, m[i * kMetaW + kQLast]);
  }
  if (q_lo_out) *q_lo_out = q_lo;
  return q_lo <= q_hi ? (q_hi - q_lo + 1) * g : 0;
}

CT_DEVICE int dkv_split_count(int items, int target) {
  return items <= target ? 1 : min(kDkvMaxSplit, (items + target - 1) / target);
}

// Builds the dK/dV work list (one workgroup of 1024 threads): chunk target from
// the total amount of work, chunk count per tile, entries bucketed by
// decreasing work.
__global__ __launch_bounds__(1024) void attn_dkv_schedule_kernel(const int* meta, int B, int S,
                                                                 int Hkv, int g, int max_entries,
                                                                 int max_partials, int* header,
                                                                 int2* entries, int* zeroed,
                                                                 int zeroed_count) {
  for (int i = threadIdx.x; i < zeroed_count; i += 1024) zeroed[i] = 0;  // dQ's work counters
  __shared__ long long red[16];  // one value per wavefront
  __shared__ int hist[256];
  __shared__ int fill[256];
  __shared__ int carry;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nrb = S / 32, ntiles = B * (nrb / 4);

  // Reductions and scans run inside the wavefronts (lane shuffles) and meet once in LDS: the
  // kernel is one workgroup on an otherwise idle GPU, so its time is its chain of barriers.
  auto block_sum = [&](long long v) {
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if (lane == 0) red[wave] = v;
    __syncthreads();
    long long out = 0;
    for (int i = 0; i < 16; ++i) out += red[i];
    __syncthreads();
    return out;
  };
  auto block_max = [&](int v) {
    for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off, 64));
    if (lane == 0) red[wave] = v;
    __syncthreads();
    int out = (int)red[0];
    for (int i = 1; i < 16; ++i) out = max(out, (int)red[i]);
    __syncthreads();
    return out;
  };
  // exclusive prefix of v over the workgroup's threads, and the total
  auto block_scan = [&](int v, int* total) {
    int inc = v;
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(inc, off, 64);
      if (lane >= off) inc += up;
    }
    if (lane == 63) red[wave] = inc;
    __syncthreads();
    int before = 0, all = 0;
    for (int i = 0; i < 16; ++i) {
      const int part = (int)red[i];
      if (i < wave) before += part;
      all += part;
    }
    __syncthreads();
    *total = all;
    return before + inc - v;
  };
  // this thread's first tile is read once; further tiles (more than 1024) are re-read per pass
  const int items_first = tid < ntiles ? dkv_tile_items(meta, nrb, tid, g) : 0;
  auto items_of = [&](int t) { return t == tid ? items_first : dkv_tile_items(meta, nrb, t, g); };

  long long local = 0;
  for (int t = tid; t < ntiles; t += 1024) local += items_of(t);
  const long long total = block_sum(local);
  long long want = (total * Hkv + kDkvSlots - 1) / kDkvSlots;  // one compute slot's fair share
  int target = (int)min((long long)INT_MAX / 2, max((long long)kDkvMinChunk, want));

  // Entry and partial-slot counts for this target; coarsen the target if they overflow the
  // space the host reserved (cannot happen for target >= want, kept as a guard).
  int max_work = 1;
  for (;;) {
    long long counts = 0;  // entries in the high half, partial slots in the low half
    int local_max = 1;
    for (int t = tid; t < ntiles; t += 1024) {
      const int items = items_of(t);
      const int ns = dkv_split_count(items, target);
      counts += ((long long)ns << 32) + (ns > 1 ? ns : 0);
      local_max = max(local_max, (items + ns - 1) / ns);
    }
    const long long both = block_sum(counts);
    max_work = block_max(local_max);
    if ((both >> 32) <= max_entries && (both & 0xffffffffll) <= max_partials) break;
    target = target >= INT_MAX / 4 ? INT_MAX / 2 : target * 2;
  }

  // Histogram of entries over 256 buckets of decreasing work.
  if (tid < 256) {
    hist[tid] = 0;
    fill[tid] = 0;
  }
  if (tid == 0) carry = 0;
  __syncthreads();
  auto bucket_of = [&](int work) { return 255 - (int)((long long)work * 255 / max_work); };
  for (int t = tid; t < ntiles; t += 1024) {
    const int items = items_of(t);
    const int ns = dkv_split_count(items, target);
    const int per = (items + ns - 1) / ns;
    for (int c = 0; c < ns; ++c) atomicAdd(&hist[bucket_of(max(0, min(per, items - c * per)))], 1);
  }
  __syncthreads();
  {
    int entries_total = 0;
    const int start = block_scan(tid < 256 ? hist[tid] : 0, &entries_total);
    if (tid < 256) hist[tid] = start;  // bucket -> first position in the list
    if (tid == 0) {
      header[0] = entries_total;
      header[1] = target;
    }
  }
  __syncthreads();

  // Partial-slot offsets by a running scan over tiles, then scatter.
  for (int base = 0; base < ntiles; base += 1024) {
    const int t = base + tid;
    int items = 0, ns = 1;
    if (t < ntiles) {
      items = items_of(t);
      ns = dkv_split_count(items, target);
    }
    const int mine = (t < ntiles && ns > 1) ? ns : 0;
    int chunk_total = 0;
    const int slot0 = carry + block_scan(mine, &chunk_total);
    __syncthreads();
    if (tid == 0) carry += chunk_total;
    if (t < ntiles) {
      const int per = (items + ns - 1) / ns;
      for (int c = 0; c < ns; ++c) {
        const int bk = bucket_of(max(0, min(per, items - c * per)));
        const int pos = hist[bk] + atomicAdd(&fill[bk], 1);
        entries[pos] = make_int2(t, c | (ns << 8) | (slot0 << 16));
      }
    }
    __syncthreads();
  }
}

// f32 partial sums of one chunk of a split key tile.
template <int D>
struct DkvPartial {
  static constexpr int kPerWave = (D / 32) * 16 * 64;  // floats of one accumulator set of a wavefront
  static constexpr int kPerTensor = 4 * kPerWave;      // dK (or dV) of the 4 wavefronts
  static constexpr size_t kPerChunk = 2 * kPerTensor;
};
template <int D>
CT_DEVICE size_t dkv_partial_offset(int slot, int Hkv, int kvh, int wave) {
  return ((size_t)slot * Hkv + kvh) * DkvPartial<D>::kPerChunk + (size_t)wave * DkvPartial<D>::kPerWave;
}

// Adds the chunks of every split key tile in chunk order (fixed order: the result does not
// depend on timing) and writes dK, dV. One workgroup per (entry, KV head); only the entry of
// chunk 0 of a split tile has work.
template <int D>
__global__ __launch_bounds__(256) void attn_dkv_reduce_kernel(AttnParams p) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr lds0 = lds_address_of(smem_raw);
  const int l = lane_id(), w = threadIdx.x >> 6;
  const int nrb = p.S / 32;
  const int kvh = blockIdx.x % p.Hkv, entry = blockIdx.x / p.Hkv;
  // This is the last kernel of a backward call: it leaves the dQ kernel's work counters at zero,
  // so that a later call on the same workspace can keep the work list and skip the kernel that
  // builds it (and clears the counters).
  if (blockIdx.x == 0)
    for (int i = threadIdx.x; i < kDqCounters; i += blockDim.x) p.dq_counters[i] = 0;
  if (entry >= uniform(p.dkv_header[0])) return;
  const int2 work_entry = p.dkv_entries[entry];
  const int tile = uniform(work_entry.x), packed = uniform(work_entry.y);
  const int chunk = packed & 255, nsplit = (packed >> 8) & 255, slot0 = (unsigned)packed >> 16;
  if (chunk != 0 || nsplit <= 1) return;
  const int b = tile / (nrb / 4), kt = tile % (nrb / 4);
  f32x16 dkacc[D / 32], dvacc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
    dkacc[db] = zero16();
    dvacc[db] = zero16();
  }
  for (int c = 0; c < nsplit; ++c) {
    const float* src = p.dkv_partials + dkv_partial_offset<D>(slot0 + c, p.Hkv, kvh, w) + l * 4;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(src + (db * 4 + q4) * 256);
        const f32x4 cv = *reinterpret_cast<const f32x4*>(src + DkvPartial<D>::kPerTensor + (db * 4 + q4) * 256);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          dkacc[db][4 * q4 + e] += a[e];
          dvacc[db][4 * q4 + e] += cv[e];
        }
      }
  }
  const lds_addr patch = lds0 + w * 32 * D * 2;
  const size_t kv_row_stride = (size_t)p.Hkv * D;
  const size_t out_off = (((size_t)b * p.S + (kt * 4 + w) * 32) * p.Hkv + kvh) * D;
  store_rows<D>(dkacc, patch, p.dk + out_off, kv_row_stride);
  __builtin_amdgcn_wave_barrier();
  store_rows<D>(dvacc, patch, p.dv + out_off, kv_row_stride);
}

// Byte address of the dS block (key block rb with table entries ds_off / q_first, query block qb)
// of query head `head`, batch row b: wave-uniform.
CT_DEVICE char* ds_block_address(const AttnParams& p, int head, int b, int ds_off, int q_first, int qb) {
  const int first_head = p.kvh_base * (p.Hq / p.Hkv);
  const size_t block = ((size_t)(head - first_head) * p.B + b) * p.ds_row_blocks + (size_t)(ds_off + qb - q_first);
  return p.ds + block * kDsBlockBytes;
}

// SPILL: every (key block, query block) step also stores its bf16 dS block to the dS region, for
// attn_dq_blocks_kernel.
template <int D, bool SPILL>
__global__ __launch_bounds__(256, 2) void attn_dkv_kernel(AttnParams p) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr lds0 = lds_address_of(smem_raw);
  constexpr int kStage = QdoStage<D>::kBytes;

  const int l = lane_id(), j = l & 31, half = l >> 5, w = threadIdx.x >> 6;
  const int nrb = p.S / 32;
  const int kvh = p.kvh_base + blockIdx.x % p.kvh_count, entry = blockIdx.x / p.kvh_count;
  if (entry >= uniform(p.dkv_header[0])) return;
  const int2 work_entry = p.dkv_entries[entry];
  const int tile = uniform(work_entry.x), packed = uniform(work_entry.y);
  const int chunk = packed & 255, nsplit = (packed >> 8) & 255, slot0 = (unsigned)packed >> 16;
  const int b = tile / (nrb / 4), kt = tile % (nrb / 4);
  const int g = p.Hq / p.Hkv;
  const int* meta_b = p.meta + (size_t)b * nrb * kMetaW;
  const DkvRowFrags<D> ro(lds0);
  const DkvTrFrags<D> to(lds0);

  int q_lo = INT_MAX, q_hi = -1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const MetaPtr m = meta_const(meta_b + (kt * 4 + i) * kMetaW);
    q_lo = min(q_lo, uniform(m[kQFirst]));
    q_hi = max(q_hi, uniform(m[kQLast]));
  }
  const int my_rb = kt * 4 + w;
  const int my_min = uniform(meta_const(meta_b)[my_rb * kMetaW + kMinNz]);
  const int my_max = uniform(meta_const(meta_b)[my_rb * kMetaW + kMaxId]);
  const int my_uni = uniform(meta_const(meta_b)[my_rb * kMetaW + kUniform]);
  const int my_q_first = uniform(meta_const(meta_b)[my_rb * kMetaW + kQFirst]);
  const int my_ds_off = uniform(meta_const(meta_b)[my_rb * kMetaW + kDsOff]);

  const int key = my_rb * 32 + j;
  const int seg_k = p.seg[(size_t)b * p.S + key];
  const bool has_end = p.end != nullptr;
  const size_t kv_row_stride = (size_t)p.Hkv * D;
  const size_t kv_off = (((size_t)b * p.S + key) * p.Hkv + kvh) * D;

  // K fragments stay in registers; V fragments are parked in LDS (this wavefront's
  // private 32-row patch) and re-read per block, which keeps the kernel under 256
  // registers so that two workgroups share a CU.
  const int vpatch_off = QdoStage<D>::kVResident + uniform(w) * 32 * D * 2;
  const lds_addr vpatch = lds0 + vpatch_off;
  bf16x8 kf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    kf[ks] = as_bf16x8(load_global16(p.k + kv_off + 16 * ks + 8 * half));
    lds_store<u32x4>(ro.addr(vpatch_off, 0, ks), load_global16(p.v + kv_off + 16 * ks + 8 * half));
  }
  f32x16 dkacc[D / 32], dvacc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
    dkacc[db] = zero16();
    dvacc[db] = zero16();
  }

  // Make the K fragment loads complete here. Left pending, their first use inside the item
  // loop gets an `s_waitcnt vmcnt(n)` whose count fits the first item only; on every later item
  // the same wait stalls until the asynchronous copies of the next stage have landed.
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) asm volatile("" : "+v"(kf[ks]));

  // The Q tiles stay unscaled in LDS: the softmax scale enters the exponent in f32
  // (S = scale * (Q K^T); the forward rounded scale * Q to bf16 first, a difference of one
  // bf16 rounding per element of Q) and dK = scale * (dS^T Q) is scaled once at the end.
  const float scale_log2e = exponent_scale(p.scale) * kLog2e;
  const float masked = masked_score(p.scale);

  // Work items: (head of the group, query block) pairs, flattened; query block fastest.
  const int nq = (q_lo <= q_hi) ? (q_hi - q_lo + 1) : 0;
  const int per_chunk = (nq * g + nsplit - 1) / nsplit;
  int it = chunk * per_chunk;
  const int items = min(nq * g, it + per_chunk);  // end of this chunk's item range
  int qb = q_lo, head = kvh * g;
  if (it < items) {
    head += it / nq;
    qb += it % nq;
  }
  const TileDma<kQueryTile, D / 8> dma((size_t)p.Hq * D * 2);
  if (it < items) {
    qdo_fetch<D>(dma, p, b, head, qb, lds0);
    dma_wait_all();
  }
  __syncthreads();

  QueryBlockBounds qb_bounds = query_block_bounds(meta_b, min(qb, nrb - 1));
  auto step = [&](auto stage_tag) {
    constexpr int CUR = decltype(stage_tag)::value;
    const lds_addr stage = lds0 + CUR * kStage;
    const bool more = it + 1 < items;
    int qb_next = qb + 1, head_next = head;
    if (qb_next > q_hi) {
      qb_next = q_lo;
      ++head_next;
    }
    if (more) qdo_fetch<D>(dma, p, b, head_next, qb_next, lds0 + (CUR ^ 1) * kStage);

    // bounds of this query block (read one item ahead: the scalar loads are long done when
    // the next item needs them)
    const int q_min = qb_bounds.min_nz, q_max = qb_bounds.max_id, q_end_max = qb_bounds.end_max,
              q_end_min = qb_bounds.end_min, q_uni = qb_bounds.uniform;
    if (more) qb_bounds = query_block_bounds(meta_b, qb_next);
    const bool visit = blocks_interact(q_min, q_max, q_end_max, my_min, my_max, my_rb * 32);
    if (visit) {
      // The row offsets below depend on the lane only; hoisted out of the loop they become
      // spilled registers whose reloads wait for every copy in flight. Recompute them here.
      int half_here = half;
      asm volatile("" : "+v"(half_here));
      // Both products start from the per-row terms of their 16 query rows instead of zero (the
      // statistics pass left -lse / scale and -delta): the sums S - lse / scale and dP - delta
      // come out of the matrix pipe, and no vector instruction adds them.
      f32x16 s, dp;
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int r0 = 8 * qd + 4 * half_here;
        const f32x4 lse4 = lds_load<f32x4>(stage + QdoStage<D>::kLse + r0 * 4);
        const f32x4 del4 = lds_load<f32x4>(stage + QdoStage<D>::kDelta + r0 * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s[4 * qd + e] = lse4[e];
          dp[4 * qd + e] = del4[e];
        }
      }
      if constexpr (D == 128) {
        // (fragment pointers built here from the lane id: held across the loop they would
        // push the kernel over its register budget)
        const RowFragOffsets<16> rp = RowFragOffsets<16>::expand(RowFragCompact<16>(lds0, lane_id_here()));
        dkv_sdp_sequence_128<CUR * kStage>(rp, kf, (unsigned)vpatch_off, s, dp);
      } else {
        s = rows_times_frags<D>(CUR * kStage + QdoStage<D>::kQ, ro, kf, s);
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks)
          dp = mfma32(ro.load(CUR * kStage + QdoStage<D>::kDo, 0, ks), ro.load(vpatch_off, 0, ks), dp);
      }
      const bool interior = tile_is_interior(q_uni, q_end_min, my_uni, my_rb * 32 + 31);
      f32x16 prob;
      if (!interior) {
        // Masked scores become -inf (their probability is then exactly 0). Written with
        // bitwise logic and selects only: the per-element tests must not turn into branches.
        const int seg_k_or_never = seg_k != 0 ? seg_k : -1;  // ids are >= 0
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          const int r0 = 8 * qd + 4 * half_here;  // first of 4 consecutive query rows
          const i32x4 seg4 = lds_load<i32x4>(stage + QdoStage<D>::kSeg + r0 * 4);
          i32x4 end4;
          if (has_end) {
            end4 = lds_load<i32x4>(stage + QdoStage<D>::kEnd + r0 * 4);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) end4[e] = qb * kQueryTile + r0 + e;
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const bool ok = (seg4[e] == seg_k_or_never) & (key <= end4[e]);
            s[4 * qd + e] = ok ? s[4 * qd + e] : masked;
          }
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pr = exp2_fast(s[r] * scale_log2e);  // s = S - lse / scale
        prob[r] = pr;
        dp[r] = pr * dp[r];                              // dp = dP - delta
      }
      if constexpr (SPILL) {
        // The block as the lanes hold it: the two operands of the dK product (8 query rows of one
        // key each) as two runs of 64 x 16 bytes in lane order, so a store writes 1 KB end to end.
        char* block = ds_block_address(p, head, b, my_ds_off, my_q_first, qb);
        const unsigned lane_off = (unsigned)lane_id_here() * 16;
        store_global16_s<0>(block, lane_off, __builtin_bit_cast(f32x4, pack_acc8(dp, 0)));
        store_global16_s<1024>(block, lane_off, __builtin_bit_cast(f32x4, pack_acc8(dp, 1)));
      }
      if constexpr (D == 128) {
        const TrFragOffsets<16, KSlots::kAccum> tp =
            TrFragOffsets<16, KSlots::kAccum>::expand(TrFragCompact<16, KSlots::kAccum>(lds0, lane_id_here()));
        dkv_acc_sequence_128<CUR * kStage>(tp, prob, dp, dvacc, dkacc);
      } else {
        accumulate_keys<D>(CUR * kStage + QdoStage<D>::kDo, to, prob, dvacc);
        accumulate_keys<D>(CUR * kStage + QdoStage<D>::kQ, to, dp, dkacc);
      }
    }
    // Vector memory operations complete in the order they were issued: the two stores of this
    // step are the youngest, so waiting for all but two has waited for every copy of the next
    // stage without waiting for the stores (they are long done one step later).
    if (SPILL && visit) __builtin_amdgcn_s_waitcnt(0x0F72);
    else dma_wait_all();
    __syncthreads();
    ++it;
    qb = qb_next;
    head = head_next;
  };
  while (it < items) {
    step(std::integral_constant<int, 0>{});
    if (it >= items) break;
    step(std::integral_constant<int, 1>{});
  }

#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) dkacc[db][e] *= p.scale;

  if (nsplit > 1) {
    // A chunk of a split tile leaves its sums as f32 for attn_dkv_reduce_kernel:
    // [dK | dV][wavefront][d block][register quad][lane][4], 16 bytes per lane and store.
    float* mine = p.dkv_partials + dkv_partial_offset<D>(slot0 + chunk, p.Hkv, kvh, w) + l * 4;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 a, c;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a[e] = dkacc[db][4 * q4 + e];
          c[e] = dvacc[db][4 * q4 + e];
        }
        *reinterpret_cast<f32x4*>(mine + (db * 4 + q4) * 256) = a;
        *reinterpret_cast<f32x4*>(mine + DkvPartial<D>::kPerTensor + (db * 4 + q4) * 256) = c;
      }
    return;
  }

  const lds_addr patch = vpatch;  // V fragments are no longer needed
  const size_t out_off = (((size_t)b * p.S + my_rb * 32) * p.Hkv + kvh) * D;
  store_rows<D>(dkacc, patch, p.dk + out_off, kv_row_stride);
  __builtin_amdgcn_wave_barrier();
  store_rows<D>(dvacc, patch, p.dv + out_off, kv_row_stride);
}

// ---------------------------------------------------------------------------
// dQ from stored dS blocks: dQ = scale * sum over visited key blocks of dS K
// (src/kernels/efficient_attention.py:1046-1048 with the dS of :1040-1045 read back instead of
// formed again). Same workgroup shape, work pulling and key-tile walk as attn_dq_kernel; a stage
// holds the K rows of a 64-key tile (shared by the 4 wavefronts) and, per wavefront, the dS blocks
// of its query block against the tile's two key blocks, copied straight from the dS region. A
// block is read back as the B operand of dQ^T += K^T dS^T with transposing LDS reads, which is
// the transposition between the key-stationary kernel that wrote it (lanes along keys) and this
// query-stationary product (lanes along queries). Bound by the bytes of the blocks it reads.
// ---------------------------------------------------------------------------
// Eight wavefronts per workgroup (HS heads x 8 / HS query blocks). A stage: the K rows of one
// 32-key block (shared by all wavefronts) and, per wavefront, the dS block of its query block
// against that key block. A dS block sits in LDS as it sits in memory (two runs of 64 x 16 bytes,
// lane (half, key) order), the second run 64 bytes further than its 1 KB so that the transposing
// reads of one fragment spread over all banks. Three stages: two key blocks are in flight while
// one is worked on (the kernel lives on bytes in flight; what bounds them is LDS, and with eight
// wavefronts per K block four fifths of a stage are dS).
constexpr int kDqbWaves = 8;
template <int D>
struct DsStage {
  static constexpr int kK = 0;
  static constexpr int kKBytes = 32 * D * 2;
  static constexpr int kRun = 1024 + 64;
  static constexpr int kPatch = 2 * kRun;
  static constexpr int kDs = kKBytes;  // [wavefront][kPatch]
  static constexpr int kBytes = kKBytes + kDqbWaves * kPatch;
  static constexpr int kStages = 3;
  static constexpr int kTotalBytes =
      kStages * kBytes > kDqbWaves * 32 * D * 2 ? kStages * kBytes : kDqbWaves * 32 * D * 2;  // >= the store patches
};

// Transposed-fragment pointers into a dS block: the B operand of dQ^T += K^T dS^T wants, for
// query slot n = lane % 32, the keys of a k-step in accumulator order (matching the K fragments).
// The 8-byte piece (key, slots 4 m .. 4 m + 3) is the half (slots & 4) of lane (half = slot >> 4,
// key)'s 16 bytes in run (slot >> 3) & 1.
struct DsFragPtrs {
  lds_addr ptr[2];
  CT_DEVICE DsFragPtrs(lds_addr base, int l) {
    const int pp = l & 15, q16 = (l >> 4) & 1, half = l >> 5;
#pragma unroll
    for (int second = 0; second < 2; ++second) {
      const int key = 4 * half + 8 * second + (pp >> 2);
      const int run = (pp & 3) >> 1, piece = pp & 1;
      ptr[second] = base + (run * (1024 + 64) + q16 * 512 + key * 16 + piece * 8);
    }
  }
  // keys 16 ks .. 16 ks + 15 of the block at byte offset `off`
  CT_DEVICE bf16x8 load(int off, int ks) const {
    const bf16x4_vs lo = lds_load_tr(ptr[0] + (off + ks * 256));
    const bf16x4_vs hi = lds_load_tr(ptr[1] + (off + ks * 256));
    bf16x8 out;
    out[0] = lo[0]; out[1] = lo[1]; out[2] = lo[2]; out[3] = lo[3];
    out[4] = hi[0]; out[5] = hi[1]; out[6] = hi[2]; out[7] = hi[3];
    return out;
  }
};

// What the walk needs to know about a 32-key block (scalar loads).
struct DsKeyBlockInfo {
  int k_min, k_max, q_first, ds_off;
};
CT_DEVICE DsKeyBlockInfo ds_key_block_info(const int* meta_b, int rbk) {
  const MetaPtr m = meta_const(meta_b + rbk * kMetaW);
  DsKeyBlockInfo info;
  info.k_min = m[kMinNz];
  info.k_max = m[kMaxId];
  info.q_first = m[kQFirst];
  info.ds_off = m[kDsOff];
  return info;
}

// store_rows_t for an accumulator whose lane j holds the query row ds_slot_row(j) of the block.
template <int D>
CT_DEVICE void store_slot_rows_t(const f32x16* acc, float row_scale, lds_addr patch, bf16* gbase,
                                 size_t row_stride) {
  constexpr int CPR = D / 8;
  int l = lane_id();
  asm volatile("" : "+v"(l));
  const int row_of_lane = ds_slot_row(l & 31), half = l >> 5;
  using Patch = PatchRows<D>;
  const lds_addr store_base = Patch::store_base(patch, row_of_lane, half);
  const unsigned row_swizzle = Patch::row_swizzle(row_of_lane);
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

// s_waitcnt vmcnt(n) for a wave-uniform n that is one of the few values the walk produces.
CT_DEVICE void wait_all_copies_but(int n) {
  if (n == 0) __builtin_amdgcn_s_waitcnt(0x0F70);
  else if (n == 1) __builtin_amdgcn_s_waitcnt(0x0F71);
  else if (n == 2) __builtin_amdgcn_s_waitcnt(0x0F72);
  else __builtin_amdgcn_s_waitcnt(0x0F73);
}

template <int D, int HS>
CT_DEVICE void attn_dq_blocks_item(const AttnParams& p, int b, int kvh, int slice, int qt, const lds_addr lds0,
                                   const TileDma<32, D / 8, (D == 128 ? 512 : 256)>& kdma,
                                   const DsFragPtrs& frags, const TrFragOffsets<D / 8, KSlots::kAccum>& tp) {
  constexpr int PB = kDqbWaves / HS;
  constexpr int kStage = DsStage<D>::kBytes;
  const int nrb = p.S / 32;
  const int g = p.Hq / p.Hkv;
  const int w = uniform(threadIdx.x >> 6);
  const int h = kvh * g + slice * HS + (w % HS);
  int rb = qt * PB + (w / HS);
  const bool active = rb < nrb;
  if (!active) rb = nrb - 1;
  const int* meta_b = p.meta + (size_t)b * nrb * kMetaW;
  QueryBlockBounds mine = query_block_bounds(meta_b, rb);
  if (!active) mine.min_nz = 0;  // interacts with nothing
  int first_tile = INT_MAX, last_tile = -1;  // 64-key tiles, as the table has them
#pragma unroll
  for (int i = 0; i < PB; ++i) {
    if (qt * PB + i >= nrb) break;
    const MetaPtr m = meta_const(meta_b + (qt * PB + i) * kMetaW);
    first_tile = min(first_tile, uniform(m[kKvFirst]));
    last_tile = max(last_tile, uniform(m[kKvLast]));
  }
  // the walk is in 32-key blocks (a tile without keys is the pair INT_MAX / -1: converted only
  // when there is a range, and clamped to the row so that no table entry can lead outside it)
  const bool any = first_tile <= last_tile && first_tile >= 0 && last_tile < nrb / 2;
  const int first = any ? 2 * first_tile : 0;
  const int last = any ? 2 * last_tile + 1 : -1;
  const char* kbase = reinterpret_cast<const char*>(p.k + ((size_t)b * p.S * p.Hkv + kvh) * D);
  const size_t kv_row_bytes = (size_t)p.Hkv * D * 2;
  const unsigned ds_lane_off = (unsigned)lane_id_here() * 16;
  const int my_ds = DsStage<D>::kDs + w * DsStage<D>::kPatch;  // this wavefront's block inside a stage
  // copies of the K rows this wavefront issues per stage (head dimension 64: 256 threads cover the block)
  const bool copies_k = D == 128 || w < 4;

  f32x16 dqacc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db) dqacc[db] = zero16();

  auto visits = [&](const DsKeyBlockInfo& info, int rbk) {
    return blocks_interact(mine.min_nz, mine.max_id, mine.end_max, uniform(info.k_min), uniform(info.k_max),
                           rbk * 32);
  };
  // K rows of key block rbk (all wavefronts) and this wavefront's dS block against it; returns the
  // number of copy instructions this wavefront issued
  auto issue = [&](int rbk, const DsKeyBlockInfo& info, lds_addr stage) {
    int issued = 0;
    if (copies_k) {
      kdma.issue(kbase + (size_t)rbk * 32 * kv_row_bytes, stage + DsStage<D>::kK);
      issued = 1;
    }
    if (visits(info, rbk)) {
      const char* block = ds_block_address(p, h, b, uniform(info.ds_off), uniform(info.q_first), rb);
      dma16_s(block, ds_lane_off, stage + my_ds);
      dma16_s(block + 1024, ds_lane_off, stage + (my_ds + DsStage<D>::kRun));
      issued += 2;
    }
    return issued;
  };

  // info[i]: key block t + i; stage of key block t + i is (stage of t + i) mod 3
  int t = first;
  DsKeyBlockInfo cur = {}, next = {}, after = {};
  int pending = 0;  // copy instructions of the youngest key block in flight
  if (t <= last) {
    cur = ds_key_block_info(meta_b, t);
    issue(t, cur, lds0);
    if (t + 1 <= last) {
      next = ds_key_block_info(meta_b, t + 1);
      pending = issue(t + 1, next, lds0 + kStage);
      if (t + 2 <= last) after = ds_key_block_info(meta_b, t + 2);
    }
  }
  wait_all_copies_but(pending);
  __syncthreads();

  auto step = [&](auto stage_tag) {
    constexpr int CUR = decltype(stage_tag)::value;
    constexpr int kFill = (CUR + 2) % 3;  // last read one step ago: every wavefront is past that barrier
    DsKeyBlockInfo later = after;
    pending = 0;
    if (t + 2 <= last) {
      pending = issue(t + 2, after, lds0 + kFill * kStage);
      if (t + 3 <= last) later = ds_key_block_info(meta_b, t + 3);
    }
    if (visits(cur, t)) {
      constexpr int ds_off = CUR * kStage;  // + my_ds, inside the pointers
      constexpr int k_off = CUR * kStage + DsStage<D>::kK;
      const bf16x8 ds0 = frags.load(ds_off, 0), ds1 = frags.load(ds_off, 1);
#pragma unroll
      for (int db = 0; db < D / 32; ++db) dqacc[db] = mfma32(tp.load(k_off, 0, db), ds0, dqacc[db]);
#pragma unroll
      for (int db = 0; db < D / 32; ++db) dqacc[db] = mfma32(tp.load(k_off, 1, db), ds1, dqacc[db]);
    }
    // Copies complete in the order they were issued: all but the ones just issued means key
    // block t + 1 has landed.
    wait_all_copies_but(pending);
    __syncthreads();
    cur = next;
    next = after;
    after = later;
    ++t;
  };
  while (t <= last) {
    step(std::integral_constant<int, 0>{});
    if (t > last) break;
    step(std::integral_constant<int, 1>{});
    if (t > last) break;
    step(std::integral_constant<int, 2>{});
  }

  if (active) {
    const lds_addr patch = lds0 + w * 32 * D * 2;
    bf16* gbase = p.dq + (((size_t)b * p.S + rb * 32) * p.Hq + h) * D;
    store_slot_rows_t<D>(dqacc, p.scale, patch, gbase, (size_t)p.Hq * D);
  }
  // the store patches overlap the stages of the next item
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __syncthreads();
}

template <int D, int HS>
__global__ __launch_bounds__(kDqbWaves * 64, 2) void attn_dq_blocks_kernel(AttnParams p) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr lds0 = lds_address_of(smem_raw);
  __shared__ int next_pull;
  constexpr int PB = kDqbWaves / HS;
  const int nrb = p.S / 32;
  const int slices = (p.Hq / p.Hkv) / HS;
  const int groups = slices * p.kvh_count;
  const int group = blockIdx.x % groups, member = blockIdx.x / groups, members = gridDim.x / groups;
  const int kvh = p.kvh_base + group % p.kvh_count, slice = group / p.kvh_count;
  const int tpr = bin_tiles_per_row(nrb, PB);
  const int total = p.B * tpr;
  const MetaPtr sched = meta_const(p.sched + query_schedule_offset(nrb, PB));
  const bool dynamic = slices * p.Hkv <= kDqCounters;
  const TileDma<32, D / 8, (D == 128 ? 512 : 256)> kdma((size_t)p.Hkv * D * 2);
  const int w = threadIdx.x >> 6;
  const DsFragPtrs frags(lds0 + (DsStage<D>::kDs + w * DsStage<D>::kPatch), lane_id());
  const TrFragOffsets<D / 8, KSlots::kAccum> tp(lds0);
  for (int pull = member;; pull += members) {
    if (dynamic) {
      if (threadIdx.x == 0) next_pull = atomicAdd(&p.dq_counters[slice * p.Hkv + kvh], 1);
      __syncthreads();
      pull = uniform(next_pull);
      __syncthreads();
    }
    if (pull >= total) break;
    const int b = pull % p.B, rank = pull / p.B;
    const int qt = uniform(sched[(size_t)b * schedule_ints(nrb) + rank]);
    attn_dq_blocks_item<D, HS>(p, b, kvh, slice, qt, lds0, kdma, frags, tp);
  }
}

}  // namespace ct
