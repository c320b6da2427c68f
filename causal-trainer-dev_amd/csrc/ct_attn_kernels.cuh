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

#include "ct_attn_meta.cuh"
#include "ct_common.cuh"

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
  float* delta;
  bf16* dq;
  bf16* dk;
  bf16* dv;
  int B, S, Hq, Hkv;
  float scale;      // already rounded to bf16
  // dK/dV work list (backward only)
  int* dkv_header;
  int* dkv_counters;
  int2* dkv_entries;
  float* dkv_partials;
  int dkv_max_entries, dkv_max_partials;
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
      : kbase(reinterpret_cast<const char*>(k)), vbase(reinterpret_cast<const char*>(v)),
        segb(seg), row_stride_bytes(row_stride_elems * 2) {}
  CT_DEVICE void issue(int tile, lds_addr stage) const {
    const size_t origin = (size_t)tile * kKeyTile * row_stride_bytes;
    dma.issue(kbase + origin, row_stride_bytes, stage + KvStage<D>::kK);
    dma.issue(vbase + origin, row_stride_bytes, stage + KvStage<D>::kV);
    if (threadIdx.x < 16)  // 64 ids = 16 lanes x 16 bytes, linear layout
      dma16(segb + tile * kKeyTile + threadIdx.x * 4, stage + KvStage<D>::kSeg);
  }
};

// Decoded position of a workgroup / wavefront in the (batch, head, row block)
// space. Hardware workgroup ids run over (rank, group): the group (batch,
// head slice, KV head) is the fast index, so a group always lands on the same
// XCD (ids are dealt round robin to the 8 XCDs) and keeps its K/V in that L2;
// the rank is the position in the batch row's work-sorted schedule, longest
// tiles first.
template <int HS>
struct QueryWork {
  static constexpr int PB = 4 / HS;  // row blocks per workgroup
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
};

// S^T (two 32-key blocks) = K_tile Q^T for this wavefront's 32 queries.
// `tile_off` is the tile's byte offset from the LDS base the offsets were built on.
template <int D>
CT_DEVICE void scores_t(int tile_off, const RowFragOffsets<D / 8>& ro, const bf16x8* qf,
                        f32x16* s) {
  s[0] = zero16();
  s[1] = zero16();
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) s[kb] = mfma32(ro.load(tile_off, kb, ks), qf[ks], s[kb]);
  }
}

// allowed(query of this lane, key held by register r of block kb)?  Writes a
// 32-bit mask per block: bit r set = allowed.
CT_DEVICE void tile_mask(lds_addr segk, int tile, int seg_q, int end_q, bool row_valid,
                         unsigned* allow) {
  const int half = lane_id() >> 5;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    unsigned bits = 0;
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const int k0 = kb * 32 + 8 * qd + 4 * half;
      const i32x4 sk = lds_load<i32x4>(segk + k0 * 4);
      const int key = tile * kKeyTile + k0;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        bits |= (unsigned)(sk[e] == seg_q && key + e <= end_q) << (4 * qd + e);
    }
    allow[kb] = row_valid ? bits : 0u;
  }
}

// acc (D x 32 queries, transposed) += X^T W^T where X is a 64-row LDS tile read
// transposed and W^T are the accumulator-layout weights wt[2].
template <int D>
CT_DEVICE void accumulate_t(int tile_off, const TrFragOffsets<D / 8, KSlots::kAccum>& to,
                            const f32x16* wt, f32x16* acc) {
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
  const int l = lane_id(), j = l & 31, half = l >> 5;
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const int d0 = db * 32 + 8 * qd + 4 * half;
      bf16x4 pk;
#pragma unroll
      for (int e = 0; e < 4; ++e) pk[e] = (bf16)(acc[db][4 * qd + e] * row_scale);
      lds_store<bf16x4>(patch + tile_byte_offset<CPR>(j, d0 >> 3) + (d0 & 4) * 2, pk);
    }
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

// Shared prologue of the forward and dQ kernels.
template <int D, int HS>
struct QueryTileContext {
  static constexpr int PB = 4 / HS;
  QueryWork<HS> work;
  const int* meta_b;
  QueryBlockBounds mine;
  int first, last;
  int pos, seg_q, end_q;
  bool row_valid;
  size_t q_off, stat_off;
  const bf16* kbase;
  const bf16* vbase;
  const int* segb;
  CT_DEVICE explicit QueryTileContext(const AttnParams& p) : work(p) {
    const int nrb = p.S / 32;
    meta_b = p.meta + (size_t)work.b * nrb * kMetaW;
    mine = query_block_bounds(meta_b, work.rb);
    first = INT_MAX;
    last = -1;
#pragma unroll
    for (int i = 0; i < PB; ++i) {
      const MetaPtr m = meta_const(meta_b + (work.qt * PB + i) * kMetaW);
      first = min(first, uniform(m[kKvFirst]));
      last = max(last, uniform(m[kKvLast]));
    }
    pos = work.rb * 32 + (lane_id() & 31);
    seg_q = p.seg[(size_t)work.b * p.S + pos];
    end_q = p.end ? p.end[(size_t)work.b * p.S + pos] : pos;
    row_valid = seg_q != 0;
    q_off = (((size_t)work.b * p.S + pos) * p.Hq + work.h) * D;
    stat_off = ((size_t)work.b * p.S + pos) * p.Hq + work.h;
    kbase = p.k + ((size_t)work.b * p.S * p.Hkv + work.kvh) * D;
    vbase = p.v + ((size_t)work.b * p.S * p.Hkv + work.kvh) * D;
    segb = p.seg + (size_t)work.b * p.S;
  }
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

// ---------------------------------------------------------------------------
// Forward
// ---------------------------------------------------------------------------
template <int D, int HS>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(AttnParams p) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr lds0 = lds_address_of(smem_raw);
  constexpr int kStage = KvStage<D>::kBytes;

  const QueryTileContext<D, HS> ctx(p);
  const int l = lane_id(), half = l >> 5, w = threadIdx.x >> 6;
  const RowFragOffsets<D / 8> ro(lds0);
  const TrFragOffsets<D / 8, KSlots::kAccum> to(lds0);
  const size_t q_row_stride = (size_t)p.Hq * D;
  const size_t kv_row_stride = (size_t)p.Hkv * D;

  bf16x8 qf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks)
    qf[ks] = scale_bf16x8(as_bf16x8(load_global16(p.q + ctx.q_off + 16 * ks + 8 * half)), p.scale);

  f32x16 oacc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db) oacc[db] = zero16();
  float m_run = kNegInf;  // running max, log2 domain
  float l_run = 0.f;      // this lane's share of the running sum

  const KvFetcher<D> fetch(ctx.kbase, ctx.vbase, ctx.segb, kv_row_stride);
  int t = ctx.first;
  KeyTileBounds kb = {0, 0, 0};
  if (t <= ctx.last) {
    fetch.issue(t, lds0);
    kb = key_tile_bounds(ctx.meta_b, t);
  }
  dma_wait_all();
  __syncthreads();

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
      f32x16 s[2];
      scores_t<D>(CUR * kStage + KvStage<D>::kK, ro, qf, s);
      float mx = kNegInf;
      if (!ctx.interior(kb, t)) {
        unsigned allow[2];
        tile_mask(stage + KvStage<D>::kSeg, t, ctx.seg_q, ctx.end_q, ctx.row_valid, allow);
#pragma unroll
        for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            s[kbk][r] = ((allow[kbk] >> r) & 1u) ? s[kbk][r] : kNegInf;
      }
#pragma unroll
      for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kbk][r]);
      mx = fmaxf(mx, xor32(mx)) * kLog2e;
      const float m_new = fmaxf(m_run, mx);
      const float m_use = (m_new == kNegInf) ? 0.f : m_new;
      float psum = 0.f;
#pragma unroll
      for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          s[kbk][r] = exp2_fast(fmaf(s[kbk][r], kLog2e, -m_use));
          psum += s[kbk][r];
        }
      if (__any(m_new != m_run)) {
        const float alpha = exp2_fast(m_run - m_use);
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
        m_run = m_new;
      }
      l_run += psum;
      accumulate_t<D>(CUR * kStage + KvStage<D>::kV, to, s, oacc);
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

  const float l_tot = l_run + xor32(l_run);
  const bool has = l_tot > 0.f;
  const float inv = has ? 1.f / l_tot : 0.f;
  if (half == 0) p.lse[ctx.stat_off] = has ? (__logf(l_tot) + m_run * kLn2) : 0.f;
  const lds_addr patch = lds0 + w * 32 * D * 2;
  bf16* obase = p.out + (((size_t)ctx.work.b * p.S + ctx.work.rb * 32) * p.Hq + ctx.work.h) * D;
  store_rows_t<D>(oacc, inv, patch, obase, q_row_stride);
}

// ---------------------------------------------------------------------------
// delta[row] = sum_d f32(out[row, d]) * f32(dout[row, d])      (HBM bound)
// One 16-byte load per lane per tensor; D/8 lanes share a row.
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_delta_kernel(const bf16* out, const bf16* dout,
                                                         float* delta, long rows) {
  constexpr int LPR = D / 8;  // lanes per row
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  const long row = gid / LPR;
  const int c = gid % LPR;
  float acc = 0.f;
  if (row < rows) {
    const bf16x8 a = as_bf16x8(load_global16(out + row * D + c * 8));
    const bf16x8 g = as_bf16x8(load_global16(dout + row * D + c * 8));
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += (float)a[e] * (float)g[e];
  }
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (row < rows && c == 0) delta[row] = acc;
}

}  // namespace ct
