// Attention kernels for gfx950: forward, delta, dQ and dK/dV.
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
  const int* meta;
  bf16* out;        // forward: written; backward: forward output
  float* lse;
  const bf16* dout;
  float* delta;
  bf16* dq;
  bf16* dk;
  bf16* dv;
  int B, S, Hq, Hkv;
  float scale;      // already rounded to bf16
};

// ---------------------------------------------------------------------------
// K/V tile staging: global -> registers -> swizzled LDS.
// ---------------------------------------------------------------------------
template <int D>
struct KvRegs {
  static constexpr int kChunks = kKeyTile * (D / 8) / 256;
  uint4 k[kChunks];
  uint4 v[kChunks];
  int seg;
};

template <int D>
CT_DEVICE void kv_fetch(KvRegs<D>& r, const bf16* kbase, const bf16* vbase, const int* segb,
                        size_t row_stride, int tile) {
  constexpr int CPR = D / 8;
  const int tid = threadIdx.x;
#pragma unroll
  for (int n = 0; n < KvRegs<D>::kChunks; ++n) {
    const int e = tid + 256 * n;
    const int row = e / CPR, c = e % CPR;
    const size_t off = (size_t)(tile * kKeyTile + row) * row_stride + c * 8;
    r.k[n] = load_global16(kbase + off);
    r.v[n] = load_global16(vbase + off);
  }
  if (tid < kKeyTile) r.seg = segb[tile * kKeyTile + tid];
}

template <int D>
CT_DEVICE void kv_commit(const KvRegs<D>& r, bf16* ktile, bf16* vtile, int* segk) {
  constexpr int CPR = D / 8;
  const int tid = threadIdx.x;
#pragma unroll
  for (int n = 0; n < KvRegs<D>::kChunks; ++n) {
    const int e = tid + 256 * n;
    const int row = e / CPR, c = e % CPR;
    tile_store_chunk<CPR>(ktile, row, c, r.k[n]);
    tile_store_chunk<CPR>(vtile, row, c, r.v[n]);
  }
  if (tid < kKeyTile) segk[tid] = r.seg;
}

// LDS carve-up for the forward / dQ kernels.
template <int D>
struct KvSmem {
  static constexpr int kTileElems = kKeyTile * D;
  static constexpr size_t kBytes = 2 * (2 * kTileElems * sizeof(bf16)) + 2 * kKeyTile * sizeof(int);
  bf16* k[2];
  bf16* v[2];
  int* seg[2];
  CT_DEVICE explicit KvSmem(char* base) {
    bf16* t = reinterpret_cast<bf16*>(base);
    k[0] = t;
    v[0] = t + kTileElems;
    k[1] = t + 2 * kTileElems;
    v[1] = t + 3 * kTileElems;
    seg[0] = reinterpret_cast<int*>(t + 4 * kTileElems);
    seg[1] = seg[0] + kKeyTile;
  }
};

// Decoded position of a workgroup / wavefront in the (batch, head, row block) space.
template <int HS>
struct QueryWork {
  static constexpr int PB = 4 / HS;  // row blocks per workgroup
  int b, h, kvh, qt, rb;
  CT_DEVICE QueryWork(const AttnParams& p) {
    const int nqt = p.S / (32 * PB);
    const int hgroups = p.Hq / HS;
    const int total = nqt * hgroups * p.B;
    int id = xcd_remap(blockIdx.x, total);
    qt = nqt - 1 - (id % nqt);  // longest key ranges first
    id /= nqt;
    const int hg = id % hgroups;
    b = id / hgroups;
    const int w = threadIdx.x >> 6;
    h = hg * HS + (w % HS);
    kvh = (hg * HS) / (p.Hq / p.Hkv);
    rb = qt * PB + (w / HS);
  }
};

// Next tile >= t (and <= last) that any row block of the workgroup visits;
// last + 1 if none.
template <int PB>
CT_DEVICE int next_tile(const int* meta_b, const QueryBlockBounds* wq, int t, int last) {
  for (; t <= last; ++t) {
    const KeyTileBounds kb = key_tile_bounds(meta_b, t);
    bool any = false;
#pragma unroll
    for (int i = 0; i < PB; ++i)
      any |= blocks_interact(wq[i].min_nz, wq[i].max_id, wq[i].end_max, kb.min_nz, kb.max_id,
                             t * kKeyTile);
    if (any) break;
  }
  return uniform(t);
}

// S^T (two 32-key blocks) = K_tile Q^T for this wavefront's 32 queries.
template <int D>
CT_DEVICE void scores_t(const bf16* ktile, const bf16x8* qf, f32x16* s) {
  constexpr int CPR = D / 8;
  const int l = lane_id(), j = l & 31, half = l >> 5;
  s[0] = zero16();
  s[1] = zero16();
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const bf16x8 a = tile_read_row8<CPR>(ktile, kb * 32 + j, 2 * ks + half);
      s[kb] = mfma32(a, qf[ks], s[kb]);
    }
  }
}

// allowed(query of this lane, key held by register r of block kb)?  Writes a
// 32-bit mask per block: bit r set = allowed.
CT_DEVICE void tile_mask(const int* segk, int tile, int seg_q, int end_q, bool row_valid,
                         unsigned* allow) {
  const int half = lane_id() >> 5;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    unsigned bits = 0;
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const int k0 = kb * 32 + 8 * qd + 4 * half;
      const int4 sk = *reinterpret_cast<const int4*>(segk + k0);
      const int key = tile * kKeyTile + k0;
      bits |= (unsigned)(sk.x == seg_q && key + 0 <= end_q) << (4 * qd + 0);
      bits |= (unsigned)(sk.y == seg_q && key + 1 <= end_q) << (4 * qd + 1);
      bits |= (unsigned)(sk.z == seg_q && key + 2 <= end_q) << (4 * qd + 2);
      bits |= (unsigned)(sk.w == seg_q && key + 3 <= end_q) << (4 * qd + 3);
    }
    allow[kb] = row_valid ? bits : 0u;
  }
}

// acc (D x 32 queries, transposed) += X^T W^T where X is a 64-row LDS tile read
// transposed and W^T are the packed accumulator-layout weights wt[2].
template <int D>
CT_DEVICE void accumulate_t(const bf16* tile, const f32x16* wt, f32x16* acc) {
  constexpr int CPR = D / 8;
  const int half = lane_id() >> 5;
#pragma unroll
  for (int step = 0; step < 4; ++step) {
    const bf16x8 bop = pack_acc8(wt[step >> 1], step & 1);
    int rowA, rowB;
    kslot_rows_accum(16 * step, half, rowA, rowB);
#pragma unroll
    for (int db = 0; db < D / 32; ++db) {
      const bf16x8 a = tile_read_tr8<CPR>(tile, rowA, rowB, db * 32);
      acc[db] = mfma32(a, bop, acc[db]);
    }
  }
}

// Write a transposed accumulator (D x 32 rows) as bf16 rows of D elements to
// global memory, staged through this wavefront's private LDS patch so that
// the global stores are 16 bytes per lane and contiguous per row.
template <int D>
CT_DEVICE void store_rows_t(const f32x16* acc, float row_scale, bf16* patch, bf16* gbase,
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
      *reinterpret_cast<bf16x4*>(patch + tile_offset<CPR>(j, d0 >> 3) + (d0 & 4)) = pk;
    }
  }
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int n = 0; n < 32 * CPR / 64; ++n) {
    const int e = l + 64 * n;
    const int row = e / CPR, c = e % CPR;
    const bf16x8 val = tile_read_row8<CPR>(patch, row, c);
    *reinterpret_cast<uint4*>(gbase + (size_t)row * row_stride + c * 8) = as_uint4(val);
  }
}

// ---------------------------------------------------------------------------
// Forward
// ---------------------------------------------------------------------------
template <int D, int HS>
__global__ __launch_bounds__(256) void attn_fwd_kernel(AttnParams p) {
  constexpr int PB = 4 / HS;
  extern __shared__ __align__(16) char smem_raw[];
  KvSmem<D> sm(smem_raw);

  const QueryWork<HS> work(p);
  const int l = lane_id(), j = l & 31, half = l >> 5, w = threadIdx.x >> 6;
  const int nrb = p.S / 32;
  const int* meta_b = p.meta + (size_t)work.b * nrb * kMetaW;
  const int pos = work.rb * 32 + j;

  QueryBlockBounds wq[PB];
#pragma unroll
  for (int i = 0; i < PB; ++i) wq[i] = query_block_bounds(meta_b, work.qt * PB + i);
  const QueryBlockBounds mine = query_block_bounds(meta_b, work.rb);
  int first = INT_MAX, last = -1;
#pragma unroll
  for (int i = 0; i < PB; ++i) {
    first = min(first, wq[i].kv_first);
    last = max(last, wq[i].kv_last);
  }

  const size_t q_row_stride = (size_t)p.Hq * D;
  const size_t kv_row_stride = (size_t)p.Hkv * D;
  const size_t q_off = (((size_t)work.b * p.S + pos) * p.Hq + work.h) * D;
  const int seg_q = p.seg[(size_t)work.b * p.S + pos];
  const int end_q = p.end ? p.end[(size_t)work.b * p.S + pos] : pos;
  const bool row_valid = seg_q != 0;

  bf16x8 qf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks)
    qf[ks] = scale_bf16x8(as_bf16x8(load_global16(p.q + q_off + 16 * ks + 8 * half)), p.scale);

  f32x16 oacc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db) oacc[db] = zero16();
  float m_run = kNegInf;  // running max, log2 domain
  float l_run = 0.f;      // this lane's share of the running sum

  const bf16* kbase = p.k + ((size_t)work.b * p.S * p.Hkv + work.kvh) * D;
  const bf16* vbase = p.v + ((size_t)work.b * p.S * p.Hkv + work.kvh) * D;
  const int* segb = p.seg + (size_t)work.b * p.S;

  int t = (first <= last) ? next_tile<PB>(meta_b, wq, first, last) : last + 1;
  if (t <= last) {
    KvRegs<D> regs;
    kv_fetch<D>(regs, kbase, vbase, segb, kv_row_stride, t);
    kv_commit<D>(regs, sm.k[0], sm.v[0], sm.seg[0]);
  }
  __syncthreads();
  int cur = 0;
  while (t <= last) {
    const int tn = next_tile<PB>(meta_b, wq, t + 1, last);
    KvRegs<D> regs;
    if (tn <= last) kv_fetch<D>(regs, kbase, vbase, segb, kv_row_stride, tn);

    const KeyTileBounds kb = key_tile_bounds(meta_b, t);
    if (blocks_interact(mine.min_nz, mine.max_id, mine.end_max, uniform(kb.min_nz),
                        uniform(kb.max_id), t * kKeyTile)) {
      f32x16 s[2];
      scores_t<D>(sm.k[cur], qf, s);
      const bool interior = tile_is_interior(mine.uniform, mine.end_min, uniform(kb.uniform),
                                             t * kKeyTile + kKeyTile - 1);
      float mx = kNegInf;
      if (interior) {
#pragma unroll
        for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            s[kbk][r] *= kLog2e;
            mx = fmaxf(mx, s[kbk][r]);
          }
      } else {
        unsigned allow[2];
        tile_mask(sm.seg[cur], t, seg_q, end_q, row_valid, allow);
#pragma unroll
        for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            s[kbk][r] = ((allow[kbk] >> r) & 1u) ? s[kbk][r] * kLog2e : kNegInf;
            mx = fmaxf(mx, s[kbk][r]);
          }
      }
      mx = fmaxf(mx, xor32(mx));
      const float m_new = fmaxf(m_run, mx);
      const float m_use = (m_new == kNegInf) ? 0.f : m_new;
      const float alpha = exp2_fast(m_run - m_use);
      float psum = 0.f;
#pragma unroll
      for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          s[kbk][r] = exp2_fast(s[kbk][r] - m_use);
          psum += s[kbk][r];
        }
      l_run = l_run * alpha + psum;
      m_run = m_new;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
      accumulate_t<D>(sm.v[cur], s, oacc);
    }

    if (tn <= last) kv_commit<D>(regs, sm.k[cur ^ 1], sm.v[cur ^ 1], sm.seg[cur ^ 1]);
    __syncthreads();
    t = tn;
    cur ^= 1;
  }

  const float l_tot = l_run + xor32(l_run);
  const bool has = l_tot > 0.f;
  const float inv = has ? 1.f / l_tot : 0.f;
  if (half == 0)
    p.lse[((size_t)work.b * p.S + pos) * p.Hq + work.h] =
        has ? (__logf(l_tot) + m_run * kLn2) : 0.f;
  bf16* patch = reinterpret_cast<bf16*>(smem_raw) + w * 32 * D;
  bf16* obase = p.out + (((size_t)work.b * p.S + work.rb * 32) * p.Hq + work.h) * D;
  // store_rows_t applies one scale per lane = per query row (lane j <-> row j).
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
