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

#include "ct_attn_kernels.cuh"

namespace ct {

// ---------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------
template <int D, int HS>
__global__ __launch_bounds__(256) void attn_dq_kernel(AttnParams p) {
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
  const size_t stat_off = ((size_t)work.b * p.S + pos) * p.Hq + work.h;
  const int seg_q = p.seg[(size_t)work.b * p.S + pos];
  const int end_q = p.end ? p.end[(size_t)work.b * p.S + pos] : pos;
  const bool row_valid = seg_q != 0;
  const float lse2 = p.lse[stat_off] * kLog2e;
  const float delta_q = p.delta[stat_off];

  bf16x8 qf[D / 16], dof[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    qf[ks] = scale_bf16x8(as_bf16x8(load_global16(p.q + q_off + 16 * ks + 8 * half)), p.scale);
    dof[ks] = as_bf16x8(load_global16(p.dout + q_off + 16 * ks + 8 * half));
  }

  f32x16 dqacc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db) dqacc[db] = zero16();

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
      f32x16 s[2], dp[2];
      scores_t<D>(sm.k[cur], qf, s);
      scores_t<D>(sm.v[cur], dof, dp);
      const bool interior = tile_is_interior(mine.uniform, mine.end_min, uniform(kb.uniform),
                                             t * kKeyTile + kKeyTile - 1);
      unsigned allow[2] = {0xffffffffu, 0xffffffffu};
      if (!interior) tile_mask(sm.seg[cur], t, seg_q, end_q, row_valid, allow);
#pragma unroll
      for (int kbk = 0; kbk < 2; ++kbk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float prob =
              ((allow[kbk] >> r) & 1u) ? exp2_fast(s[kbk][r] * kLog2e - lse2) : 0.f;
          s[kbk][r] = prob * (dp[kbk][r] - delta_q);
        }
      accumulate_t<D>(sm.k[cur], s, dqacc);
    }

    if (tn <= last) kv_commit<D>(regs, sm.k[cur ^ 1], sm.v[cur ^ 1], sm.seg[cur ^ 1]);
    __syncthreads();
    t = tn;
    cur ^= 1;
  }

  bf16* patch = reinterpret_cast<bf16*>(smem_raw) + w * 32 * D;
  bf16* gbase = p.dq + (((size_t)work.b * p.S + work.rb * 32) * p.Hq + work.h) * D;
  store_rows_t<D>(dqacc, p.scale, patch, gbase, q_row_stride);
}

// ---------------------------------------------------------------------------
// dK / dV
// ---------------------------------------------------------------------------
constexpr int kQueryTile = 32;

template <int D>
struct DkvSmem {
  static constexpr int kTileElems = kQueryTile * D;
  // per stage: Q tile, dO tile, then lse2 / delta (f32) and seg / end (i32) rows
  static constexpr size_t kStageBytes = 2 * kTileElems * sizeof(bf16) + 4 * kQueryTile * 4;
  static constexpr size_t kPatchBytes = 4 * 32 * D * sizeof(bf16);
  static constexpr size_t kBytes =
      (2 * kStageBytes > kPatchBytes) ? 2 * kStageBytes : kPatchBytes;
  bf16* q[2];
  bf16* dout[2];
  float* lse2[2];
  float* delta[2];
  int* seg[2];
  int* end[2];
  CT_DEVICE explicit DkvSmem(char* base) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      char* b = base + s * kStageBytes;
      q[s] = reinterpret_cast<bf16*>(b);
      dout[s] = q[s] + kTileElems;
      lse2[s] = reinterpret_cast<float*>(dout[s] + kTileElems);
      delta[s] = lse2[s] + kQueryTile;
      seg[s] = reinterpret_cast<int*>(delta[s] + kQueryTile);
      end[s] = seg[s] + kQueryTile;
    }
  }
};

template <int D>
struct QdoRegs {
  static constexpr int kChunks = kQueryTile * (D / 8) / 256;
  uint4 q[kChunks];
  uint4 dout[kChunks];
  float lse2, delta;
  int seg, end;
};

template <int D>
CT_DEVICE void qdo_fetch(QdoRegs<D>& r, const AttnParams& p, int b, int h, int qb) {
  constexpr int CPR = D / 8;
  const int tid = threadIdx.x;
#pragma unroll
  for (int n = 0; n < QdoRegs<D>::kChunks; ++n) {
    const int e = tid + 256 * n;
    const int row = e / CPR, c = e % CPR;
    const size_t off = (((size_t)b * p.S + qb * kQueryTile + row) * p.Hq + h) * D + c * 8;
    r.q[n] = load_global16(p.q + off);
    r.dout[n] = load_global16(p.dout + off);
  }
  if (tid < kQueryTile) {
    const int pos = qb * kQueryTile + tid;
    const size_t so = ((size_t)b * p.S + pos) * p.Hq + h;
    r.lse2 = p.lse[so] * kLog2e;
    r.delta = p.delta[so];
    r.seg = p.seg[(size_t)b * p.S + pos];
    r.end = p.end ? p.end[(size_t)b * p.S + pos] : pos;
  }
}

template <int D>
CT_DEVICE void qdo_commit(const QdoRegs<D>& r, const DkvSmem<D>& sm, int stage, float scale) {
  constexpr int CPR = D / 8;
  const int tid = threadIdx.x;
#pragma unroll
  for (int n = 0; n < QdoRegs<D>::kChunks; ++n) {
    const int e = tid + 256 * n;
    const int row = e / CPR, c = e % CPR;
    tile_store_chunk<CPR>(sm.q[stage], row, c, as_uint4(scale_bf16x8(as_bf16x8(r.q[n]), scale)));
    tile_store_chunk<CPR>(sm.dout[stage], row, c, r.dout[n]);
  }
  if (tid < kQueryTile) {
    sm.lse2[stage][tid] = r.lse2;
    sm.delta[stage][tid] = r.delta;
    sm.seg[stage][tid] = r.seg;
    sm.end[stage][tid] = r.end;
  }
}

// X (32 rows of an LDS tile) times register fragments: C[row, key] = sum_d X[row, d] F[key, d].
template <int D>
CT_DEVICE f32x16 rows_times_frags(const bf16* tile, const bf16x8* frags) {
  constexpr int CPR = D / 8;
  const int l = lane_id(), j = l & 31, half = l >> 5;
  f32x16 c = zero16();
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    const bf16x8 a = tile_read_row8<CPR>(tile, j, 2 * ks + half);
    c = mfma32(a, frags[ks], c);
  }
  return c;
}

// acc (32 keys x D) += W^T X, W in accumulator layout (rows = the 32 tile rows,
// cols = keys), X the 32-row LDS tile read transposed.
template <int D>
CT_DEVICE void accumulate_keys(const bf16* tile, const f32x16& wt, f32x16* acc) {
  constexpr int CPR = D / 8;
  const int half = lane_id() >> 5;
#pragma unroll
  for (int step = 0; step < 2; ++step) {
    const bf16x8 aop = pack_acc8(wt, step);
    int rowA, rowB;
    kslot_rows_accum(16 * step, half, rowA, rowB);
#pragma unroll
    for (int db = 0; db < D / 32; ++db) {
      const bf16x8 bop = tile_read_tr8<CPR>(tile, rowA, rowB, db * 32);
      acc[db] = mfma32(aop, bop, acc[db]);
    }
  }
}

// Store a (32 rows x D) accumulator (lanes along D) as bf16 rows via an LDS patch.
template <int D>
CT_DEVICE void store_rows(const f32x16* acc, bf16* patch, bf16* gbase, size_t row_stride) {
  constexpr int CPR = D / 8;
  const int l = lane_id(), j = l & 31, half = l >> 5;
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
    const int col = db * 32 + j;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = acc_row(r, half);
      patch[tile_offset<CPR>(row, col >> 3) + (col & 7)] = (bf16)acc[db][r];
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

template <int D>
__global__ __launch_bounds__(256) void attn_dkv_kernel(AttnParams p) {
  extern __shared__ __align__(16) char smem_raw[];
  DkvSmem<D> sm(smem_raw);

  const int l = lane_id(), j = l & 31, half = l >> 5, w = threadIdx.x >> 6;
  const int nkt = p.S / 128;
  const int total = nkt * p.Hkv * p.B;
  int id = xcd_remap(blockIdx.x, total);
  const int kt = id % nkt;  // early key tiles are seen by the most queries
  id /= nkt;
  const int kvh = id % p.Hkv;
  const int b = id / p.Hkv;
  const int g = p.Hq / p.Hkv;
  const int nrb = p.S / 32;
  const int* meta_b = p.meta + (size_t)b * nrb * kMetaW;

  // Key-side bounds of the 4 row blocks of this workgroup; [4] is this wavefront's.
  int k_min[4], k_max[4], k_uni[4];
  int q_lo = INT_MAX, q_hi = -1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int* m = meta_b + (kt * 4 + i) * kMetaW;
    k_min[i] = uniform(m[kMinNz]);
    k_max[i] = uniform(m[kMaxId]);
    k_uni[i] = uniform(m[kUniform]);
    q_lo = min(q_lo, uniform(m[kQFirst]));
    q_hi = max(q_hi, uniform(m[kQLast]));
  }
  const int my_rb = kt * 4 + w;
  const int my_min = uniform(meta_b[my_rb * kMetaW + kMinNz]);
  const int my_max = uniform(meta_b[my_rb * kMetaW + kMaxId]);
  const int my_uni = uniform(meta_b[my_rb * kMetaW + kUniform]);

  const int key = my_rb * 32 + j;
  const int seg_k = p.seg[(size_t)b * p.S + key];
  const size_t kv_row_stride = (size_t)p.Hkv * D;
  const size_t kv_off = (((size_t)b * p.S + key) * p.Hkv + kvh) * D;

  bf16x8 kf[D / 16], vf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) {
    kf[ks] = as_bf16x8(load_global16(p.k + kv_off + 16 * ks + 8 * half));
    vf[ks] = as_bf16x8(load_global16(p.v + kv_off + 16 * ks + 8 * half));
  }
  f32x16 dkacc[D / 32], dvacc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
    dkacc[db] = zero16();
    dvacc[db] = zero16();
  }

  // Work items: (head of the group, query block) pairs, flattened.
  const int nq = (q_lo <= q_hi) ? (q_hi - q_lo + 1) : 0;
  const int items = nq * g;
  auto item_needed = [&](int it) -> bool {
    const int* m = meta_b + (q_lo + it % nq) * kMetaW;
    const int q_min = m[kMinNz], q_max = m[kMaxId], q_end = m[kEndMax];
    bool any = false;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      any |= blocks_interact(q_min, q_max, q_end, k_min[i], k_max[i], (kt * 4 + i) * 32);
    return any;
  };
  auto next_item = [&](int it) -> int {
    while (it < items && !item_needed(it)) ++it;
    return uniform(it);
  };

  int it = next_item(0);
  if (it < items) {
    QdoRegs<D> regs;
    qdo_fetch<D>(regs, p, b, kvh * g + it / nq, q_lo + it % nq);
    qdo_commit<D>(regs, sm, 0, p.scale);
  }
  __syncthreads();
  int cur = 0;
  while (it < items) {
    const int itn = next_item(it + 1);
    QdoRegs<D> regs;
    if (itn < items) qdo_fetch<D>(regs, p, b, kvh * g + itn / nq, q_lo + itn % nq);

    const int qb = q_lo + it % nq;
    const int* qm = meta_b + qb * kMetaW;
    const int q_min = uniform(qm[kMinNz]), q_max = uniform(qm[kMaxId]),
              q_end_max = uniform(qm[kEndMax]), q_end_min = uniform(qm[kEndMin]),
              q_uni = uniform(qm[kUniform]);
    if (blocks_interact(q_min, q_max, q_end_max, my_min, my_max, my_rb * 32)) {
      f32x16 s = rows_times_frags<D>(sm.q[cur], kf);
      f32x16 dp = rows_times_frags<D>(sm.dout[cur], vf);
      const bool interior = tile_is_interior(q_uni, q_end_min, my_uni, my_rb * 32 + 31);
      f32x16 prob;
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int r0 = 8 * qd + 4 * half;  // first of 4 consecutive query rows
        const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sm.lse2[cur] + r0);
        const f32x4 del4 = *reinterpret_cast<const f32x4*>(sm.delta[cur] + r0);
        const int4 seg4 = *reinterpret_cast<const int4*>(sm.seg[cur] + r0);
        const int4 end4 = *reinterpret_cast<const int4*>(sm.end[cur] + r0);
        const int segs[4] = {seg4.x, seg4.y, seg4.z, seg4.w};
        const int ends[4] = {end4.x, end4.y, end4.z, end4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = 4 * qd + e;
          const bool ok = interior || (segs[e] == seg_k && seg_k != 0 && key <= ends[e]);
          const float pr = ok ? exp2_fast(s[r] * kLog2e - lse4[e]) : 0.f;
          prob[r] = pr;
          dp[r] = pr * (dp[r] - del4[e]);
        }
      }
      accumulate_keys<D>(sm.dout[cur], prob, dvacc);
      accumulate_keys<D>(sm.q[cur], dp, dkacc);
    }

    if (itn < items) qdo_commit<D>(regs, sm, cur ^ 1, p.scale);
    __syncthreads();
    it = itn;
    cur ^= 1;
  }

  bf16* patch = reinterpret_cast<bf16*>(smem_raw) + w * 32 * D;
  const size_t out_off = (((size_t)b * p.S + my_rb * 32) * p.Hkv + kvh) * D;
  store_rows<D>(dkacc, patch, p.dk + out_off, kv_row_stride);
  __builtin_amdgcn_wave_barrier();
  store_rows<D>(dvacc, patch, p.dv + out_off, kv_row_stride);
}

}  // namespace ct
