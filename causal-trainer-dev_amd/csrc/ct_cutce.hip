// Projection-fused cut cross-entropy for gfx950: kernels and C ABI.
//
// Forward (logits never reach memory):
//   index    stable list of active rows (weight != 0) -> gather indices
//   stats    persistent GEMM workgroups: logits^T tile = head_tile^T hidden_tile^T,
//            folded on the fly into per-row running (max, sum exp, target logit)
//            for one (vocab chunk, row block) unit at a time
//   merge    combine the vocab chunks per row -> lse, weighted loss, block sums
//   finalize fixed-order sum of the block sums -> nll_sum, weight_sum
// Backward:
//   dlogits  G = w * dy * (exp(logits - lse) - onehot), rounded to bf16, written
//            vocabulary-major to a workspace slab G^T [vocab slab, rows]
//   dhidden  dHidden = G head^T
//   dhead    dHead   = hidden^T G
// The reference recomputes the logits in both backward kernels
// (src/kernels/cut_cross_entropy.py:258, :383); here G is formed once and shared,
// which keeps the reference's rounding points (G is cast to bf16 before both
// products, :272, :396). Its logits come either from a second GEMM (4 GEMMs
// instead of the reference's 5) or, when the caller lends the forward a cache,
// from the f32 logits the forward left there (3 GEMMs, the algorithmic count).
// The cache is vocabulary-major [vocab, rows] like G^T: in the transposed tile
// the GEMMs produce, the lanes of a wavefront run along the rows, so both are
// written with contiguous stores.
#include <mutex>

#include "ct_error.h"
#include "ct_gemm.hip.h"

namespace ct {

constexpr int kBK = kGemmBK;
constexpr int kTilesPerChunk = 4;  // vocab tiles per stats work unit
#ifndef CT_CUTCE_SWEEP
#define CT_CUTCE_SWEEP 1
#endif
constexpr bool kSweepUnits = CT_CUTCE_SWEEP != 0;  // unit order of the two projection kernels
constexpr float kNegInfF = -__builtin_inff();

struct CutceHeader {
  int n_act;
  int counter;
  // per-XCD work counters: set 0 statistics kernel / hidden gradient, set 1 head gradient,
  // set 2 the dlogits kernel that recomputes the projection
  int xcd_counter[3][8];
  int pad[6];
};

// Clears counter sets 0 and 1 (called by workgroup 0 of a kernel that runs before their users).
CT_DEVICE void reset_unit_counters(CutceHeader* header) {
  if (threadIdx.x < 16) (&header->xcd_counter[0][0])[threadIdx.x] = 0;
}
// Clears counter set 2.
CT_DEVICE void reset_dlogits_counters(CutceHeader* header) {
  if (threadIdx.x < 8) header->xcd_counter[2][threadIdx.x] = 0;
}

// Work order of the persistent GEMM kernels. A unit is a pair (a, b) of operand tile indices,
// a < a_count, b < b_count; every unit is one 256 x 256 GEMM tile (or a run of them) that
// reads tile a of one operand and tile b of the other. Each XCD has its own L2, so the
// workgroups of one XCD should work at the same time on units that share operands: the
// (a, b) grid is walked in blocks of kA x kB = 32 units (the 32 compute units of an XCD: 4 + 8
// operand tiles feed 32 GEMM tiles), the sequence of blocks is cut into 8 equal ranges, and an
// XCD takes the units of its range through its own counter. Indices that fall outside the
// grid (ragged edges) are skipped. An XCD that runs dry helps the next one.
//
// Sweep mode (the two projection kernels, a = vocabulary chunk, b = row block): XCD x owns the
// row blocks x, x + 8, ... and walks (a, its row blocks) with a as the slow index, so all eight
// XCDs are on the same few vocabulary chunks at the same time. The head is the large operand
// (1 GB against 0.1 GB of hidden rows): with every XCD on the same chunk it leaves HBM about once
// per pass, and the other XCDs find it in the memory-side cache; in block mode each XCD streams
// its own range of the vocabulary and the head is read from HBM once per 8 row blocks.
struct XcdUnits {
  static constexpr int kA = 4, kB = 8, kXcds = 8;
  int* counters;
  int a_count, b_count, b_groups, padded_total, per_xcd, my_xcd;
  int helping;  // how many XCDs further the counter in use belongs to
  bool sweep;
  CT_DEVICE void init(int* counters_, int a_count_, int b_count_, bool sweep_ = false) {
    sweep = sweep_;
    counters = counters_;
    a_count = a_count_;
    b_count = b_count_;
    b_groups = (b_count + kB - 1) / kB;
    padded_total = ((a_count + kA - 1) / kA) * b_groups * kA * kB;
    per_xcd = (padded_total + kXcds - 1) / kXcds;
    unsigned xcc_id;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc_id));
    my_xcd = (int)(xcc_id & 7u);
    helping = 0;
  }
  // Called by all threads of the workgroup (contains barriers); false when nothing is left.
  CT_DEVICE bool next_sweep(int& a, int& b, int* lds_slot) {
    while (helping < kXcds) {
      const int x = (my_xcd + helping) % kXcds;
      const int mine = x < b_count ? (b_count - x + kXcds - 1) / kXcds : 0;  // row blocks of XCD x
      if (threadIdx.x == 0) *lds_slot = mine ? atomicAdd(&counters[x], 1) : 0;
      __syncthreads();
      const int local = uniform(*lds_slot);  // scalar from here on: unit indices feed scalar address arithmetic
      __syncthreads();
      if (mine && local < a_count * mine) {
        a = local / mine;
        b = x + kXcds * (local % mine);
        return true;
      }
      ++helping;
    }
    return false;
  }
  CT_DEVICE bool next(int& a, int& b, int* lds_slot) {
    if (sweep) return next_sweep(a, b, lds_slot);
    for (;;) {
      int index = -1;
      while (helping < kXcds) {
        const int x = (my_xcd + helping) % kXcds;
        if (threadIdx.x == 0) *lds_slot = atomicAdd(&counters[x], 1);
        __syncthreads();
        const int local = uniform(*lds_slot);  // scalar from here on: unit indices feed scalar address arithmetic
        __syncthreads();
        if (local < per_xcd && x * per_xcd + local < padded_total) {
          index = x * per_xcd + local;
          break;
        }
        ++helping;
      }
      if (index < 0) return false;
      const int in_block = index % (kA * kB), block = index / (kA * kB);
      a = (block / b_groups) * kA + in_block / kB;
      b = (block % b_groups) * kB + in_block % kB;
      if (a < a_count && b < b_count) return true;
    }
  }
};

struct CutceParams {
  const bf16* hidden;
  const bf16* head;
  const int* targets;
  const float* weights;
  int N, d, V, n_pad;
  int* idx;
  CutceHeader* header;
  bool hidden_aligned, head_aligned;
};

// ---------------------------------------------------------------------------
// index: stable compaction of active rows
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void cutce_index_kernel(const float* weights, int N, int n_pad,
                                                           int compact, int* idx,
                                                           CutceHeader* header) {
  __shared__ int wave_total[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
  if (!compact) {
    for (int i = tid; i < n_pad; i += blockDim.x) idx[i] = i < N ? i : 0;
    if (tid == 0) {
      header->n_act = N;
      header->counter = 0;
    }
    reset_unit_counters(header);
    reset_dlogits_counters(header);
    return;
  }
  int carry = 0;
  for (int base = 0; base < N; base += blockDim.x) {
    const int i = base + tid;
    const bool active = i < N && weights[i] != 0.f;
    const unsigned long long ballot = __ballot(active);
    const int before = __popcll(ballot & ((1ull << lane) - 1ull));
    if (lane == 0) wave_total[wave] = __popcll(ballot);
    __syncthreads();
    int offset = 0, all = 0;
    for (int k = 0; k < nwaves; ++k) {
      if (k < wave) offset += wave_total[k];
      all += wave_total[k];
    }
    if (active) idx[carry + offset + before] = i;
    carry += all;
    __syncthreads();
  }
  __syncthreads();
  const int filler = carry > 0 ? idx[0] : 0;  // keeps gathers past the end on a live row
  for (int i = carry + tid; i < n_pad; i += blockDim.x) idx[i] = filler;
  if (tid == 0) {
    header->n_act = carry;
    header->counter = 0;
  }
  reset_unit_counters(header);
  reset_dlogits_counters(header);
}

// ---------------------------------------------------------------------------
// stats
// ---------------------------------------------------------------------------
CT_DEVICE void merge_stats(float& m, float& s, float m_o, float s_o) {
  const float m_new = fmaxf(m, m_o);
  const float m_use = (m_new == kNegInfF) ? 0.f : m_new;
  s = s * exp2_fast(m - m_use) + s_o * exp2_fast(m_o - m_use);
  m = m_new;
}

template <bool CACHE>
__global__ __launch_bounds__(256) void cutce_stats_kernel(CutceParams p, float* part, int chunks,
                                                          float* cache) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr smem = lds_address_of(smem_raw);
  __shared__ int unit_s;
  const int tid = threadIdx.x, l = tid & 63, j = l & 31, half = l >> 5, w = tid >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  const int vocab_tiles = (p.V + kGemmTile - 1) / kGemmTile;
  const int n_act = p.header->n_act;

  // units: (vocabulary chunk, row block)
  const int active_blocks = (n_act + kGemmTile - 1) / kGemmTile;
  XcdUnits units;
  units.init(p.header->xcd_counter[0], chunks, active_blocks, kSweepUnits);
  int chunk, rb;
  while (units.next(chunk, rb, &unit_s)) {
    const int n0 = rb * kGemmTile;
    const int my_slot = n0 + tid;
    const int active = my_slot < n_act && p.weights[p.idx[my_slot]] != 0.f;
    if (!__syncthreads_or(active)) continue;  // no row of this block carries weight

    // Rows are interleaved in the tile (KcLoader): column block nb of lane j is row slot
    // n0 + wn + 4 j + nb, so a lane owns 4 consecutive slots.
    int tgt[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      const int slot = n0 + wn + 4 * j + nb;
      tgt[nb] = slot < n_act ? p.targets[p.idx[slot]] : -1;
    }
    float m2[4], sum[4], tl[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      m2[nb] = kNegInfF;
      sum[nb] = 0.f;
      tl[nb] = 0.f;
    }
    KcLoader B;
    B.init(p.hidden, p.d, p.idx, n0, n_act, p.d, p.hidden_aligned, true, true);

    const int vt_end = min((chunk + 1) * kTilesPerChunk, vocab_tiles);
    for (int vt = chunk * kTilesPerChunk; vt < vt_end; ++vt) {
      const int v0 = vt * kGemmTile;
      McLoader A;
      A.init(p.head, p.V, nullptr, v0, p.V, p.d, p.head_aligned);
      GemmAcc acc;
      acc.clear();
      gemm_tile(A, B, 0, p.d, smem, acc);

      const int vbase = v0 + wm + 4 * half;  // vocab id of (i, r) = vbase + 32 i + 8 (r/4) + r%4
      const bool ragged = v0 + kGemmTile > p.V;
      if constexpr (CACHE) {
        // cache^T[v][slot]: a lane stores its 4 consecutive slots with one 16-byte access, 32
        // lanes = 512 contiguous bytes. Address = wave-uniform tile origin + uniform row offset +
        // a 32-bit lane offset, so the stores need no per-store vector address arithmetic.
        float* origin = cache + (size_t)(v0 + uniform(wm)) * p.n_pad + n0 + uniform(wn);
        const unsigned lane_off = (unsigned)(4 * half * p.n_pad + 4 * j) * 4u;  // bytes
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float* row = origin + (size_t)(32 * i + 8 * (r >> 2) + (r & 3)) * p.n_pad;
            const f32x4 quad = {acc.c[i][0][r], acc.c[i][1][r], acc.c[i][2][r], acc.c[i][3][r]};
            store_global16_s<0>(row, lane_off, quad);
          }
      }
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        float tmax = kNegInfF;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            if (ragged && vbase + 32 * i + 8 * (r >> 2) + (r & 3) >= p.V) acc.c[i][nb][r] = kNegInfF;
            tmax = fmaxf(tmax, acc.c[i][nb][r]);
          }
        const int rel = tgt[nb] - (v0 + wm);
        if (__any(rel >= 0 && rel < 128)) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if (vbase + 32 * i + 8 * (r >> 2) + (r & 3) == tgt[nb]) tl[nb] += acc.c[i][nb][r];
        }
        const float m_new = fmaxf(m2[nb], tmax * kLog2e);
        const float m_use = (m_new == kNegInfF) ? 0.f : m_new;
        float add = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) add += exp2_fast(acc.c[i][nb][r] * kLog2e - m_use);
        sum[nb] = sum[nb] * exp2_fast(m2[nb] - m_use) + add;
        m2[nb] = m_new;
      }
    }

    // lanes l and l^32 hold the same rows; then the two wavefronts with equal wn.
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      merge_stats(m2[nb], sum[nb], xor32(m2[nb]), xor32(sum[nb]));
      tl[nb] += xor32(tl[nb]);
    }
    float* exch = reinterpret_cast<float*>(smem_raw);  // [2 wn][128 rows][3]
    if (wm != 0 && half == 0) {
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        float* e = exch + ((w & 1) * 128 + 32 * nb + j) * 3;
        e[0] = m2[nb];
        e[1] = sum[nb];
        e[2] = tl[nb];
      }
    }
    __syncthreads();
    if (wm == 0 && half == 0) {
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        const float* e = exch + ((w & 1) * 128 + 32 * nb + j) * 3;
        merge_stats(m2[nb], sum[nb], e[0], e[1]);
        tl[nb] += e[2];
        float* out = part + ((size_t)chunk * p.n_pad + n0 + wn + 4 * j + nb) * 3;
        out[0] = m2[nb];
        out[1] = sum[nb];
        out[2] = tl[nb];
      }
    }
    // the barrier at the top of the loop orders these LDS reads before the next GEMM
  }
}

// ---------------------------------------------------------------------------
// merge + finalize
// ---------------------------------------------------------------------------
// A workgroup merges the per-chunk partials of kMergeSlots row slots: kMergeParts threads per slot
// each walk every kMergeParts-th vocabulary chunk (so a row's chain of dependent loads is an
// eighth as long and eight times as many loads are in flight: the pass is bound by the bytes of
// the partials, not by their latency), then the parts are combined in a fixed order.
constexpr int kMergeSlots = 32, kMergeParts = 8;
__global__ __launch_bounds__(kMergeSlots * kMergeParts) void cutce_merge_kernel(CutceParams p, const float* part,
                                                                                int chunks, float* lse_out,
                                                                                double* block_sums) {
  __shared__ float exch[kMergeParts][kMergeSlots][3];
  __shared__ double red[2][kMergeSlots];
  const int tid = threadIdx.x, lane_slot = tid % kMergeSlots, piece = tid / kMergeSlots;
  const int slot = blockIdx.x * kMergeSlots + lane_slot;
  const int n_act = p.header->n_act;
  double loss = 0.0, wsum = 0.0;
  if (piece == 0 && slot < p.N) {
    const float wi = p.weights[slot];
    wsum = (double)wi;
    if (wi == 0.f) lse_out[slot] = 0.f;
  }
  int row = 0;
  float wr = 0.f;
  if (slot < n_act) {
    row = p.idx[slot];
    wr = p.weights[row];
  }
  float m = kNegInfF, s = 0.f, t = 0.f;
  if (wr != 0.f) {
    for (int c = piece; c < chunks; c += kMergeParts) {
      const float* e = part + ((size_t)c * p.n_pad + slot) * 3;
      merge_stats(m, s, e[0], e[1]);
      t += e[2];
    }
  }
  exch[piece][lane_slot][0] = m;
  exch[piece][lane_slot][1] = s;
  exch[piece][lane_slot][2] = t;
  __syncthreads();
  if (piece == 0) {
    if (wr != 0.f) {
      for (int k = 1; k < kMergeParts; ++k) {
        merge_stats(m, s, exch[k][lane_slot][0], exch[k][lane_slot][1]);
        t += exch[k][lane_slot][2];
      }
      const float lse = (__log2f(s) + m) * kLn2;
      lse_out[row] = lse;
      loss = (double)wr * ((double)lse - (double)t);
    }
    red[0][lane_slot] = loss;
    red[1][lane_slot] = wsum;
  }
  __syncthreads();
  if (tid == 0) {
    double loss_sum = 0.0, weight_sum = 0.0;
    for (int k = 0; k < kMergeSlots; ++k) {  // fixed order
      loss_sum += red[0][k];
      weight_sum += red[1][k];
    }
    block_sums[2 * blockIdx.x + 0] = loss_sum;
    block_sums[2 * blockIdx.x + 1] = weight_sum;
  }
}

__global__ __launch_bounds__(64) void cutce_finalize_kernel(const double* block_sums, int blocks,
                                                            float* nll_sum, float* weight_sum) {
  // lane l adds the blocks l, l + 64, ... in order, then the lanes are added in order: the
  // result does not depend on timing
  __shared__ double red[2][64];
  double loss = 0.0, wsum = 0.0;
  for (int b = threadIdx.x; b < blocks; b += 64) {
    loss += block_sums[2 * b];
    wsum += block_sums[2 * b + 1];
  }
  red[0][threadIdx.x] = loss;
  red[1][threadIdx.x] = wsum;
  __syncthreads();
  if (threadIdx.x != 0) return;
  loss = 0.0;
  wsum = 0.0;
  for (int k = 0; k < 64; ++k) {
    loss += red[0][k];
    wsum += red[1][k];
  }
  *nll_sum = (float)loss;
  *weight_sum = (float)wsum;
}

// ---------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------
// dHidden rows of ignored tokens are exactly zero.
__global__ __launch_bounds__(256) void cutce_zero_rows_kernel(const float* weights, int N, int d,
                                                              bf16* dhidden) {
  const int row = blockIdx.x;
  if (row >= N || weights[row] != 0.f) return;
  u32x4* dst = reinterpret_cast<u32x4*>(dhidden + (size_t)row * d);
  for (int c = threadIdx.x; c < d / 8; c += 256) dst[c] = u32x4{0u, 0u, 0u, 0u};
}

// packed[slot] = hidden[idx[slot]] for the slots of every started 256-slot block. The head
// gradient contracts over slots; with the rows packed its operand tiles are plain strided
// copies instead of a gather through idx at every step. (idx repeats the first active row
// past n_act, so the padding rows hold finite values; their G^T entries are zero.)
__global__ __launch_bounds__(256) void cutce_pack_rows_kernel(CutceParams p, bf16* packed) {
  const int slot = blockIdx.x;
  const int n_act = p.header->n_act;
  if (slot >= (n_act + kGemmTile - 1) / kGemmTile * kGemmTile) return;
  const bf16* src = p.hidden + (size_t)p.idx[slot] * p.d;
  bf16* dst = packed + (size_t)slot * p.d;
  if (p.hidden_aligned) {
    for (int c = threadIdx.x; c < p.d / 8; c += 256)
      reinterpret_cast<u32x4*>(dst)[c] = reinterpret_cast<const u32x4*>(src)[c];
  } else {
    for (int c = threadIdx.x; c < p.d; c += 256) dst[c] = src[c];
  }
}

// Per-slot constants of the backward: (w dy, lse log2 e, target), zeros / -1 past the active rows.
struct CutceRowParams {
  float* fac;
  float* lse2;
  int* tgt;
};

__global__ __launch_bounds__(256) void cutce_rowparams_kernel(CutceParams p, const float* lse,
                                                              const float* dy, CutceRowParams rp) {
  const int slot = blockIdx.x * 256 + threadIdx.x;
  if (slot >= p.n_pad) return;
  // A slot without weight gets factor 0 and lse = +inf: exp2(x - inf) is exactly 0 for every finite
  // logit, so the gradient formula gives 0 for it without a per-element test.
  float f = 0.f, l2 = __builtin_inff();
  int t = -1;
  if (slot < p.header->n_act) {
    const int row = p.idx[slot];
    const float wr = p.weights[row];
    if (wr != 0.f) {
      f = wr * dy[0];
      l2 = lse[row] * kLog2e;
      t = p.targets[row];
    }
  }
  rp.fac[slot] = f;
  rp.lse2[slot] = l2;
  rp.tgt[slot] = t;
}

CT_DEVICE float dlogit(float logit, float fac, float lse2, int tgt, int v) {
  return fac * (exp2_fast(logit * kLog2e - lse2) - (v == tgt ? 1.f : 0.f));
}

// G^T[v - slab0][slot], logits recomputed (transposed tile as in the statistics kernel: rows =
// vocabulary, lanes = row slots). Persistent like the statistics kernel and with its unit order:
// a unit is kTilesPerChunk vocabulary tiles of the slab times one block of 256 active rows.
__global__ __launch_bounds__(256) void cutce_dlogits_kernel(CutceParams p, CutceRowParams rp,
                                                            int slab0, int slab_tiles, bf16* G) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr smem = lds_address_of(smem_raw);
  __shared__ int unit_s;
  const int tid = threadIdx.x, l = tid & 63, j = l & 31, half = l >> 5, w = tid >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  const int n_act = p.header->n_act;
  // the two GEMM kernels that follow start from fresh work counters
  if (blockIdx.x == 0) reset_unit_counters(p.header);
  const int active_blocks = (n_act + kGemmTile - 1) / kGemmTile;  // G^T columns past them are never read
  const int chunks = (slab_tiles + kTilesPerChunk - 1) / kTilesPerChunk;
  XcdUnits units;
  units.init(p.header->xcd_counter[2], chunks, active_blocks, kSweepUnits);
  int chunk, rb;
  while (units.next(chunk, rb, &unit_s)) {
    const int n0 = rb * kGemmTile;
    // Rows are interleaved in the tile (KcLoader): column block nb of lane j is row slot
    // n0 + wn + 4 j + nb, so a lane owns 4 consecutive slots of G^T and stores them together.
    const int slot4 = n0 + wn + 4 * j;
    const f32x4 fac = *reinterpret_cast<const f32x4*>(rp.fac + slot4);
    const f32x4 lse2 = *reinterpret_cast<const f32x4*>(rp.lse2 + slot4);
    const i32x4 tgt = *reinterpret_cast<const i32x4*>(rp.tgt + slot4);
    KcLoader B;
    B.init(p.hidden, p.d, p.idx, n0, n_act, p.d, p.hidden_aligned, true, true);
    const int vt_end = min((chunk + 1) * kTilesPerChunk, slab_tiles);
    for (int vt = chunk * kTilesPerChunk; vt < vt_end; ++vt) {
      const int v0 = slab0 + vt * kGemmTile;
      McLoader A;
      A.init(p.head, p.V, nullptr, v0, p.V, p.d, p.head_aligned);
      GemmAcc acc;
      acc.clear();
      gemm_tile(A, B, 0, p.d, smem, acc);

      bf16* origin = G + (size_t)(v0 - slab0 + uniform(wm)) * p.n_pad + n0 + uniform(wn);
      const unsigned lane_off = (unsigned)(4 * half * p.n_pad + 4 * j) * 2u;  // bytes
      // Most tiles hold no target of the wavefront's rows and lie inside the vocabulary: there the
      // gradient is factor * softmax, three instructions per element. (Slots without weight have
      // factor 0 and lse = +inf.)
      bool target_here = false;
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) target_here |= (unsigned)(tgt[nb] - (v0 + wm)) < 128u;
      const bool plain = v0 + kGemmTile <= p.V && !__any(target_here);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int vrel = 32 * i + 8 * (r >> 2) + (r & 3);
          const int v = v0 + wm + 4 * half + vrel;
          bf16x4 quad;
          if (plain) {
#pragma unroll
            for (int nb = 0; nb < 4; ++nb)
              quad[nb] = (bf16)(fac[nb] * exp2_fast(acc.c[i][nb][r] * kLog2e - lse2[nb]));
          } else {
#pragma unroll
            for (int nb = 0; nb < 4; ++nb)
              quad[nb] = (bf16)((fac[nb] != 0.f && v < p.V)
                                    ? dlogit(acc.c[i][nb][r], fac[nb], lse2[nb], tgt[nb], v) : 0.f);
          }
          store_global8_s<0>(origin + (size_t)vrel * p.n_pad, lane_off, quad);
        }
    }
  }
}

// Same G^T from the f32 logits the forward left in its cache: one pass over memory. A thread
// owns 8 slots and walks kDlogitsRows vocabulary rows with them, so the per-slot constants
// (factor, lse, target: 96 bytes per thread) are loaded once per kDlogitsRows * 32 bytes of
// logits and all of a thread's logits loads are in flight together.
// grid = (slab rows / kDlogitsRows, ceil(n_pad / 2048)).
constexpr int kDlogitsRows = 8;
__global__ __launch_bounds__(256) void cutce_dlogits_cached_kernel(CutceParams p, CutceRowParams rp,
                                                                   const float* cache, int slab0,
                                                                   bf16* G) {
  const int vrel0 = blockIdx.x * kDlogitsRows;
  const int slot0 = (blockIdx.y * 256 + threadIdx.x) * 8;
  // the two GEMM kernels that follow start from fresh work counters
  if (blockIdx.x == 0 && blockIdx.y == 0) reset_unit_counters(p.header);
  const int n_act = p.header->n_act;
  if (slot0 >= (n_act + kGemmTile - 1) / kGemmTile * kGemmTile) return;
  const f32x4 f0 = *reinterpret_cast<const f32x4*>(rp.fac + slot0);
  const f32x4 f1 = *reinterpret_cast<const f32x4*>(rp.fac + slot0 + 4);
  const f32x4 l0 = *reinterpret_cast<const f32x4*>(rp.lse2 + slot0);
  const f32x4 l1 = *reinterpret_cast<const f32x4*>(rp.lse2 + slot0 + 4);
  const i32x4 t0 = *reinterpret_cast<const i32x4*>(rp.tgt + slot0);
  const i32x4 t1 = *reinterpret_cast<const i32x4*>(rp.tgt + slot0 + 4);
  f32x4 a[kDlogitsRows], b[kDlogitsRows];
#pragma unroll
  for (int r = 0; r < kDlogitsRows; ++r) {
    // rows past the vocabulary read the last row (the value is not used)
    const float* src = cache + (size_t)min(slab0 + vrel0 + r, p.V - 1) * p.n_pad + slot0;
    a[r] = *reinterpret_cast<const f32x4*>(src);
    b[r] = *reinterpret_cast<const f32x4*>(src + 4);
  }
#pragma unroll
  for (int r = 0; r < kDlogitsRows; ++r) {
    const int v = slab0 + vrel0 + r;
    bf16x8 out;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      out[e] = (bf16)((f0[e] != 0.f && v < p.V) ? dlogit(a[r][e], f0[e], l0[e], t0[e], v) : 0.f);
      out[4 + e] = (bf16)((f1[e] != 0.f && v < p.V) ? dlogit(b[r][e], f1[e], l1[e], t1[e], v) : 0.f);
    }
    store_global16(G + (size_t)(vrel0 + r) * p.n_pad + slot0, as_u32x4(out));
  }
}

// dHidden[idx[slot], n] (+)= sum_v G^T[v, slot] head[n, slab0 + v]: the workgroup's share of the
// units, pulled from counter set 0.
CT_DEVICE void dhidden_units(const CutceParams& p, const bf16* G, int slab0, int slab_width, int mode,
                             float* dh_acc, bf16* dhidden, const lds_addr smem) {
  // mode: 0 = single slab (store bf16), 1 = first slab (store f32), 2 = middle
  // slab (add f32), 3 = last slab (add, store bf16)
  const int tid = threadIdx.x, l = tid & 63, j = l & 31, half = l >> 5, w = tid >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  const int col_blocks = (p.d + kGemmTile - 1) / kGemmTile;
  const int n_act = p.header->n_act;
  __shared__ int unit_s;
  // the dlogits kernel of the next vocabulary slab starts from fresh work counters
  if (blockIdx.x == 0) reset_dlogits_counters(p.header);
  // units: (row block, column block) over the started row blocks
  XcdUnits units;
  units.init(p.header->xcd_counter[0], (n_act + kGemmTile - 1) / kGemmTile, col_blocks);
  int rb, cb;
  while (units.next(rb, cb, &unit_s)) {
    const int n0 = rb * kGemmTile, c0 = cb * kGemmTile;
    McLoader A;
    A.init(G, p.n_pad, nullptr, n0, p.n_pad, slab_width, true);
    // (rows of B interleaved: lane j owns the 4 consecutive columns c0 + wn + 4 j + nb)
    KcLoader B;
    B.init(p.head + slab0, p.V, nullptr, c0, p.d, min(slab_width, p.V - slab0), p.head_aligned,
           false, true);
    GemmAcc acc;
    acc.clear();
    gemm_tile(A, B, 0, slab_width, smem, acc);

    const int col = c0 + wn + 4 * j;  // hidden sizes are multiples of 128: col < d implies col + 3 < d
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int slot = n0 + wm + 32 * i + acc_row(r, half);
        if (slot >= n_act || col >= p.d) continue;
        const long row = p.idx[slot];
        f32x4 val = {acc.c[i][0][r], acc.c[i][1][r], acc.c[i][2][r], acc.c[i][3][r]};
        f32x4* a = reinterpret_cast<f32x4*>(dh_acc + (size_t)slot * p.d + col);
        if (mode >= 2) val += *a;
        if (mode == 1 || mode == 2) *a = val;
        if (mode == 0 || mode == 3) {
          bf16x4 out;
#pragma unroll
          for (int nb = 0; nb < 4; ++nb) out[nb] = (bf16)val[nb];
          *reinterpret_cast<bf16x4*>(dhidden + row * p.d + col) = out;
        }
      }
  }
}

__global__ __launch_bounds__(256) void cutce_dhidden_kernel(CutceParams p, const bf16* G,
                                                            int slab0, int slab_width, int mode,
                                                            float* dh_acc, bf16* dhidden) {
  extern __shared__ __align__(16) char smem_raw[];
  dhidden_units(p, G, slab0, slab_width, mode, dh_acc, dhidden, lds_address_of(smem_raw));
}

// dHead[m, slab0 + v] = sum_slot packed[slot, m] G^T[v, slot], packed[slot] = hidden[idx[slot]]:
// the workgroup's share of the units, pulled from counter set 1.
CT_DEVICE void dhead_units(const CutceParams& p, const bf16* packed, const bf16* G, int slab0,
                           int slab_tiles, bf16* dhead, const lds_addr smem) {
  const int tid = threadIdx.x, l = tid & 63, j = l & 31, half = l >> 5, w = tid >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  const int m_blocks = (p.d + kGemmTile - 1) / kGemmTile;
  const int n_act = p.header->n_act;
  // 4 contraction steps at a time; slots n_act .. k_end-1 are valid memory: G^T holds zeros
  // there (the dlogits kernels write whole 256-slot blocks) and the packed rows are finite.
  const int k_end = min(p.n_pad, (n_act + 4 * kBK - 1) / (4 * kBK) * (4 * kBK));
  __shared__ int unit_s;
  // units: (vocabulary tile of the slab, hidden column block)
  XcdUnits units;
  units.init(p.header->xcd_counter[1], slab_tiles, m_blocks);
  int vt, mb;
  while (units.next(vt, mb, &unit_s)) {
    const int m0 = mb * kGemmTile, v0 = vt * kGemmTile;  // v0 relative to the slab
    McLoader A;
    A.init(packed, p.d, nullptr, m0, p.d, k_end, true);
    // (rows of B interleaved: lane j owns the 4 consecutive vocabulary ids v .. v + 3)
    KcLoader B;
    B.init(G, p.n_pad, nullptr, v0, slab_tiles * kGemmTile, k_end, true, false, true);
    GemmAcc acc;
    acc.clear();
    gemm_tile(A, B, 0, k_end, smem, acc);

    const int v = slab0 + v0 + wn + 4 * j;
    const bool vector_store = (p.V % 4 == 0) && ((reinterpret_cast<uintptr_t>(dhead) & 7u) == 0);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + 32 * i + acc_row(r, half);
        if (m >= p.d) continue;
        bf16* dst = dhead + (size_t)m * p.V + v;
        if (vector_store && v + 3 < p.V) {
          bf16x4 out;
#pragma unroll
          for (int nb = 0; nb < 4; ++nb) out[nb] = (bf16)acc.c[i][nb][r];
          *reinterpret_cast<bf16x4*>(dst) = out;
        } else {
#pragma unroll
          for (int nb = 0; nb < 4; ++nb)
            if (v + nb < p.V) dst[nb] = (bf16)acc.c[i][nb][r];
        }
      }
  }
}

__global__ __launch_bounds__(256) void cutce_dhead_kernel(CutceParams p, const bf16* packed,
                                                          const bf16* G, int slab0, int slab_tiles,
                                                          bf16* dhead) {
  extern __shared__ __align__(16) char smem_raw[];
  dhead_units(p, packed, G, slab0, slab_tiles, dhead, lds_address_of(smem_raw));
}

// Both gradients of a slab in one launch. The hidden gradient has few, long units (45 x 16 at
// N = 16384, d = 4096: 2.8 per compute unit, so its last round leaves a sixth of the device idle);
// a workgroup that finds no hidden-gradient unit left goes on to the head-gradient units, which
// are many and short, and the idle tail of the first fills with work of the second. The two
// read the same G^T and write different tensors: neither waits for the other.
__global__ __launch_bounds__(256) void cutce_grads_kernel(CutceParams p, const bf16* packed,
                                                         const bf16* G, int slab0, int slab_width,
                                                         int slab_tiles, int mode, float* dh_acc,
                                                         bf16* dhidden, bf16* dhead) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr smem = lds_address_of(smem_raw);
  dhidden_units(p, G, slab0, slab_width, mode, dh_acc, dhidden, smem);
  dhead_units(p, packed, G, slab0, slab_tiles, dhead, smem);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

static int padded_rows(int N) { return (int)align_up((size_t)N, kGemmTile); }
static int vocab_tile_count(int V) { return (V + kGemmTile - 1) / kGemmTile; }
static int stats_chunks(int V) {
  return (vocab_tile_count(V) + kTilesPerChunk - 1) / kTilesPerChunk;
}

struct FwdLayout {
  size_t header, idx, part, sums, total;
};
static FwdLayout fwd_layout(const ct_cutce_shape& s) {
  const int n_pad = padded_rows(s.rows);
  FwdLayout L;
  L.header = 0;
  L.idx = align_up(sizeof(CutceHeader), 256);
  L.part = L.idx + align_up((size_t)n_pad * sizeof(int), 256);
  L.sums = L.part + align_up((size_t)stats_chunks(s.vocab) * n_pad * 3 * sizeof(float), 256);
  L.total = L.sums + align_up((size_t)(n_pad / kMergeSlots) * 2 * sizeof(double), 256);
  return L;
}

struct BwdLayout {
  size_t header, idx, rowparams, packed, g, acc, total;
  int slab_cols;  // multiple of 256
  int slabs;
};
// header, idx, 3 row parameter arrays, packed hidden rows
static size_t bwd_fixed_bytes(int n_pad, int d) {
  return align_up(sizeof(CutceHeader), 256) + 4 * align_up((size_t)n_pad * sizeof(int), 256) +
         align_up((size_t)n_pad * d * sizeof(bf16), 256);
}
// Largest slab that fits in `bytes` (0 if even one tile column does not).
static BwdLayout bwd_layout(const ct_cutce_shape& s, size_t bytes) {
  const int n_pad = padded_rows(s.rows);
  const int tiles = vocab_tile_count(s.vocab);
  BwdLayout L = {};
  L.header = 0;
  L.idx = align_up(sizeof(CutceHeader), 256);
  L.rowparams = L.idx + align_up((size_t)n_pad * sizeof(int), 256);
  L.packed = L.rowparams + 3 * align_up((size_t)n_pad * sizeof(int), 256);
  L.g = bwd_fixed_bytes(n_pad, s.hidden);
  const size_t per_tile = (size_t)n_pad * kGemmTile * sizeof(bf16);
  const size_t acc_bytes = align_up((size_t)n_pad * s.hidden * sizeof(float), 256);
  if (bytes >= L.g + per_tile * tiles) {
    L.slab_cols = tiles * kGemmTile;
    L.slabs = 1;
    L.acc = 0;
    L.total = L.g + per_tile * tiles;
    return L;
  }
  if (bytes < L.g + acc_bytes + per_tile) return L;  // slab_cols == 0
  const size_t fit = (bytes - L.g - acc_bytes) / per_tile;
  L.slab_cols = (int)fit * kGemmTile;
  L.slabs = (tiles + (int)fit - 1) / (int)fit;
  L.acc = L.g + per_tile * fit;
  L.total = L.acc + acc_bytes;
  return L;
}

static int validate_cutce(const char* fn, const ct_cutce_shape& s) {
  CT_REQUIRE(s.rows > 0, "%s: Cut cross-entropy requires at least one token row", fn);
  CT_REQUIRE(s.hidden > 0 && s.hidden % 128 == 0,
             "%s: Cut cross-entropy hidden size must be divisible by 128, got %d", fn, s.hidden);
  CT_REQUIRE(s.vocab > 0, "%s: Cut cross-entropy requires a non-empty vocabulary", fn);
  return CT_OK;
}

static bool is_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <class K>
static int set_smem(K kernel, size_t bytes, const char* what) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) return fail(CT_LAUNCH_FAILED, "%s: %s", what, hipGetErrorString(e));
  return CT_OK;
}

static int device_cu_count() {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess)
    hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  return cus > 0 ? cus : 256;
}

}  // namespace ct

using namespace ct;

extern "C" size_t ct_cutce_fwd_workspace_bytes(const ct_cutce_shape* shape) {
  if (!shape || shape->rows <= 0 || shape->vocab <= 0) return 0;
  return fwd_layout(*shape).total;
}

extern "C" size_t ct_cutce_logits_cache_bytes(const ct_cutce_shape* shape) {
  if (!shape || shape->rows <= 0 || shape->vocab <= 0) return 0;
  return (size_t)padded_rows(shape->rows) * vocab_tile_count(shape->vocab) * kGemmTile * sizeof(float);
}

extern "C" size_t ct_cutce_bwd_workspace_bytes(const ct_cutce_shape* shape) {
  if (!shape || shape->rows <= 0 || shape->vocab <= 0) return 0;
  const int n_pad = padded_rows(shape->rows);
  return bwd_fixed_bytes(n_pad, shape->hidden) +
         (size_t)n_pad * vocab_tile_count(shape->vocab) * kGemmTile * sizeof(bf16);
}

extern "C" size_t ct_cutce_bwd_workspace_min_bytes(const ct_cutce_shape* shape) {
  if (!shape || shape->rows <= 0 || shape->vocab <= 0) return 0;
  const int n_pad = padded_rows(shape->rows);
  if (vocab_tile_count(shape->vocab) == 1) return ct_cutce_bwd_workspace_bytes(shape);
  return bwd_fixed_bytes(n_pad, shape->hidden) +
         align_up((size_t)n_pad * shape->hidden * sizeof(float), 256) +
         (size_t)n_pad * kGemmTile * sizeof(bf16);
}

static CutceParams make_params(const uint16_t* hidden, const uint16_t* head, const int32_t* targets,
                               const float* weights, const ct_cutce_shape& s, char* ws) {
  CutceParams p;
  p.hidden = reinterpret_cast<const bf16*>(hidden);
  p.head = reinterpret_cast<const bf16*>(head);
  p.targets = targets;
  p.weights = weights;
  p.N = s.rows;
  p.d = s.hidden;
  p.V = s.vocab;
  p.n_pad = padded_rows(s.rows);
  p.header = reinterpret_cast<CutceHeader*>(ws);
  p.idx = reinterpret_cast<int*>(ws + align_up(sizeof(CutceHeader), 256));
  p.hidden_aligned = is_aligned16(hidden);
  p.head_aligned = is_aligned16(head) && (s.vocab % 8 == 0);
  return p;
}

// Shared body of ct_cutce_fwd and ct_cutce_fwd_noalloc: `ws` / `ws_bytes` is the workspace to use
// (the caller's, or this device's static scratch array), `fn` the name for error texts.
static int32_t cutce_fwd_on(void* stream_, const ct_cutce_fwd_args* a, void* ws_, size_t ws_bytes,
                            const char* fn) {
  CT_REQUIRE(a->hidden && a->head && a->targets && a->weights && a->nll_sum && a->weight_sum &&
                 a->lse && ws_,
             "%s: null pointer", fn);
  int rc = validate_cutce(fn, a->shape);
  if (rc) return rc;
  const FwdLayout L = fwd_layout(a->shape);
  if (ws_bytes < L.total)
    return fail(CT_WORKSPACE_TOO_SMALL, "%s: workspace %zu < %zu bytes", fn, ws_bytes, L.total);
  CT_REQUIRE(is_aligned16(ws_), "%s: workspace must be 16-byte aligned", fn);
  if (a->logits_cache) {
    CT_REQUIRE(is_aligned16(a->logits_cache), "%s: logits cache must be 16-byte aligned", fn);
    if (a->logits_cache_bytes < ct_cutce_logits_cache_bytes(&a->shape))
      return fail(CT_WORKSPACE_TOO_SMALL, "%s: logits cache %zu < %zu bytes", fn,
                  a->logits_cache_bytes, ct_cutce_logits_cache_bytes(&a->shape));
  }
  hipStream_t stream = (hipStream_t)stream_;
  char* ws = static_cast<char*>(ws_);
  CutceParams p = make_params(a->hidden, a->head, a->targets, a->weights, a->shape, ws);
  float* part = reinterpret_cast<float*>(ws + L.part);
  double* sums = reinterpret_cast<double*>(ws + L.sums);
  const int chunks = stats_chunks(p.V);
  const int row_blocks = p.n_pad / kGemmTile;

  LaunchScope scope1("cutce_index_kernel", stream);
  hipLaunchKernelGGL(cutce_index_kernel, dim3(1), dim3(1024), 0, stream, p.weights, p.N, p.n_pad,
                     a->sparse_compaction ? 1 : 0, p.idx, p.header);
  if ((rc = scope1.done())) return rc;

  const size_t smem = GemmSmem::kBytes;
  if ((rc = set_smem(cutce_stats_kernel<false>, smem, fn))) return rc;
  if ((rc = set_smem(cutce_stats_kernel<true>, smem, fn))) return rc;
  const int persistent = min(device_cu_count(), chunks * row_blocks);
  LaunchScope scope2("cutce_stats_kernel", stream);
  if (a->logits_cache)
    hipLaunchKernelGGL(cutce_stats_kernel<true>, dim3(persistent), dim3(256), smem, stream, p, part,
                       chunks, static_cast<float*>(a->logits_cache));
  else
    hipLaunchKernelGGL(cutce_stats_kernel<false>, dim3(persistent), dim3(256), smem, stream, p, part,
                       chunks, static_cast<float*>(nullptr));
  if ((rc = scope2.done())) return rc;

  const int merge_blocks = p.n_pad / kMergeSlots;
  LaunchScope scope3("cutce_merge_kernel", stream);
  hipLaunchKernelGGL(cutce_merge_kernel, dim3(merge_blocks), dim3(kMergeSlots * kMergeParts), 0, stream, p, part,
                     chunks, a->lse, sums);
  if ((rc = scope3.done())) return rc;
  LaunchScope scope4("cutce_finalize_kernel", stream);
  hipLaunchKernelGGL(cutce_finalize_kernel, dim3(1), dim3(64), 0, stream, sums, merge_blocks,
                     a->nll_sum, a->weight_sum);
  return scope4.done();
}

extern "C" int32_t ct_cutce_fwd(void* stream, const ct_cutce_fwd_args* a) {
  CT_REQUIRE(a, "ct_cutce_fwd: null args");
  return cutce_fwd_on(stream, a, a->workspace, a->workspace_bytes, "ct_cutce_fwd");
}

// ---------------------------------------------------------------------------
// The forward for callers that cannot allocate: its workspace (header, active-row
// index list, per-chunk row statistics, per-block loss sums) lives in a static
// device array instead of a caller buffer. Every GPU that loads the library holds
// its own copy of the array at its own address, so the address is looked up once
// per device, with that device current, and kept.
// ---------------------------------------------------------------------------
namespace ct {
constexpr size_t kNoAllocScratchBytes = (size_t)32 << 20;
constexpr int kNoAllocMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
static void* g_scratch_ptr[kNoAllocMaxDevices];  // device address of `scratch`, per device
static std::mutex g_scratch_mutex;
}  // namespace ct

extern "C" size_t ct_cutce_fwd_noalloc_max_bytes(void) { return kNoAllocScratchBytes; }

extern "C" int32_t ct_cutce_fwd_noalloc(void* stream, const ct_cutce_fwd_args* a) {
  CT_REQUIRE(a, "ct_cutce_fwd_noalloc: null args");
  int rc = validate_cutce("ct_cutce_fwd_noalloc", a->shape);
  if (rc) return rc;
  const size_t need = fwd_layout(a->shape).total;
  if (need > kNoAllocScratchBytes)
    return fail(CT_UNSUPPORTED,
                "ct_cutce_fwd_noalloc: rows=%d, vocab=%d need %zu bytes of scratch, the static "
                "array holds %zu; use ct_cutce_fwd with a caller workspace",
                a->shape.rows, a->shape.vocab, need, kNoAllocScratchBytes);
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess)
    return fail(CT_LAUNCH_FAILED, "ct_cutce_fwd_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  CT_REQUIRE(device >= 0 && device < kNoAllocMaxDevices, "ct_cutce_fwd_noalloc: device %d out of range",
             device);
  void* ws = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
      void* ptr = nullptr;
      e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
      if (e != hipSuccess || !ptr)
        return fail(CT_LAUNCH_FAILED, "ct_cutce_fwd_noalloc: hipGetSymbolAddress: %s",
                    hipGetErrorString(e));
      g_scratch_ptr[device] = ptr;
    }
    ws = g_scratch_ptr[device];
  }
  return cutce_fwd_on(stream, a, ws, kNoAllocScratchBytes, "ct_cutce_fwd_noalloc");
}

extern "C" int32_t ct_cutce_bwd(void* stream_, const ct_cutce_bwd_args* a) {
  CT_REQUIRE(a, "ct_cutce_bwd: null args");
  CT_REQUIRE(a->hidden && a->head && a->targets && a->weights && a->lse && a->dy && a->dhidden &&
                 a->workspace,
             "ct_cutce_bwd: null pointer");
  int rc = validate_cutce("ct_cutce_bwd", a->shape);
  if (rc) return rc;
  CT_REQUIRE(is_aligned16(a->workspace) && is_aligned16(a->dhidden),
             "ct_cutce_bwd: workspace and dhidden must be 16-byte aligned");
  const BwdLayout L = bwd_layout(a->shape, a->workspace_bytes);
  if (L.slab_cols == 0)
    return fail(CT_WORKSPACE_TOO_SMALL, "ct_cutce_bwd: workspace %zu < %zu bytes",
                a->workspace_bytes, ct_cutce_bwd_workspace_min_bytes(&a->shape));
  hipStream_t stream = (hipStream_t)stream_;
  char* ws = static_cast<char*>(a->workspace);
  CutceParams p = make_params(a->hidden, a->head, a->targets, a->weights, a->shape, ws);
  bf16* G = reinterpret_cast<bf16*>(ws + L.g);
  float* dh_acc = L.slabs > 1 ? reinterpret_cast<float*>(ws + L.acc) : nullptr;
  bf16* dhidden = reinterpret_cast<bf16*>(a->dhidden);
  bf16* dhead = reinterpret_cast<bf16*>(a->dhead);
  const float* cache = static_cast<const float*>(a->logits_cache);
  if (cache) {
    CT_REQUIRE(is_aligned16(cache), "ct_cutce_bwd: logits cache must be 16-byte aligned");
    if (a->logits_cache_bytes < ct_cutce_logits_cache_bytes(&a->shape))
      return fail(CT_WORKSPACE_TOO_SMALL, "ct_cutce_bwd: logits cache %zu < %zu bytes",
                  a->logits_cache_bytes, ct_cutce_logits_cache_bytes(&a->shape));
  }
  const int row_blocks = p.n_pad / kGemmTile;
  const size_t params_stride = align_up((size_t)p.n_pad * sizeof(int), 256);
  CutceRowParams rp;
  rp.fac = reinterpret_cast<float*>(ws + L.rowparams);
  rp.lse2 = reinterpret_cast<float*>(ws + L.rowparams + params_stride);
  rp.tgt = reinterpret_cast<int*>(ws + L.rowparams + 2 * params_stride);
  const size_t smem = GemmSmem::kBytes;
  if ((rc = set_smem(cutce_dlogits_kernel, smem, "ct_cutce_bwd"))) return rc;
  if ((rc = set_smem(cutce_dhidden_kernel, smem, "ct_cutce_bwd"))) return rc;
  if ((rc = set_smem(cutce_dhead_kernel, smem, "ct_cutce_bwd"))) return rc;
  if ((rc = set_smem(cutce_grads_kernel, smem, "ct_cutce_bwd"))) return rc;

  LaunchScope scope5("cutce_index_kernel", stream);
  hipLaunchKernelGGL(cutce_index_kernel, dim3(1), dim3(1024), 0, stream, p.weights, p.N, p.n_pad,
                     a->sparse_compaction ? 1 : 0, p.idx, p.header);
  if ((rc = scope5.done())) return rc;
  LaunchScope scope6("cutce_zero_rows_kernel", stream);
  hipLaunchKernelGGL(cutce_zero_rows_kernel, dim3(p.N), dim3(256), 0, stream, p.weights, p.N, p.d,
                     dhidden);
  if ((rc = scope6.done())) return rc;
  LaunchScope scope10("cutce_rowparams_kernel", stream);
  hipLaunchKernelGGL(cutce_rowparams_kernel, dim3(row_blocks), dim3(256), 0, stream, p, a->lse, a->dy,
                     rp);
  if ((rc = scope10.done())) return rc;

  const int cus = device_cu_count();
  bf16* packed = reinterpret_cast<bf16*>(ws + L.packed);
  if (dhead) {
    LaunchScope scope12("cutce_pack_rows_kernel", stream);
    hipLaunchKernelGGL(cutce_pack_rows_kernel, dim3(p.n_pad), dim3(256), 0, stream, p, packed);
    if ((rc = scope12.done())) return rc;
  }

  const int tiles = vocab_tile_count(p.V);
  const int tiles_per_slab = L.slab_cols / kGemmTile;
  for (int s = 0; s < L.slabs; ++s) {
    const int slab0 = s * L.slab_cols;
    const int slab_tiles = min(tiles_per_slab, tiles - s * tiles_per_slab);
    const int slab_width = slab_tiles * kGemmTile;
    if (cache) {
      LaunchScope scope11("cutce_dlogits_cached_kernel", stream);
      hipLaunchKernelGGL(cutce_dlogits_cached_kernel, dim3(slab_width / kDlogitsRows, (p.n_pad + 2047) / 2048),
                         dim3(256), 0, stream, p, rp, cache, slab0, G);
      if ((rc = scope11.done())) return rc;
    } else {
      LaunchScope scope7("cutce_dlogits_kernel", stream);
      const int dl_units = ((slab_tiles + kTilesPerChunk - 1) / kTilesPerChunk) * row_blocks;
      hipLaunchKernelGGL(cutce_dlogits_kernel, dim3(min(cus, dl_units)), dim3(256), smem, stream,
                         p, rp, slab0, slab_tiles, G);
      if ((rc = scope7.done())) return rc;
    }
    const int mode = L.slabs == 1 ? 0 : (s == 0 ? 1 : (s == L.slabs - 1 ? 3 : 2));
    const int col_blocks = (p.d + kGemmTile - 1) / kGemmTile;
    if (dhead) {
      // both gradients in one launch: the head-gradient units fill the hidden gradient's tail
      LaunchScope scope8("cutce_grads_kernel", stream);
      const int units = max(row_blocks * col_blocks, col_blocks * slab_tiles);
      hipLaunchKernelGGL(cutce_grads_kernel, dim3(min(cus, units)), dim3(256), smem, stream, p, packed, G,
                         slab0, slab_width, slab_tiles, mode, dh_acc, dhidden, dhead);
      if ((rc = scope8.done())) return rc;
    } else {
      LaunchScope scope8("cutce_dhidden_kernel", stream);
      hipLaunchKernelGGL(cutce_dhidden_kernel, dim3(min(cus, row_blocks * col_blocks)), dim3(256), smem,
                         stream, p, G, slab0, slab_width, mode, dh_acc, dhidden);
      if ((rc = scope8.done())) return rc;
    }
  }
  return CT_OK;
}
