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
//            to a workspace slab [rows, vocab slab]
//   dhidden  dHidden = G head^T            (k-contiguous x k-contiguous GEMM)
//   dhead    dHead   = hidden^T G          (both operands read transposed)
// The reference recomputes the logits in both backward kernels
// (src/kernels/cut_cross_entropy.py:258, :383); here they are recomputed once
// and the bf16 G slab is shared, which keeps the reference's rounding points
// (G is cast to bf16 before both products, :272, :396) and needs 4 GEMMs
// instead of 5.
#include "ct_error.h"
#include "ct_gemm.cuh"

namespace ct {

constexpr int kBK = kGemmBK;
constexpr int kTilesPerChunk = 4;  // vocab tiles per stats work unit
constexpr float kNegInfF = -__builtin_inff();

struct CutceHeader {
  int n_act;
  int counter;
  int pad[14];
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

__global__ __launch_bounds__(256) void cutce_stats_kernel(CutceParams p, float* part, int chunks) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr smem = lds_address_of(smem_raw);
  __shared__ int unit_s;
  const int tid = threadIdx.x, l = tid & 63, j = l & 31, half = l >> 5, w = tid >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  const int row_blocks = p.n_pad / kGemmTile;
  const int vocab_tiles = (p.V + kGemmTile - 1) / kGemmTile;
  const int total = chunks * row_blocks;
  const int n_act = p.header->n_act;

  for (;;) {
    if (tid == 0) unit_s = atomicAdd(&p.header->counter, 1);
    __syncthreads();
    const int unit = unit_s;
    if (unit >= total) break;
    const int chunk = unit / row_blocks, rb = unit % row_blocks;
    const int n0 = rb * kGemmTile;
    const int my_slot = n0 + tid;
    const int active = my_slot < n_act && p.weights[p.idx[my_slot]] != 0.f;
    if (!__syncthreads_or(active)) continue;  // no row of this block carries weight

    int tgt[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      const int slot = n0 + wn + 32 * nb + j;
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
    B.init(p.hidden, p.d, p.idx, n0, n_act, p.d, p.hidden_aligned, true);

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
        float* out = part + ((size_t)chunk * p.n_pad + n0 + wn + 32 * nb + j) * 3;
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
__global__ __launch_bounds__(256) void cutce_merge_kernel(CutceParams p, const float* part,
                                                          int chunks, float* lse_out,
                                                          double* block_sums) {
  __shared__ double red[2][4];
  const int tid = threadIdx.x;
  const int slot = blockIdx.x * 256 + tid;
  const int n_act = p.header->n_act;
  double loss = 0.0, wsum = 0.0;
  if (slot < p.N) {
    const float wi = p.weights[slot];
    wsum = (double)wi;
    if (wi == 0.f) lse_out[slot] = 0.f;
  }
  if (slot < n_act) {
    const int row = p.idx[slot];
    const float wr = p.weights[row];
    if (wr != 0.f) {
      float m = kNegInfF, s = 0.f, t = 0.f;
      for (int c = 0; c < chunks; ++c) {
        const float* e = part + ((size_t)c * p.n_pad + slot) * 3;
        merge_stats(m, s, e[0], e[1]);
        t += e[2];
      }
      const float lse = (__log2f(s) + m) * kLn2;
      lse_out[row] = lse;
      loss = (double)wr * ((double)lse - (double)t);
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    loss += __shfl_xor(loss, off, 64);
    wsum += __shfl_xor(wsum, off, 64);
  }
  if ((tid & 63) == 0) {
    red[0][tid >> 6] = loss;
    red[1][tid >> 6] = wsum;
  }
  __syncthreads();
  if (tid == 0) {
    block_sums[2 * blockIdx.x + 0] = red[0][0] + red[0][1] + red[0][2] + red[0][3];
    block_sums[2 * blockIdx.x + 1] = red[1][0] + red[1][1] + red[1][2] + red[1][3];
  }
}

__global__ __launch_bounds__(64) void cutce_finalize_kernel(const double* block_sums, int blocks,
                                                            float* nll_sum, float* weight_sum) {
  if (threadIdx.x != 0) return;
  double loss = 0.0, wsum = 0.0;
  for (int b = 0; b < blocks; ++b) {
    loss += block_sums[2 * b];
    wsum += block_sums[2 * b + 1];
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

// G[slot, v - slab0] for one 256 x 256 tile.
__global__ __launch_bounds__(256) void cutce_dlogits_kernel(CutceParams p, const float* lse,
                                                            const float* dy, int slab0,
                                                            int slab_tiles, bf16* G, int ldg) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr smem = lds_address_of(smem_raw);
  __shared__ float lse2_s[kGemmTile];
  __shared__ float fac_s[kGemmTile];
  __shared__ int tgt_s[kGemmTile];
  const int tid = threadIdx.x, l = tid & 63, j = l & 31, half = l >> 5, w = tid >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  const int row_blocks = p.n_pad / kGemmTile;
  int id = xcd_remap(blockIdx.x, slab_tiles * row_blocks);
  const int rb = id % row_blocks, vt = id / row_blocks;
  const int n0 = rb * kGemmTile;
  const int n_act = p.header->n_act;
  if (n0 >= n_act) return;  // G rows past the active count are never read
  const int v0 = slab0 + vt * kGemmTile;

  {
    const int slot = n0 + tid;
    float f = 0.f, l2 = 0.f;
    int t = -1;
    if (slot < n_act) {
      const int row = p.idx[slot];
      const float wr = p.weights[row];
      if (wr != 0.f) {
        f = wr * dy[0];
        l2 = lse[row] * kLog2e;
        t = p.targets[row];
      }
    }
    fac_s[tid] = f;
    lse2_s[tid] = l2;
    tgt_s[tid] = t;
  }
  KcLoader A;
  A.init(p.hidden, p.d, p.idx, n0, n_act, p.d, p.hidden_aligned, true);
  McLoader B;
  B.init(p.head, p.V, nullptr, v0, p.V, p.d, p.head_aligned);
  GemmAcc acc;
  acc.clear();
  gemm_tile(A, B, 0, p.d, smem, acc);  // barriers inside also publish the row arrays

#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const int r0 = wm + 32 * i + 8 * qd + 4 * half;
      const f32x4 l4 = *reinterpret_cast<const f32x4*>(lse2_s + r0);
      const f32x4 f4 = *reinterpret_cast<const f32x4*>(fac_s + r0);
      const int4 t4 = *reinterpret_cast<const int4*>(tgt_s + r0);
      const int tg[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        bf16* grow = G + (size_t)(n0 + r0 + e) * ldg + (v0 - slab0);
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
          const int col = wn + 32 * nb + j;
          const int v = v0 + col;
          float g = 0.f;
          if (f4[e] != 0.f && v < p.V) {
            const float prob = exp2_fast(acc.c[i][nb][4 * qd + e] * kLog2e - l4[e]);
            g = f4[e] * (prob - (v == tg[e] ? 1.f : 0.f));
          }
          grow[col] = (bf16)g;
        }
      }
    }
  }
}

// dHidden[idx[slot], n] (+)= sum_v G[slot, v] head[n, slab0 + v]
__global__ __launch_bounds__(256) void cutce_dhidden_kernel(CutceParams p, const bf16* G, int ldg,
                                                            int slab0, int slab_width, int mode,
                                                            float* dh_acc, bf16* dhidden) {
  // mode: 0 = single slab (store bf16), 1 = first slab (store f32), 2 = middle
  // slab (add f32), 3 = last slab (add, store bf16)
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr smem = lds_address_of(smem_raw);
  const int tid = threadIdx.x, l = tid & 63, j = l & 31, half = l >> 5, w = tid >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  const int row_blocks = p.n_pad / kGemmTile, col_blocks = (p.d + kGemmTile - 1) / kGemmTile;
  int id = xcd_remap(blockIdx.x, row_blocks * col_blocks);
  const int cb = id % col_blocks, rb = id / col_blocks;
  const int n0 = rb * kGemmTile, c0 = cb * kGemmTile;
  const int n_act = p.header->n_act;
  if (n0 >= n_act) return;

  KcLoader A;
  A.init(G, ldg, nullptr, n0, p.n_pad, slab_width, true, false);
  KcLoader B;
  B.init(p.head + slab0, p.V, nullptr, c0, p.d, min(slab_width, p.V - slab0), p.head_aligned, false);
  GemmAcc acc;
  acc.clear();
  gemm_tile(A, B, 0, slab_width, smem, acc);

#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int slot = n0 + wm + 32 * i + acc_row(r, half);
      if (slot >= n_act) continue;
      const long row = p.idx[slot];
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        const int col = c0 + wn + 32 * nb + j;
        if (col >= p.d) continue;
        float val = acc.c[i][nb][r];
        float* a = dh_acc + (size_t)slot * p.d + col;
        if (mode >= 2) val += *a;
        if (mode == 1 || mode == 2) *a = val;
        if (mode == 0 || mode == 3) dhidden[row * p.d + col] = (bf16)val;
      }
    }
}

// dHead[m, slab0 + v] = sum_slot hidden[idx[slot], m] G[slot, v]
__global__ __launch_bounds__(256) void cutce_dhead_kernel(CutceParams p, const bf16* G, int ldg,
                                                          int slab0, int slab_tiles, bf16* dhead) {
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr smem = lds_address_of(smem_raw);
  const int tid = threadIdx.x, l = tid & 63, j = l & 31, half = l >> 5, w = tid >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  const int m_blocks = (p.d + kGemmTile - 1) / kGemmTile;
  int id = xcd_remap(blockIdx.x, m_blocks * slab_tiles);
  const int mb = id % m_blocks, vt = id / m_blocks;
  const int m0 = mb * kGemmTile, v0 = vt * kGemmTile;  // v0 relative to the slab
  const int n_act = p.header->n_act;
  const int k_end = min(p.n_pad, (n_act + kBK - 1) / kBK * kBK);

  McLoader A;
  // Rows n_act .. k_end-1 are valid memory: G holds zeros there (written by the
  // dlogits kernel for the whole 256-row block) and idx repeats the first active row.
  A.init(p.hidden, p.d, p.idx, m0, p.d, k_end, p.hidden_aligned);
  McLoader B;
  B.init(G, ldg, nullptr, v0, ldg, k_end, true);
  GemmAcc acc;
  acc.clear();
  gemm_tile(A, B, 0, k_end, smem, acc);

#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + wm + 32 * i + acc_row(r, half);
      if (m >= p.d) continue;
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        const int v = slab0 + v0 + wn + 32 * nb + j;
        if (v < p.V) dhead[(size_t)m * p.V + v] = (bf16)acc.c[i][nb][r];
      }
    }
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
  L.total = L.sums + align_up((size_t)(n_pad / kGemmTile) * 2 * sizeof(double), 256);
  return L;
}

struct BwdLayout {
  size_t header, idx, g, acc, total;
  int slab_cols;  // multiple of 256
  int slabs;
};
static size_t bwd_fixed_bytes(int n_pad) {
  return align_up(sizeof(CutceHeader), 256) + align_up((size_t)n_pad * sizeof(int), 256);
}
// Largest slab that fits in `bytes` (0 if even one tile column does not).
static BwdLayout bwd_layout(const ct_cutce_shape& s, size_t bytes) {
  const int n_pad = padded_rows(s.rows);
  const int tiles = vocab_tile_count(s.vocab);
  BwdLayout L = {};
  L.header = 0;
  L.idx = align_up(sizeof(CutceHeader), 256);
  L.g = bwd_fixed_bytes(n_pad);
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

extern "C" size_t ct_cutce_bwd_workspace_bytes(const ct_cutce_shape* shape) {
  if (!shape || shape->rows <= 0 || shape->vocab <= 0) return 0;
  const int n_pad = padded_rows(shape->rows);
  return bwd_fixed_bytes(n_pad) +
         (size_t)n_pad * vocab_tile_count(shape->vocab) * kGemmTile * sizeof(bf16);
}

extern "C" size_t ct_cutce_bwd_workspace_min_bytes(const ct_cutce_shape* shape) {
  if (!shape || shape->rows <= 0 || shape->vocab <= 0) return 0;
  const int n_pad = padded_rows(shape->rows);
  if (vocab_tile_count(shape->vocab) == 1) return ct_cutce_bwd_workspace_bytes(shape);
  return bwd_fixed_bytes(n_pad) + align_up((size_t)n_pad * shape->hidden * sizeof(float), 256) +
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

extern "C" int32_t ct_cutce_fwd(void* stream_, const ct_cutce_fwd_args* a) {
  CT_REQUIRE(a, "ct_cutce_fwd: null args");
  CT_REQUIRE(a->hidden && a->head && a->targets && a->weights && a->nll_sum && a->weight_sum &&
                 a->lse && a->workspace,
             "ct_cutce_fwd: null pointer");
  int rc = validate_cutce("ct_cutce_fwd", a->shape);
  if (rc) return rc;
  const FwdLayout L = fwd_layout(a->shape);
  if (a->workspace_bytes < L.total)
    return fail(CT_WORKSPACE_TOO_SMALL, "ct_cutce_fwd: workspace %zu < %zu bytes",
                a->workspace_bytes, L.total);
  CT_REQUIRE(is_aligned16(a->workspace), "ct_cutce_fwd: workspace must be 16-byte aligned");
  hipStream_t stream = (hipStream_t)stream_;
  char* ws = static_cast<char*>(a->workspace);
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
  if ((rc = set_smem(cutce_stats_kernel, smem, "ct_cutce_fwd"))) return rc;
  const int persistent = min(device_cu_count(), chunks * row_blocks);
  LaunchScope scope2("cutce_stats_kernel", stream);
  hipLaunchKernelGGL(cutce_stats_kernel, dim3(persistent), dim3(256), smem, stream, p, part, chunks);
  if ((rc = scope2.done())) return rc;

  LaunchScope scope3("cutce_merge_kernel", stream);
  hipLaunchKernelGGL(cutce_merge_kernel, dim3(row_blocks), dim3(256), 0, stream, p, part, chunks,
                     a->lse, sums);
  if ((rc = scope3.done())) return rc;
  LaunchScope scope4("cutce_finalize_kernel", stream);
  hipLaunchKernelGGL(cutce_finalize_kernel, dim3(1), dim3(64), 0, stream, sums, row_blocks,
                     a->nll_sum, a->weight_sum);
  return scope4.done();
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
  const int row_blocks = p.n_pad / kGemmTile;
  const int ldg = L.slab_cols;
  const size_t smem = GemmSmem::kBytes;
  if ((rc = set_smem(cutce_dlogits_kernel, smem, "ct_cutce_bwd"))) return rc;
  if ((rc = set_smem(cutce_dhidden_kernel, smem, "ct_cutce_bwd"))) return rc;
  if ((rc = set_smem(cutce_dhead_kernel, smem, "ct_cutce_bwd"))) return rc;

  LaunchScope scope5("cutce_index_kernel", stream);
  hipLaunchKernelGGL(cutce_index_kernel, dim3(1), dim3(1024), 0, stream, p.weights, p.N, p.n_pad,
                     a->sparse_compaction ? 1 : 0, p.idx, p.header);
  if ((rc = scope5.done())) return rc;
  LaunchScope scope6("cutce_zero_rows_kernel", stream);
  hipLaunchKernelGGL(cutce_zero_rows_kernel, dim3(p.N), dim3(256), 0, stream, p.weights, p.N, p.d,
                     dhidden);
  if ((rc = scope6.done())) return rc;

  const int tiles = vocab_tile_count(p.V);
  const int tiles_per_slab = L.slab_cols / kGemmTile;
  for (int s = 0; s < L.slabs; ++s) {
    const int slab0 = s * L.slab_cols;
    const int slab_tiles = min(tiles_per_slab, tiles - s * tiles_per_slab);
    const int slab_width = slab_tiles * kGemmTile;
    LaunchScope scope7("cutce_dlogits_kernel", stream);
    hipLaunchKernelGGL(cutce_dlogits_kernel, dim3(slab_tiles * row_blocks), dim3(256), smem, stream,
                       p, a->lse, a->dy, slab0, slab_tiles, G, ldg);
    if ((rc = scope7.done())) return rc;
    const int mode = L.slabs == 1 ? 0 : (s == 0 ? 1 : (s == L.slabs - 1 ? 3 : 2));
    LaunchScope scope8("cutce_dhidden_kernel", stream);
    hipLaunchKernelGGL(cutce_dhidden_kernel, dim3(row_blocks * ((p.d + kGemmTile - 1) / kGemmTile)), dim3(256), smem,
                       stream, p, G, ldg, slab0, slab_width, mode, dh_acc, dhidden);
    if ((rc = scope8.done())) return rc;
    if (dhead) {
      LaunchScope scope9("cutce_dhead_kernel", stream);
      hipLaunchKernelGGL(cutce_dhead_kernel, dim3(((p.d + kGemmTile - 1) / kGemmTile) * slab_tiles), dim3(256), smem,
                         stream, p, G, ldg, slab0, slab_tiles, dhead);
      if ((rc = scope9.done())) return rc;
    }
  }
  return CT_OK;
}
