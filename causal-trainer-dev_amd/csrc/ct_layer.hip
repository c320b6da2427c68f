// The decoder-layer neighbours of the attention operator: reset position ids, the per-token
// rotary tables, partial rotary embedding of Q and K (both channel pairings, optionally fused
// with the bf16 pre-scale of Q that the attention operator otherwise does), and RMS
// normalisation forward and backward. All are single passes over HBM.
//
// Reference: src/modeling/rotary.py:82-110 (positions), :132-157 (tables), :113-129 and :160-204 (apply),
// src/modeling/architecture.py:155-162 (rms_norm).
#include "ct_error.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ct {

typedef __bf16 bf16;
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }
__device__ __forceinline__ u32x4 as_u32x4(bf16x8 v) { return __builtin_bit_cast(u32x4, v); }
__device__ __forceinline__ bf16x4 as_bf16x4(u32x2 v) { return __builtin_bit_cast(bf16x4, v); }

// One workgroup per batch row. A run starts at a valid position whose canonical id differs
// from its predecessor's or whose predecessor's id is 0 (position 0: predecessor id 0);
// position = index - index of the latest run start (running maximum), 0 where invalid.
__global__ __launch_bounds__(1024) void position_ids_kernel(const int* mask, const int* ids, int S,
                                                            int* out) {
  __shared__ int wave_max[16];
  __shared__ int carry_s;
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nwaves = blockDim.x >> 6;
  const int* mrow = mask + (size_t)b * S;
  const int* irow = ids + (size_t)b * S;
  int* orow = out + (size_t)b * S;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (int base = 0; base < S; base += blockDim.x) {
    const int s = base + tid;
    bool valid = false;
    int start_index = 0;
    if (s < S) {
      valid = mrow[s] != 0;
      const int prev = s > 0 ? irow[s - 1] : 0;
      if (valid && (irow[s] != prev || prev == 0)) start_index = s;
    }
    int incl = start_index;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int other = __shfl_up(incl, off, 64);
      if (lane >= off) incl = max(incl, other);
    }
    if (lane == 63) wave_max[wave] = incl;
    __syncthreads();
    int latest = carry_s;
    for (int k = 0; k < wave; ++k) latest = max(latest, wave_max[k]);
    latest = max(latest, incl);
    if (s < S) orow[s] = valid ? s - latest : 0;
    __syncthreads();
    if (tid == 0) {
      int total = carry_s;
      for (int k = 0; k < nwaves; ++k) total = max(total, wave_max[k]);
      carry_s = total;
    }
    __syncthreads();
  }
}

// cos / sin of f32(position) * inv_freq[p] evaluated in f32, rounded once to bf16.
__global__ __launch_bounds__(256) void rotary_tables_kernel(const int* positions,
                                                            const float* inv_freq, long tokens,
                                                            int pairs, bf16* cosine, bf16* sine) {
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= tokens * pairs) return;
  const long t = gid / pairs;
  const int p = (int)(gid % pairs);
  const float angle = (float)positions[t] * inv_freq[p];
  cosine[gid] = (bf16)cosf(angle);
  sine[gid] = (bf16)sinf(angle);
}

__device__ __forceinline__ bf16 scaled(bf16 v, float s, bool on) {
  return on ? (bf16)((float)v * s) : v;
}

// One thread per 16-byte chunk (8 channels) of a (token, head) row; Q heads first, then K
// heads. ADJACENT: pairs (2i, 2i+1), a chunk holds 4 pairs. Otherwise pairs (i, i + R/2): the
// threads of the first half of the rotated channels also handle the partner chunk, those of
// the second half do nothing. Channels past the rotated ones are copied (and scaled).
// forward: out = bf16(bf16(R x) * s); inverse: out = bf16(R^T bf16(x * s)). The rotation is
// evaluated in f32 from the bf16 operands and rounded once.
template <bool ADJACENT>
__device__ __forceinline__ void apply_rotary_chunk(const ct_rotary_args& a, long t, int h, int c);

// One workgroup per token walks the (head, chunk) pairs of that token: no 64-bit index
// arithmetic per chunk, and the token's cos / sin row is shared by the whole workgroup.
template <bool ADJACENT>
__global__ __launch_bounds__(256) void apply_rotary_kernel(ct_rotary_args a) {
  const int cpr = a.head_dim / 8;  // chunks per head row
  const int heads = a.q_heads + a.kv_heads;
  const long t = blockIdx.x;
  for (unsigned item = threadIdx.x; item < (unsigned)(heads * cpr); item += 256)
    apply_rotary_chunk<ADJACENT>(a, t, (int)(item / (unsigned)cpr), (int)(item % (unsigned)cpr));
}

template <bool ADJACENT>
__device__ __forceinline__ void apply_rotary_chunk(const ct_rotary_args& a, long t, int h, int c) {
  const bool is_q = h < a.q_heads;
  const uint16_t* in = is_q ? a.q_in : a.k_in;
  uint16_t* out = is_q ? a.q_out : a.k_out;
  const size_t row = is_q ? ((size_t)t * a.q_heads + h) : ((size_t)t * a.kv_heads + (h - a.q_heads));
  const size_t base = row * a.head_dim;
  const bool scale_on = is_q && a.q_scale != 1.0f;
  const float s = (float)(bf16)a.q_scale;  // the scale is rounded to bf16 first
  const int rot_chunks = a.rotary_pairs / 4;  // rotary_dim / 8
  const float sign = a.inverse ? -1.f : 1.f;

  if (c >= rot_chunks) {
    bf16x8 v = as_bf16x8(*reinterpret_cast<const u32x4*>(in + base + c * 8));
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = scaled(v[e], s, scale_on);
    *reinterpret_cast<u32x4*>(out + base + c * 8) = as_u32x4(v);
    return;
  }
  const bf16* cs = reinterpret_cast<const bf16*>(a.cosine) + (size_t)t * a.rotary_pairs;
  const bf16* sn = reinterpret_cast<const bf16*>(a.sine) + (size_t)t * a.rotary_pairs;
  if constexpr (ADJACENT) {
    bf16x8 v = as_bf16x8(*reinterpret_cast<const u32x4*>(in + base + c * 8));
    const bf16x4 cv = as_bf16x4(*reinterpret_cast<const u32x2*>(cs + c * 4));
    const bf16x4 sv = as_bf16x4(*reinterpret_cast<const u32x2*>(sn + c * 4));
    bf16x8 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      bf16 even = v[2 * i], odd = v[2 * i + 1];
      if (a.inverse) {
        even = scaled(even, s, scale_on);
        odd = scaled(odd, s, scale_on);
      }
      const float co = (float)cv[i], si = sign * (float)sv[i];
      bf16 oe = (bf16)((float)even * co - (float)odd * si);
      bf16 oo = (bf16)((float)odd * co + (float)even * si);
      if (!a.inverse) {
        oe = scaled(oe, s, scale_on);
        oo = scaled(oo, s, scale_on);
      }
      o[2 * i] = oe;
      o[2 * i + 1] = oo;
    }
    *reinterpret_cast<u32x4*>(out + base + c * 8) = as_u32x4(o);
  } else {
    const int half_chunks = rot_chunks / 2;
    if (c >= half_chunks) return;  // written by the thread of the partner chunk
    bf16x8 first = as_bf16x8(*reinterpret_cast<const u32x4*>(in + base + c * 8));
    bf16x8 second = as_bf16x8(*reinterpret_cast<const u32x4*>(in + base + (c + half_chunks) * 8));
    const bf16x8 cv = as_bf16x8(*reinterpret_cast<const u32x4*>(cs + c * 8));
    const bf16x8 sv = as_bf16x8(*reinterpret_cast<const u32x4*>(sn + c * 8));
    bf16x8 o1, o2;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      bf16 x1 = first[i], x2 = second[i];
      if (a.inverse) {
        x1 = scaled(x1, s, scale_on);
        x2 = scaled(x2, s, scale_on);
      }
      const float co = (float)cv[i], si = sign * (float)sv[i];
      bf16 r1 = (bf16)((float)x1 * co - (float)x2 * si);
      bf16 r2 = (bf16)((float)x2 * co + (float)x1 * si);
      if (!a.inverse) {
        r1 = scaled(r1, s, scale_on);
        r2 = scaled(r2, s, scale_on);
      }
      o1[i] = r1;
      o2[i] = r2;
    }
    *reinterpret_cast<u32x4*>(out + base + c * 8) = as_u32x4(o1);
    *reinterpret_cast<u32x4*>(out + base + (c + half_chunks) * 8) = as_u32x4(o2);
  }
}

// Any head_dim and any even rotary dimension, one thread per (token, head) row and one channel
// pair at a time: the shapes the 16-byte kernel above does not take (e.g. 4 rotated channels of 8).
// Same arithmetic, element for element.
template <bool ADJACENT>
__global__ __launch_bounds__(256) void apply_rotary_rows_kernel(ct_rotary_args a) {
  const int heads = a.q_heads + a.kv_heads;
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= (long)a.tokens * heads) return;
  const long t = gid / heads;
  const int h = (int)(gid % heads);
  const bool is_q = h < a.q_heads;
  const bf16* in = reinterpret_cast<const bf16*>(is_q ? a.q_in : a.k_in);
  bf16* out = reinterpret_cast<bf16*>(is_q ? a.q_out : a.k_out);
  const size_t base = (is_q ? ((size_t)t * a.q_heads + h) : ((size_t)t * a.kv_heads + (h - a.q_heads))) * a.head_dim;
  const bool scale_on = is_q && a.q_scale != 1.0f;
  const float s = (float)(bf16)a.q_scale;
  const float sign = a.inverse ? -1.f : 1.f;
  const bf16* cs = reinterpret_cast<const bf16*>(a.cosine) + (size_t)t * a.rotary_pairs;
  const bf16* sn = reinterpret_cast<const bf16*>(a.sine) + (size_t)t * a.rotary_pairs;
  for (int i = 0; i < a.rotary_pairs; ++i) {
    const int c1 = ADJACENT ? 2 * i : i, c2 = ADJACENT ? 2 * i + 1 : i + a.rotary_pairs;
    bf16 x1 = in[base + c1], x2 = in[base + c2];
    if (a.inverse) {
      x1 = scaled(x1, s, scale_on);
      x2 = scaled(x2, s, scale_on);
    }
    const float co = (float)cs[i], si = sign * (float)sn[i];
    bf16 r1 = (bf16)((float)x1 * co - (float)x2 * si);
    bf16 r2 = (bf16)((float)x2 * co + (float)x1 * si);
    if (!a.inverse) {
      r1 = scaled(r1, s, scale_on);
      r2 = scaled(r2, s, scale_on);
    }
    out[base + c1] = r1;
    out[base + c2] = r2;
  }
  for (int c = 2 * a.rotary_pairs; c < a.head_dim; ++c) out[base + c] = scaled(in[base + c], s, scale_on);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// One wavefront per row: f32 mean of squares, r = 1 / sqrt(mean + eps),
// y = bf16(bf16(x r) * scale). The second pass over the row is served from cache.
__global__ __launch_bounds__(256) void rms_norm_fwd_kernel(const uint16_t* x, const uint16_t* scale,
                                                           float eps, long rows, int d, uint16_t* y,
                                                           float* rstd) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const uint16_t* xr = x + (size_t)row * d;
  float ss = 0.f;
  for (int c = lane; c < d / 8; c += 64) {
    const bf16x8 v = as_bf16x8(*reinterpret_cast<const u32x4*>(xr + c * 8));
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += (float)v[e] * (float)v[e];
  }
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)d + eps);
  if (rstd && lane == 0) rstd[row] = r;
  uint16_t* yr = y + (size_t)row * d;
  for (int c = lane; c < d / 8; c += 64) {
    const bf16x8 v = as_bf16x8(*reinterpret_cast<const u32x4*>(xr + c * 8));
    const bf16x8 w = as_bf16x8(*reinterpret_cast<const u32x4*>(scale + c * 8));
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)((float)(bf16)((float)v[e] * r) * (float)w[e]);
    *reinterpret_cast<u32x4*>(yr + c * 8) = as_u32x4(o);
  }
}

// The same for d = 512 NCH with the row held in registers: every load of the row is in flight
// at once and x is read from memory exactly once.
template <int NCH>
__global__ __launch_bounds__(256) void rms_norm_fwd_rows_kernel(const uint16_t* x, const uint16_t* scale,
                                                                float eps, long rows, uint16_t* y,
                                                                float* rstd) {
  constexpr int d = 512 * NCH;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const uint16_t* xr = x + (size_t)row * d;
  bf16x8 v[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) v[i] = as_bf16x8(*reinterpret_cast<const u32x4*>(xr + (lane + 64 * i) * 8));
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += (float)v[i][e] * (float)v[i][e];
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)d + eps);
  if (rstd && lane == 0) rstd[row] = r;
  uint16_t* yr = y + (size_t)row * d;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const bf16x8 w = as_bf16x8(*reinterpret_cast<const u32x4*>(scale + (lane + 64 * i) * 8));
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)((float)(bf16)((float)v[i][e] * r) * (float)w[e]);
    *reinterpret_cast<u32x4*>(yr + (lane + 64 * i) * 8) = as_u32x4(o);
  }
}

// Backward of y = bf16(xhat) * w, xhat = x r: with g = dy w (f32),
//   dx = r (g - xhat mean(g xhat)),   dscale = sum over rows of dy bf16(xhat).
// Wavefront `wv` of the launch takes rows wv, wv + W, ... and keeps its share of dscale in
// registers (NCH chunks of 8 channels per lane, d = 512 NCH); it leaves one f32 partial row
// which rms_norm_dscale_kernel adds up in wavefront order.
template <int NCH>
__global__ __launch_bounds__(256) void rms_norm_bwd_kernel(const uint16_t* x, const uint16_t* scale,
                                                           const uint16_t* dy, float eps, long rows,
                                                           uint16_t* dx, float* partial) {
  constexpr int d = 512 * NCH;
  const int lane = threadIdx.x & 63;
  const long wv = (long)blockIdx.x * 4 + (threadIdx.x >> 6), waves = (long)gridDim.x * 4;
  float acc[NCH][8];
#pragma unroll
  for (int i = 0; i < NCH; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[i][e] = 0.f;
  bf16x8 w[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i)
    w[i] = as_bf16x8(*reinterpret_cast<const u32x4*>(scale + (lane + 64 * i) * 8));

  for (long row = wv; row < rows; row += waves) {
    const uint16_t* xr = x + (size_t)row * d;
    const uint16_t* gr = dy + (size_t)row * d;
    bf16x8 xv[NCH], gv[NCH];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      xv[i] = as_bf16x8(*reinterpret_cast<const u32x4*>(xr + (lane + 64 * i) * 8));
      gv[i] = as_bf16x8(*reinterpret_cast<const u32x4*>(gr + (lane + 64 * i) * 8));
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += (float)xv[i][e] * (float)xv[i][e];
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)d + eps);
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xhat = (float)xv[i][e] * r;
        dot += (float)gv[i][e] * (float)w[i][e] * xhat;
        acc[i][e] += (float)gv[i][e] * (float)(bf16)xhat;
      }
    dot = wave_sum(dot) / (float)d;
    uint16_t* dr = dx + (size_t)row * d;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      bf16x8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xhat = (float)xv[i][e] * r;
        o[e] = (bf16)(r * ((float)gv[i][e] * (float)w[i][e] - xhat * dot));
      }
      *reinterpret_cast<u32x4*>(dr + (lane + 64 * i) * 8) = as_u32x4(o);
    }
  }
  float* prow = partial + (size_t)wv * d;
#pragma unroll
  for (int i = 0; i < NCH; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) prow[(lane + 64 * i) * 8 + e] = acc[i][e];
}

// dscale[col] = sum of the wavefronts' partial rows in a fixed order: thread (c, g) adds the rows
// of sixteenth g for column 64 blockIdx.x + c (four independent chains, joined in order), then the
// sixteen group sums are added in order.
// Any hidden size that is a multiple of 8: the row is walked three times (sum of squares, the
// dot product, dx; the repeats are served from cache) and the wavefront's dscale sums live in its
// row of `partial` instead of registers (a lane only ever touches its own columns of it).
__global__ __launch_bounds__(256) void rms_norm_bwd_any_kernel(const uint16_t* x, const uint16_t* scale,
                                                               const uint16_t* dy, float eps, long rows, int d,
                                                               uint16_t* dx, float* partial) {
  const int lane = threadIdx.x & 63, chunks = d / 8;
  const long wv = (long)blockIdx.x * 4 + (threadIdx.x >> 6), waves = (long)gridDim.x * 4;
  float* prow = partial + (size_t)wv * d;
  for (int c = lane; c < chunks; c += 64)
#pragma unroll
    for (int e = 0; e < 8; ++e) prow[c * 8 + e] = 0.f;
  for (long row = wv; row < rows; row += waves) {
    const uint16_t* xr = x + (size_t)row * d;
    const uint16_t* gr = dy + (size_t)row * d;
    float ss = 0.f;
    for (int c = lane; c < chunks; c += 64) {
      const bf16x8 xv = as_bf16x8(*reinterpret_cast<const u32x4*>(xr + c * 8));
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += (float)xv[e] * (float)xv[e];
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)d + eps);
    float dot = 0.f;
    for (int c = lane; c < chunks; c += 64) {
      const bf16x8 xv = as_bf16x8(*reinterpret_cast<const u32x4*>(xr + c * 8));
      const bf16x8 gv = as_bf16x8(*reinterpret_cast<const u32x4*>(gr + c * 8));
      const bf16x8 wv8 = as_bf16x8(*reinterpret_cast<const u32x4*>(scale + c * 8));
#pragma unroll
      for (int e = 0; e < 8; ++e) dot += (float)gv[e] * (float)wv8[e] * ((float)xv[e] * r);
    }
    dot = wave_sum(dot) / (float)d;
    uint16_t* dr = dx + (size_t)row * d;
    for (int c = lane; c < chunks; c += 64) {
      const bf16x8 xv = as_bf16x8(*reinterpret_cast<const u32x4*>(xr + c * 8));
      const bf16x8 gv = as_bf16x8(*reinterpret_cast<const u32x4*>(gr + c * 8));
      const bf16x8 wv8 = as_bf16x8(*reinterpret_cast<const u32x4*>(scale + c * 8));
      bf16x8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xhat = (float)xv[e] * r;
        o[e] = (bf16)(r * ((float)gv[e] * (float)wv8[e] - xhat * dot));
        prow[c * 8 + e] += (float)gv[e] * (float)(bf16)xhat;
      }
      *reinterpret_cast<u32x4*>(dr + c * 8) = as_u32x4(o);
    }
  }
}

__global__ __launch_bounds__(1024) void rms_norm_dscale_kernel(const float* partial, int waves, int d,
                                                               float* dscale) {
  __shared__ float group[16][64];
  const int c = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int col = blockIdx.x * 64 + c;
  const int per = waves / 16;  // a multiple of 4
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (col < d) {
    const float* p = partial + (size_t)g * per * d + col;
    for (int i = 0; i < per; i += 4) {
      s0 += p[(size_t)i * d];
      s1 += p[(size_t)(i + 1) * d];
      s2 += p[(size_t)(i + 2) * d];
      s3 += p[(size_t)(i + 3) * d];
    }
  }
  group[g][c] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (g == 0 && col < d) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) s += group[k][c];
    dscale[col] = s;
  }
}

constexpr int kNormBwdBlocks = 512;  // 2048 wavefronts, 8 per compute unit

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace ct

using namespace ct;

extern "C" int32_t ct_position_ids(void* stream, const int32_t* attention_mask,
                                   const int32_t* canonical_ids, int32_t batch, int32_t seq,
                                   int32_t* position_ids) {
  CT_REQUIRE(attention_mask && canonical_ids && position_ids, "ct_position_ids: null pointer");
  CT_REQUIRE(batch > 0 && seq > 0, "ct_position_ids: batch and sequence must be positive, got [%d, %d]",
             batch, seq);
  const int threads = seq >= 1024 ? 1024 : ((seq + 63) / 64) * 64;
  LaunchScope scope("position_ids_kernel", (hipStream_t)stream);
  hipLaunchKernelGGL(position_ids_kernel, dim3(batch), dim3(threads), 0, (hipStream_t)stream,
                     attention_mask, canonical_ids, seq, position_ids);
  return scope.done();
}

extern "C" int32_t ct_rotary_cos_sin(void* stream, const int32_t* position_ids, const float* inv_freq,
                                     int64_t tokens, int32_t rotary_pairs, uint16_t* cosine,
                                     uint16_t* sine) {
  CT_REQUIRE(position_ids && inv_freq && cosine && sine, "ct_rotary_cos_sin: null pointer");
  CT_REQUIRE(tokens > 0, "ct_rotary_cos_sin: token count must be positive");
  CT_REQUIRE(rotary_pairs > 0, "ct_rotary_cos_sin: inv_freq must be a non-empty vector");
  const long total = (long)tokens * rotary_pairs;
  LaunchScope scope("rotary_tables_kernel", (hipStream_t)stream);
  hipLaunchKernelGGL(rotary_tables_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, position_ids, inv_freq, (long)tokens, rotary_pairs,
                     reinterpret_cast<bf16*>(cosine), reinterpret_cast<bf16*>(sine));
  return scope.done();
}

extern "C" int32_t ct_apply_rotary(void* stream, const ct_rotary_args* a) {
  CT_REQUIRE(a, "ct_apply_rotary: null args");
  CT_REQUIRE(a->q_in && a->k_in && a->q_out && a->k_out && a->cosine && a->sine,
             "ct_apply_rotary: null pointer");
  CT_REQUIRE(a->tokens > 0 && a->q_heads > 0 && a->kv_heads > 0 && a->head_dim > 0,
             "ct_apply_rotary: dimensions must be positive");
  CT_REQUIRE(a->rope_style == CT_ROPE_GPT_J || a->rope_style == CT_ROPE_GPT_NEOX,
             "ct_apply_rotary: rope_style must be 'gpt-j' or 'gpt-neox'");
  const int rotary_dim = 2 * a->rotary_pairs;
  CT_REQUIRE(a->rotary_pairs > 0 && rotary_dim <= a->head_dim,
             "ct_apply_rotary: invalid rotary dimension %d for head_dim=%d", rotary_dim, a->head_dim);
  const bool vector_path = a->head_dim % 8 == 0 && rotary_dim % 16 == 0;
  CT_REQUIRE(a->q_scale == a->q_scale && a->q_scale - a->q_scale == 0.f,
             "ct_apply_rotary: q_scale must be finite");
  CT_REQUIRE(!vector_path || (aligned16(a->q_in) && aligned16(a->k_in) && aligned16(a->q_out) && aligned16(a->k_out) &&
                              aligned16(a->cosine) && aligned16(a->sine)),
             "ct_apply_rotary: pointers must be 16-byte aligned");
  CT_REQUIRE(a->tokens <= 0x7fffffffll, "ct_apply_rotary: at most 2^31 - 1 tokens per call");
  LaunchScope scope("apply_rotary_kernel", (hipStream_t)stream);
  if (!vector_path) {
    // head_dim not a multiple of 8 or fewer than 16 rotated channels at a time: element-wise kernel
    const long rows = (long)a->tokens * (a->q_heads + a->kv_heads);
    const dim3 grid((unsigned)((rows + 255) / 256));
    if (a->rope_style == CT_ROPE_GPT_J)
      hipLaunchKernelGGL((apply_rotary_rows_kernel<true>), grid, dim3(256), 0, (hipStream_t)stream, *a);
    else
      hipLaunchKernelGGL((apply_rotary_rows_kernel<false>), grid, dim3(256), 0, (hipStream_t)stream, *a);
    return scope.done();
  }
  if (a->rope_style == CT_ROPE_GPT_J)
    hipLaunchKernelGGL((apply_rotary_kernel<true>), dim3((unsigned)a->tokens), dim3(256), 0,
                       (hipStream_t)stream, *a);
  else
    hipLaunchKernelGGL((apply_rotary_kernel<false>), dim3((unsigned)a->tokens), dim3(256), 0,
                       (hipStream_t)stream, *a);
  return scope.done();
}

extern "C" int32_t ct_rms_norm_fwd(void* stream, const uint16_t* x, const uint16_t* scale, float eps,
                                   int64_t rows, int32_t hidden, uint16_t* y, float* rstd) {
  CT_REQUIRE(x && scale && y, "ct_rms_norm_fwd: null pointer");
  CT_REQUIRE(rows > 0 && hidden > 0 && hidden % 8 == 0,
             "ct_rms_norm_fwd: rows must be positive and the hidden size a multiple of 8, got [%lld, %d]",
             (long long)rows, hidden);
  CT_REQUIRE(aligned16(x) && aligned16(scale) && aligned16(y),
             "ct_rms_norm_fwd: pointers must be 16-byte aligned");
  LaunchScope scope("rms_norm_fwd_kernel", (hipStream_t)stream);
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  hipStream_t st = (hipStream_t)stream;
  switch (hidden % 512 == 0 ? hidden / 512 : 0) {
    case 1: hipLaunchKernelGGL((rms_norm_fwd_rows_kernel<1>), grid, block, 0, st, x, scale, eps, (long)rows, y, rstd); break;
    case 2: hipLaunchKernelGGL((rms_norm_fwd_rows_kernel<2>), grid, block, 0, st, x, scale, eps, (long)rows, y, rstd); break;
    case 4: hipLaunchKernelGGL((rms_norm_fwd_rows_kernel<4>), grid, block, 0, st, x, scale, eps, (long)rows, y, rstd); break;
    case 8: hipLaunchKernelGGL((rms_norm_fwd_rows_kernel<8>), grid, block, 0, st, x, scale, eps, (long)rows, y, rstd); break;
    case 16: hipLaunchKernelGGL((rms_norm_fwd_rows_kernel<16>), grid, block, 0, st, x, scale, eps, (long)rows, y, rstd); break;
    default: hipLaunchKernelGGL(rms_norm_fwd_kernel, grid, block, 0, st, x, scale, eps, (long)rows, hidden, y, rstd);
  }
  return scope.done();
}

extern "C" size_t ct_rms_norm_bwd_workspace_bytes(int32_t hidden) {
  if (hidden <= 0) return 0;
  return (size_t)kNormBwdBlocks * 4 * hidden * sizeof(float);
}

extern "C" int32_t ct_rms_norm_bwd(void* stream_, const uint16_t* x, const uint16_t* scale,
                                   const uint16_t* dy, float eps, int64_t rows, int32_t hidden,
                                   uint16_t* dx, float* dscale, void* workspace,
                                   size_t workspace_bytes) {
  CT_REQUIRE(x && scale && dy && dx && dscale && workspace, "ct_rms_norm_bwd: null pointer");
  CT_REQUIRE(rows > 0, "ct_rms_norm_bwd: rows must be positive");
  CT_REQUIRE(hidden > 0 && hidden % 8 == 0, "ct_rms_norm_bwd: hidden size must be a multiple of 8, got %d", hidden);
  CT_REQUIRE(aligned16(x) && aligned16(scale) && aligned16(dy) && aligned16(dx) && aligned16(workspace),
             "ct_rms_norm_bwd: pointers must be 16-byte aligned");
  if (workspace_bytes < ct_rms_norm_bwd_workspace_bytes(hidden))
    return fail(CT_WORKSPACE_TOO_SMALL, "ct_rms_norm_bwd: workspace %zu < %zu bytes", workspace_bytes,
                ct_rms_norm_bwd_workspace_bytes(hidden));
  hipStream_t stream = (hipStream_t)stream_;
  float* partial = static_cast<float*>(workspace);
  LaunchScope scope("rms_norm_bwd_kernel", stream);
  const dim3 grid(kNormBwdBlocks), block(256);
  // rows held in registers for 512 * {1, 2, 4, 8, 16}; any other multiple of 8 walks the row
  const bool in_registers = hidden == 512 || hidden == 1024 || hidden == 2048 || hidden == 4096 || hidden == 8192;
  switch (in_registers ? hidden / 512 : 0) {
    case 0: hipLaunchKernelGGL(rms_norm_bwd_any_kernel, grid, block, 0, stream, x, scale, dy, eps, (long)rows, hidden, dx, partial); break;
    case 1: hipLaunchKernelGGL((rms_norm_bwd_kernel<1>), grid, block, 0, stream, x, scale, dy, eps, (long)rows, dx, partial); break;
    case 2: hipLaunchKernelGGL((rms_norm_bwd_kernel<2>), grid, block, 0, stream, x, scale, dy, eps, (long)rows, dx, partial); break;
    case 4: hipLaunchKernelGGL((rms_norm_bwd_kernel<4>), grid, block, 0, stream, x, scale, dy, eps, (long)rows, dx, partial); break;
    case 8: hipLaunchKernelGGL((rms_norm_bwd_kernel<8>), grid, block, 0, stream, x, scale, dy, eps, (long)rows, dx, partial); break;
    default: hipLaunchKernelGGL((rms_norm_bwd_kernel<16>), grid, block, 0, stream, x, scale, dy, eps, (long)rows, dx, partial); break;
  }
  int rc = scope.done();
  if (rc) return rc;
  LaunchScope scope2("rms_norm_dscale_kernel", stream);
  static_assert(kNormBwdBlocks * 4 % 64 == 0, "dscale kernel splits the partial rows 16 x 4 ways");
  hipLaunchKernelGGL(rms_norm_dscale_kernel, dim3((hidden + 63) / 64), dim3(1024), 0, stream, partial,
                     kNormBwdBlocks * 4, hidden, dscale);
  return scope2.done();
}
