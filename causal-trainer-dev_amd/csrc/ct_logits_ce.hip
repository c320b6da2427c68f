// Sparse cross-entropy on materialised logits: per-row weighted loss with an online
// log-sum-exp in one pass over HBM, and the analytic logits gradient in one more. The loss
// backend the trainer falls back to when the projection-fused operator is not selected.
//
// Reference: src/kernels/cross_entropy.py:99-190 (_ce_stats_kernel), :254-323 (_ce_bwd_kernel),
// :400-420 (_replicated_loss_and_lse); semantics of the XLA path
// src/kernels/fused_cross_entropy.py:64-106.
#include "ct_error.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ct {

typedef __bf16 bf16;
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2eF = 1.4426950408889634f;
constexpr float kLn2F = 0.6931471805599453f;
constexpr float kNegInfinity = -__builtin_inff();

template <class T>
__device__ __forceinline__ float to_f32(T v) { return (float)v; }

// (m, s): running maximum (log2 domain) and sum of exp2(x log2e - m)
__device__ __forceinline__ void online_add(float& m, float& s, const float* x, int n) {
  float cm = kNegInfinity;
  for (int e = 0; e < n; ++e) cm = fmaxf(cm, x[e]);
  cm *= kLog2eF;
  if (cm > m) {
    s *= exp2f(m - cm);  // m = -inf: s is 0 and stays 0
    m = cm;
  }
  if (m == kNegInfinity) return;  // only -inf so far
  for (int e = 0; e < n; ++e) s += exp2f(fmaf(x[e], kLog2eF, -m));
}
__device__ __forceinline__ void online_merge(float& m, float& s, float mo, float so) {
  const float mn = fmaxf(m, mo);
  if (mn == kNegInfinity) return;
  s = s * exp2f(m - mn) + so * exp2f(mo - mn);
  m = mn;
}

// One workgroup per row. valid = target != ignore_index && weight != 0; invalid rows cost no
// traffic and give loss = lse = 0. A target outside [0, vocab) on a valid row contributes a
// target logit of 0, as the reference's masked lookup does.
template <class T>
__global__ __launch_bounds__(256) void sparse_ce_fwd_kernel(const T* logits, const int* targets,
                                                            const float* weights, int vocab,
                                                            int ignore_index, bool vector_ok,
                                                            float* loss, float* lse) {
  __shared__ float wm[4], ws[4];
  const long row = blockIdx.x;
  const int tid = threadIdx.x;
  const int target = targets[row];
  const float weight = weights[row];
  if (target == ignore_index || weight == 0.f) {
    if (tid == 0) {
      loss[row] = 0.f;
      lse[row] = 0.f;
    }
    return;
  }
  const T* x = logits + (size_t)row * vocab;
  float m = kNegInfinity, s = 0.f;
  constexpr int kPer = 16 / sizeof(T);  // elements per 16-byte access
  int done = 0;
  if (vector_ok) {
    const int chunks = vocab / kPer;
    for (int c = tid; c < chunks; c += 256) {
      float v[kPer];
      if constexpr (sizeof(T) == 2) {
        const bf16x8 raw = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(x + (size_t)c * kPer));
#pragma unroll
        for (int e = 0; e < kPer; ++e) v[e] = (float)raw[e];
      } else {
        const f32x4 raw = *reinterpret_cast<const f32x4*>(x + (size_t)c * kPer);
#pragma unroll
        for (int e = 0; e < kPer; ++e) v[e] = raw[e];
      }
      online_add(m, s, v, kPer);
    }
    done = chunks * kPer;
  }
  for (int i = done + tid; i < vocab; i += 256) {
    const float v = to_f32(x[i]);
    online_add(m, s, &v, 1);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float mo = __shfl_xor(m, off, 64), so = __shfl_xor(s, off, 64);
    online_merge(m, s, mo, so);
  }
  if ((tid & 63) == 0) {
    wm[tid >> 6] = m;
    ws[tid >> 6] = s;
  }
  __syncthreads();
  if (tid == 0) {
    for (int k = 1; k < 4; ++k) online_merge(m, s, wm[k], ws[k]);
    const float row_lse = logf(s) + m * kLn2F;
    const float target_logit = (target >= 0 && target < vocab) ? to_f32(x[target]) : 0.f;
    lse[row] = row_lse;
    loss[row] = weight * (row_lse - target_logit);
  }
}

// grid = (rows, column chunks of 256 * kPer * kIter elements).
// dlogits = w dy (exp(x - lse) - onehot) on valid rows, 0 elsewhere, in the logits dtype.
template <class T>
__global__ __launch_bounds__(256) void sparse_ce_bwd_kernel(const T* logits, const float* lse,
                                                            const int* targets, const float* weights,
                                                            const float* dy, int vocab, int ignore_index,
                                                            bool vector_ok, int chunk_elems, T* dlogits) {
  const long row = blockIdx.x;
  const int tid = threadIdx.x;
  const int target = targets[row];
  const float weight = weights[row];
  const bool valid = target != ignore_index && weight != 0.f;
  const float factor = valid ? weight * dy[row] : 0.f;
  const float lse2 = valid ? lse[row] * kLog2eF : 0.f;
  const T* x = logits + (size_t)row * vocab;
  T* g = dlogits + (size_t)row * vocab;
  constexpr int kPer = 16 / sizeof(T);
  const int begin = blockIdx.y * chunk_elems, end = min(vocab, begin + chunk_elems);
  auto grad = [&](float v, int index) {
    if (!valid) return 0.f;
    return factor * (exp2f(fmaf(v, kLog2eF, -lse2)) - (index == target ? 1.f : 0.f));
  };
  int done = begin;
  if (vector_ok) {  // begin is a multiple of kPer
    const int chunks = (end - begin) / kPer;
    for (int c = tid; c < chunks; c += 256) {
      const int i0 = begin + c * kPer;
      if constexpr (sizeof(T) == 2) {
        bf16x8 out;
        if (valid) {
          const bf16x8 raw = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(x + i0));
#pragma unroll
          for (int e = 0; e < kPer; ++e) out[e] = (bf16)grad((float)raw[e], i0 + e);
        } else {
#pragma unroll
          for (int e = 0; e < kPer; ++e) out[e] = (bf16)0.f;
        }
        *reinterpret_cast<u32x4*>(g + i0) = __builtin_bit_cast(u32x4, out);
      } else {
        f32x4 out = {0.f, 0.f, 0.f, 0.f};
        if (valid) {
          const f32x4 raw = *reinterpret_cast<const f32x4*>(x + i0);
#pragma unroll
          for (int e = 0; e < kPer; ++e) out[e] = grad(raw[e], i0 + e);
        }
        *reinterpret_cast<f32x4*>(g + i0) = out;
      }
    }
    done = begin + chunks * kPer;
  }
  for (int i = done + tid; i < end; i += 256) g[i] = (T)grad(valid ? to_f32(x[i]) : 0.f, i);
}

constexpr int kCeBwdChunk = 256 * 8 * 8;  // elements of a row per workgroup (a multiple of 8)

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static int check_ce(const char* fn, const ct_sparse_ce_args* a) {
  CT_REQUIRE(a, "%s: null args", fn);
  CT_REQUIRE(a->logits && a->targets && a->weights, "%s: null pointer", fn);
  CT_REQUIRE(a->rows > 0 && a->vocab > 0, "%s: logits must have at least one row and one column", fn);
  CT_REQUIRE(a->logits_dtype == CT_DTYPE_BF16 || a->logits_dtype == CT_DTYPE_F32,
             "%s: logits must be bfloat16 or float32", fn);
  CT_REQUIRE(a->rows <= 0x7fffffffLL, "%s: at most 2^31 - 1 rows", fn);
  return CT_OK;
}

}  // namespace ct

using namespace ct;

extern "C" int32_t ct_sparse_ce_fwd(void* stream_, const ct_sparse_ce_args* a, float* loss, float* lse) {
  int rc = check_ce("ct_sparse_ce_fwd", a);
  if (rc) return rc;
  CT_REQUIRE(loss && lse, "ct_sparse_ce_fwd: null output");
  hipStream_t stream = (hipStream_t)stream_;
  const size_t elem = a->logits_dtype == CT_DTYPE_BF16 ? 2 : 4;
  const bool vector_ok = aligned16(a->logits) && ((size_t)a->vocab * elem) % 16 == 0;
  LaunchScope scope("sparse_ce_fwd_kernel", stream);
  if (a->logits_dtype == CT_DTYPE_BF16)
    hipLaunchKernelGGL((sparse_ce_fwd_kernel<bf16>), dim3((unsigned)a->rows), dim3(256), 0, stream,
                       static_cast<const bf16*>(a->logits), a->targets, a->weights, a->vocab,
                       a->ignore_index, vector_ok, loss, lse);
  else
    hipLaunchKernelGGL((sparse_ce_fwd_kernel<float>), dim3((unsigned)a->rows), dim3(256), 0, stream,
                       static_cast<const float*>(a->logits), a->targets, a->weights, a->vocab,
                       a->ignore_index, vector_ok, loss, lse);
  return scope.done();
}

extern "C" int32_t ct_sparse_ce_bwd(void* stream_, const ct_sparse_ce_args* a, const float* lse,
                                    const float* dy, void* dlogits) {
  int rc = check_ce("ct_sparse_ce_bwd", a);
  if (rc) return rc;
  CT_REQUIRE(lse && dy && dlogits, "ct_sparse_ce_bwd: null pointer");
  hipStream_t stream = (hipStream_t)stream_;
  const size_t elem = a->logits_dtype == CT_DTYPE_BF16 ? 2 : 4;
  const bool vector_ok = aligned16(a->logits) && aligned16(dlogits) && ((size_t)a->vocab * elem) % 16 == 0;
  const dim3 grid((unsigned)a->rows, (unsigned)((a->vocab + kCeBwdChunk - 1) / kCeBwdChunk));
  LaunchScope scope("sparse_ce_bwd_kernel", stream);
  if (a->logits_dtype == CT_DTYPE_BF16)
    hipLaunchKernelGGL((sparse_ce_bwd_kernel<bf16>), grid, dim3(256), 0, stream,
                       static_cast<const bf16*>(a->logits), lse, a->targets, a->weights, dy, a->vocab,
                       a->ignore_index, vector_ok, kCeBwdChunk, static_cast<bf16*>(dlogits));
  else
    hipLaunchKernelGGL((sparse_ce_bwd_kernel<float>), grid, dim3(256), 0, stream,
                       static_cast<const float*>(a->logits), lse, a->targets, a->weights, dy, a->vocab,
                       a->ignore_index, vector_ok, kCeBwdChunk, static_cast<float*>(dlogits));
  return scope.done();
}
