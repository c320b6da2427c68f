// Device-side preparation steps that sit directly in front of the two hot paths and define
// their ignored-token sets: segment id canonicalisation and shifted targets / loss weights.
// Integer work, bit-exact against the reference (src/modeling/rotary.py:13-50,
// src/training/losses.py:21-85).
#include "ct_error.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ct {

// One workgroup per batch row. ids[s] = number of run starts in [0, s] where position s is
// valid, else 0; a run starts at a valid position whose predecessor is invalid or carries a
// different label (position 0 compares its label with itself, as the reference does).
// VALID_IS_ONE: a position is valid iff mask == 1 (the loss path), else iff mask != 0.
template <bool VALID_IS_ONE>
__global__ __launch_bounds__(1024) void canonicalize_kernel(const int* mask, const int* labels,
                                                            int S, int* out) {
  __shared__ int wave_sums[16];
  __shared__ int carry_s;
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nwaves = blockDim.x >> 6;
  const int* mrow = mask ? mask + (size_t)b * S : nullptr;
  const int* lrow = labels ? labels + (size_t)b * S : nullptr;
  int* orow = out + (size_t)b * S;
  auto valid_at = [&](int s) {
    if (!mrow) return true;
    return VALID_IS_ONE ? mrow[s] == 1 : mrow[s] != 0;
  };
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (int base = 0; base < S; base += blockDim.x) {
    const int s = base + tid;
    bool valid = false, start = false;
    if (s < S) {
      valid = valid_at(s);
      const bool prev_valid = s > 0 && valid_at(s - 1);
      const int label = lrow ? lrow[s] : 0;
      const int prev_label = lrow ? lrow[s > 0 ? s - 1 : 0] : 0;
      start = valid && (!prev_valid || label != prev_label);
    }
    // inclusive scan of `start` over the workgroup
    int incl = start ? 1 : 0;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int other = __shfl_up(incl, off, 64);
      if (lane >= off) incl += other;
    }
    if (lane == 63) wave_sums[wave] = incl;
    __syncthreads();
    int before = carry_s;
    for (int k = 0; k < wave; ++k) before += wave_sums[k];
    if (s < S) orow[s] = valid ? before + incl : 0;
    __syncthreads();
    if (tid == 0) {
      int total = carry_s;
      for (int k = 0; k < nwaves; ++k) total += wave_sums[k];
      carry_s = total;
    }
    __syncthreads();
  }
}

// targets[b, s] = labels[b, s + 1] where the weight is positive, else 0;
// weights[b, s] = valid edge * assistant[s + 1] * loss_mask[s + 1]  (f32 products in that order).
__global__ __launch_bounds__(256) void shifted_targets_kernel(
    const int* input_ids, const int* labels, const int* mask, const int* canonical,
    const int* assistant, const float* loss_mask, int ignore_index, int B, int S, int* targets,
    float* weights) {
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  const long total = (long)B * (S - 1);
  if (gid >= total) return;
  const int b = (int)(gid / (S - 1)), s = (int)(gid % (S - 1));
  const size_t here = (size_t)b * S + s, next = here + 1;
  const int* lab = labels ? labels : input_ids;
  const int target = lab[next];
  bool valid = target != ignore_index;
  if (mask) valid = valid && mask[here] == 1 && mask[next] == 1;
  if (canonical) valid = valid && canonical[here] == canonical[next] && canonical[next] != 0;
  float w = valid ? 1.f : 0.f;
  if (assistant) w *= (assistant[next] != 0) ? 1.f : 0.f;
  if (loss_mask) w *= loss_mask[next];
  weights[gid] = w;
  targets[gid] = w > 0.f ? target : 0;
}

static int check_dims(const char* fn, int batch, int seq) {
  CT_REQUIRE(batch > 0 && seq > 0, "%s: batch and sequence must be positive, got [%d, %d]", fn,
             batch, seq);
  return CT_OK;
}

}  // namespace ct

using namespace ct;

extern "C" int32_t ct_canonicalize_segment_ids(void* stream, const int32_t* attention_mask,
                                               const int32_t* segment_ids, int32_t batch,
                                               int32_t seq, int32_t* canonical_ids) {
  CT_REQUIRE(attention_mask && canonical_ids, "ct_canonicalize_segment_ids: null pointer");
  int rc = check_dims("ct_canonicalize_segment_ids", batch, seq);
  if (rc) return rc;
  const int threads = seq >= 1024 ? 1024 : ((seq + 63) / 64) * 64;
  LaunchScope scope("canonicalize_kernel", (hipStream_t)stream);
  hipLaunchKernelGGL((canonicalize_kernel<false>), dim3(batch), dim3(threads), 0, (hipStream_t)stream,
                     attention_mask, segment_ids, seq, canonical_ids);
  return scope.done();
}

extern "C" size_t ct_shifted_targets_scratch_bytes(int32_t batch, int32_t seq) {
  if (batch <= 0 || seq <= 0) return 0;
  return (size_t)batch * seq * sizeof(int32_t);
}

extern "C" int32_t ct_shifted_targets_and_weights(void* stream_, const ct_shifted_targets_args* a) {
  CT_REQUIRE(a, "ct_shifted_targets_and_weights: null args");
  CT_REQUIRE(a->input_ids && a->targets && a->weights, "ct_shifted_targets_and_weights: null pointer");
  int rc = check_dims("ct_shifted_targets_and_weights", a->batch, a->seq);
  if (rc) return rc;
  CT_REQUIRE(a->seq >= 2, "ct_shifted_targets_and_weights: sequence length %d leaves no prediction edge",
             a->seq);
  hipStream_t stream = (hipStream_t)stream_;
  int* canonical = nullptr;
  if (a->segment_ids) {
    CT_REQUIRE(a->scratch && a->scratch_bytes >= ct_shifted_targets_scratch_bytes(a->batch, a->seq),
               "ct_shifted_targets_and_weights: scratch of %zu bytes needed with segment ids",
               ct_shifted_targets_scratch_bytes(a->batch, a->seq));
    canonical = static_cast<int*>(a->scratch);
    const int threads = a->seq >= 1024 ? 1024 : ((a->seq + 63) / 64) * 64;
    LaunchScope scope1("canonicalize_kernel", stream);
    // validity for the loss is "mask == 1" (src/training/losses.py:52), not "mask != 0"
    hipLaunchKernelGGL((canonicalize_kernel<true>), dim3(a->batch), dim3(threads), 0, stream,
                       a->attention_mask, a->segment_ids, a->seq, canonical);
    if ((rc = scope1.done())) return rc;
  }
  const long total = (long)a->batch * (a->seq - 1);
  LaunchScope scope2("shifted_targets_kernel", stream);
  hipLaunchKernelGGL(shifted_targets_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                     a->input_ids, a->labels, a->attention_mask, canonical, a->assistant_mask,
                     a->loss_mask, a->ignore_index, a->batch, a->seq, a->targets, a->weights);
  return scope2.done();
}
