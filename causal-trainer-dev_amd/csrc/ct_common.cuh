// Shared device helpers for the gfx950 (CDNA4) hot-path kernels.
//
// Everything here is written for 64-lane wavefronts and the
// v_mfma_f32_32x32x16_bf16 matrix instruction:
//   A operand: lane l holds row  i = l % 32, k-slots 8*(l/32) .. 8*(l/32)+7
//   B operand: lane l holds col  j = l % 32, k-slots 8*(l/32) .. 8*(l/32)+7
//   C / D    : lane l holds col  j = l % 32, register r holds
//              row 8*(r/4) + 4*(l/32) + (r%4)
// Operand tiles live in LDS as dense row-major bf16 with an XOR swizzle on
// 16-byte chunks so that both access patterns below are bank-conflict free:
//   * "k-contiguous" reads (ds_read_b128): 16 consecutive lanes read the
//     same chunk column of 16 consecutive rows;
//   * "transposed" reads (ds_read_b64_tr_b16): 16 lanes read a 4-row x
//     16-column patch and receive it transposed, which is how an operand
//     whose contraction index runs along LDS rows is fetched.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ct {

typedef __bf16 bf16;
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_vs;

#define CT_LDS __attribute__((address_space(3)))
#define CT_DEVICE __device__ __forceinline__

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

CT_DEVICE int lane_id() { return threadIdx.x & 63; }

CT_DEVICE int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

CT_DEVICE f32x16 zero16() {
  f32x16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.f;
  return z;
}

CT_DEVICE f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// Row index (0..31) that accumulator register r of this lane holds.
CT_DEVICE int acc_row(int r, int half) { return 8 * (r >> 2) + 4 * half + (r & 3); }

CT_DEVICE float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

CT_DEVICE float xor32(float v) { return __shfl_xor(v, 32, 64); }

// ---------------------------------------------------------------------------
// Swizzled LDS tiles. CPR = 16-byte chunks per row (row length / 8 elements).
// ---------------------------------------------------------------------------
template <int CPR>
CT_DEVICE int swizzle(int row) {
  if constexpr (CPR >= 16) {
    return ((row & 3) << 2) | ((row >> 2) & 3);
  } else if constexpr (CPR == 8) {
    return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
  } else {
    static_assert(CPR == 4, "unsupported tile width");
    return (row >> 2) & 3;
  }
}

// Element offset of 16-byte chunk `chunk` of `row` inside a swizzled tile.
template <int CPR>
CT_DEVICE int tile_offset(int row, int chunk) {
  return (row * CPR + (chunk ^ swizzle<CPR>(row))) * 8;
}

template <int CPR>
CT_DEVICE void tile_store_chunk(bf16* tile, int row, int chunk, uint4 value) {
  *reinterpret_cast<uint4*>(tile + tile_offset<CPR>(row, chunk)) = value;
}

// k-contiguous operand: 8 consecutive elements of one row.
template <int CPR>
CT_DEVICE bf16x8 tile_read_row8(const bf16* tile, int row, int chunk) {
  return *reinterpret_cast<const bf16x8*>(tile + tile_offset<CPR>(row, chunk));
}

// Transposed operand for mfma32: MFMA index i = lane % 32 runs along tile
// columns col0 .. col0+31, and the 8 k-slots of this lane are tile rows
// rowA .. rowA+3 then rowB .. rowB+3 (callers pass lane-half dependent
// bases, see kslot_rows_*). Two ds_read_b64_tr_b16 per operand.
template <int CPR>
CT_DEVICE bf16x8 tile_read_tr8(const bf16* tile, int rowA, int rowB, int col0) {
  const int l = lane_id();
  const int p = l & 15;
  const int col = col0 + (((l >> 4) & 1) << 4) + ((p & 3) << 2);
  const int chunk = col >> 3;
  const int sub = col & 4;
  const int r0 = rowA + (p >> 2);
  const int r1 = rowB + (p >> 2);
  const bf16* a0 = tile + tile_offset<CPR>(r0, chunk) + sub;
  const bf16* a1 = tile + tile_offset<CPR>(r1, chunk) + sub;
  bf16x4_vs lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((CT_LDS bf16x4_vs*)(a0));
  bf16x4_vs hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((CT_LDS bf16x4_vs*)(a1));
  bf16x8 out;
  out[0] = lo[0]; out[1] = lo[1]; out[2] = lo[2]; out[3] = lo[3];
  out[4] = hi[0]; out[5] = hi[1]; out[6] = hi[2]; out[7] = hi[3];
  return out;
}

// k-slot -> contraction index maps.
// "natural":  slot 8*half+e  <->  k0 + 8*half + e        (matches tile_read_row8)
// "accum":    slot 8*half+e  <->  index held by accumulator registers
//             8t+e of a 32-row block, i.e. k0 + 4*half + e (e<4) and
//             k0 + 8 + 4*half + (e-4) (e>=4), with k0 = 16*t.
// This lets an MFMA result be fed back as the other operand of the next
// MFMA without any cross-lane movement.
CT_DEVICE void kslot_rows_natural(int k0, int half, int& rowA, int& rowB) {
  rowA = k0 + 8 * half;
  rowB = rowA + 4;
}
CT_DEVICE void kslot_rows_accum(int k0, int half, int& rowA, int& rowB) {
  rowA = k0 + 4 * half;
  rowB = rowA + 8;
}

// Pack accumulator registers 8t .. 8t+7 into a bf16 operand (round to nearest even).
CT_DEVICE bf16x8 pack_acc8(const f32x16& c, int t) {
  bf16x8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (bf16)c[8 * t + e];
  return out;
}

CT_DEVICE uint4 load_global16(const void* p) { return *reinterpret_cast<const uint4*>(p); }

CT_DEVICE bf16x8 as_bf16x8(uint4 v) {
  union { uint4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}
CT_DEVICE uint4 as_uint4(bf16x8 v) {
  union { uint4 u; bf16x8 b; } c;
  c.b = v;
  return c.u;
}

// bf16 * bf16 rounded to bf16 (the product of two bf16 values is exact in f32).
CT_DEVICE bf16x8 scale_bf16x8(bf16x8 v, float scale_as_bf16) {
  bf16x8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (bf16)((float)v[e] * scale_as_bf16);
  return out;
}

// Workgroup index remap: consecutive hardware workgroup ids are dealt round
// robin to the 8 XCDs (each with its own L2). Give every XCD one contiguous
// slice of the logical index space so workgroups that share operands share
// an L2.
CT_DEVICE int xcd_remap(int id, int total) {
  constexpr int kXcd = 8;
  if (total % kXcd) return id;
  return (id % kXcd) * (total / kXcd) + id / kXcd;
}

}  // namespace ct
