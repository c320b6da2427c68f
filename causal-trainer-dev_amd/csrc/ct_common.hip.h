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
// LDS is always addressed through 32-bit byte addresses (lds_addr) and
// address_space(3) accesses, so the compiler emits ds_* instructions with
// immediate offsets instead of flat loads; the lane-dependent, swizzled part
// of every fragment address is computed once per kernel (RowFragOffsets,
// TrFragOffsets) and tile / block / stage bases are added as immediates.
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
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_vs;
// A byte address in LDS. Kept as an address_space(3) pointer so that "pointer + constant"
// folds into the 16-bit offset field of ds_* instructions.
#define CT_LDS __attribute__((address_space(3)))
typedef CT_LDS char* lds_addr;

#define CT_DEVICE __device__ __forceinline__

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

CT_DEVICE int lane_id() { return threadIdx.x & 63; }
// The lane id read from the execution mask at the point of use (all lanes active). Being a
// volatile asm without inputs it is neither hoisted out of a loop nor kept in a register
// across one: values derived from it are recomputed where they are needed.
CT_DEVICE int lane_id_here() {
  int l;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
  return l;
}

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

// Reductions over the lane pair (l, l ^ 32) without an LDS round trip:
// v_permlane32_swap exchanges the upper half of its first operand with the
// lower half of its second, so two copies of v become {lo, lo} and {hi, hi}.
// Both lanes of a pair get the same bits.
CT_DEVICE void halves_of(float v, float& lo, float& hi) {
  lo = v;
  hi = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lo), "+v"(hi));
}
CT_DEVICE float pair_max(float v) {
  float lo, hi;
  halves_of(v, lo, hi);
  return fmaxf(lo, hi);
}
CT_DEVICE float pair_sum(float v) {
  float lo, hi;
  halves_of(v, lo, hi);
  return lo + hi;
}

// ---------------------------------------------------------------------------
// LDS access through 32-bit addresses
// ---------------------------------------------------------------------------
CT_DEVICE lds_addr lds_address_of(void* shared_ptr) { return (lds_addr)shared_ptr; }
template <class T>
CT_DEVICE T lds_load(lds_addr a) {
  return *(CT_LDS const T*)a;
}
template <class T>
CT_DEVICE void lds_store(lds_addr a, T v) {
  *(CT_LDS T*)a = v;
}
CT_DEVICE bf16x4_vs lds_load_tr(lds_addr a) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((CT_LDS bf16x4_vs*)a);
}

// Asynchronous global -> LDS copy of 16 bytes per lane (no registers): lane l
// of the wavefront writes LDS bytes [dst + 16 l, dst + 16 l + 16). `dst` must
// be wave-uniform. Completion is tracked by vmcnt: call dma_wait_all() (or a
// partial vmcnt wait) and then a barrier before other wavefronts read the data.
// Issued through inline assembly on purpose: with the compiler builtin every
// later LDS read is preceded by a full vmcnt(0) wait (the compiler cannot tell
// that the reads touch another stage), which serialises copy and compute.
CT_DEVICE void dma16(const void* src, lds_addr dst) {
  const unsigned m0_value = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)dst);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(src), "s"(m0_value)
               : "memory", "m0");
}
// Same copy with the address split into a wave-uniform base (scalar registers) and a 32-bit
// per-lane byte offset. With loop-invariant lane offsets a copy costs no vector ALU work and
// no vector register is rewritten between copies (rewriting the address registers of a
// queued copy stalls the wavefront until the copy has left the queue).
CT_DEVICE void dma16_s(const void* uniform_base, unsigned lane_offset, lds_addr dst) {
  const unsigned m0_value = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)dst);
  const unsigned long long b = (unsigned long long)(uintptr_t)uniform_base;
  // (the builtin returns a signed int: go through unsigned so that the low half is not sign extended)
  const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)b);
  const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
  const unsigned long long base = ((unsigned long long)hi << 32) | (unsigned long long)lo;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_offset), "s"(base), "s"(m0_value)
               : "memory", "m0");
}
// s_waitcnt vmcnt(0) only (expcnt / lgkmcnt fields left at "no wait")
CT_DEVICE void dma_wait_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// ---------------------------------------------------------------------------
// Swizzled LDS tiles. CPR = 16-byte chunks per row (row length / 8 elements).
// The swizzle only depends on row bits 0..3, and only touches chunk bits
// 0..3, so row offsets that are multiples of 16 rows and chunk offsets that
// are multiples of 16 chunks are plain additive constants.
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

// Byte offset of 16-byte chunk `chunk` of `row` inside a swizzled tile.
template <int CPR>
CT_DEVICE int tile_byte_offset(int row, int chunk) {
  return (row * CPR + (chunk ^ swizzle<CPR>(row))) * 16;
}

// Global -> LDS copy of a ROWS x (8 CPR) bf16 tile into its swizzled layout by
// the THREADS threads of a workgroup: thread t owns the 16-byte LDS slots
// t + THREADS n; the swizzle is undone on the global side (each lane fetches the
// chunk that belongs in its slot). Requires 16 | THREADS / CPR, so one lane
// constant describes all of a thread's slots.
template <int ROWS, int CPR, int THREADS = 256>
struct TileDma {
  static constexpr int kRowsPerPass = THREADS / CPR;
  static constexpr int kPasses = ROWS / kRowsPerPass;
  static_assert(kRowsPerPass % 16 == 0 && ROWS % kRowsPerPass == 0, "unsupported tile shape");
  unsigned lane_off[kPasses];  // byte offset of this thread's chunk in pass n from the tile origin
  // tile row r lives at origin + r * row_stride_bytes (ROWS * row_stride_bytes < 4 GiB)
  CT_DEVICE explicit TileDma(size_t row_stride_bytes) {
    const int t = threadIdx.x;
    const int row0 = t / CPR;
    const int chunk = (t % CPR) ^ swizzle<CPR>(row0);
#pragma unroll
    for (int n = 0; n < kPasses; ++n)
      lane_off[n] = (unsigned)((size_t)(row0 + n * kRowsPerPass) * row_stride_bytes + chunk * 16);
  }
  // origin and tile are workgroup-uniform
  CT_DEVICE void issue(const char* origin, lds_addr tile) const {
    const int wave = uniform(threadIdx.x >> 6);
#pragma unroll
    for (int n = 0; n < kPasses; ++n) dma16_s(origin, lane_off[n], tile + (n * THREADS + wave * 64) * 16);
  }
};

// Per-lane LDS addresses of the k-contiguous MFMA fragments of tiles placed at
// constant offsets from `base`: fragment (row block rb, k-step ks) of the tile
// at base + tile_off is the 16 bytes at
//   ptr[ks] + tile_off + rb * kRowBlockBytes
// and holds row rb*32 + l%32, elements 16 ks + 8 (l/32) .. +7. Keeping the
// lane-dependent part in registers as pointers lets every other term fold into
// the instruction's immediate offset.
template <int CPR>
struct RowFragOffsets {
  static constexpr int kSteps = CPR / 2;
  static constexpr int kRowBlockBytes = 32 * CPR * 16;
  lds_addr ptr[kSteps];
  CT_DEVICE explicit RowFragOffsets(lds_addr base) : RowFragOffsets(base, lane_id()) {}
  CT_DEVICE RowFragOffsets(lds_addr base, int l) {
    const int row = l & 31, half = l >> 5;
#pragma unroll
    for (int ks = 0; ks < kSteps; ++ks) ptr[ks] = base + tile_byte_offset<CPR>(row, 2 * ks + half);
  }
  // The same table from the compact form of the addresses (RowFragCompact): one xor-add per
  // pointer instead of the three operations per pointer of the constructor above.
  template <class Compact>
  CT_DEVICE static RowFragOffsets expand(const Compact& c) {
    RowFragOffsets out;
#pragma unroll
    for (int ks = 0; ks < kSteps; ++ks) out.ptr[ks] = c.row_base + (((unsigned)(2 * ks) << 4) ^ c.x16);
    return out;
  }
  RowFragOffsets() = default;
  CT_DEVICE lds_addr addr(int tile_off, int rb, int ks) const {
    return ptr[ks] + (tile_off + rb * kRowBlockBytes);
  }
  CT_DEVICE bf16x8 load(int tile_off, int rb, int ks) const {
    return lds_load<bf16x8>(addr(tile_off, rb, ks));
  }
};

// k-slot -> contraction index maps for transposed fragments.
// "natural":  slot 8*half+e  <->  k0 + 8*half + e   (matches k-contiguous fragments)
// "accum":    slot 8*half+e  <->  index held by accumulator registers 8t+e
//             of a 32-row block, i.e. k0 + 4*half + e (e<4) and
//             k0 + 8 + 4*half + (e-4) (e>=4), k0 = 16 t. This lets an MFMA
//             result be fed back as an operand without cross-lane movement.
enum class KSlots { kNatural, kAccum };

// Per-lane LDS addresses of transposed MFMA fragments: the MFMA row/column
// index i = l % 32 runs along tile columns cb*32 .. cb*32+31 and the 8
// k-slots of a lane are tile rows. Fragment (column block cb, k-step ks) of
// the tile at base + tile_off is two ds_read_b64_tr_b16 at
//   ptr[second][cb % 4] + tile_off + ks * kStepBytes + (cb / 4) * 256
template <int CPR, KSlots MAP>
struct TrFragOffsets {
  static constexpr int kStepBytes = 16 * CPR * 16;
  lds_addr ptr[2][4];
  CT_DEVICE explicit TrFragOffsets(lds_addr base) : TrFragOffsets(base, lane_id()) {}
  CT_DEVICE TrFragOffsets(lds_addr base, int l) {
    const int p = l & 15, q16 = (l >> 4) & 1, half = l >> 5;
#pragma unroll
    for (int second = 0; second < 2; ++second) {
      const int row = (MAP == KSlots::kNatural ? 8 * half + 4 * second : 4 * half + 8 * second) +
                      (p >> 2);
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) {
        const int col = cb * 32 + 16 * q16 + 4 * (p & 3);
        ptr[second][cb] = base + (tile_byte_offset<CPR>(row, col >> 3) + (col & 4) * 2);
      }
    }
  }
  CT_DEVICE static TrFragOffsets fresh(lds_addr base) { return TrFragOffsets(base); }
  // The same table from the compact form (TrFragCompact): one xor-add per pointer.
  template <class Compact>
  CT_DEVICE static TrFragOffsets expand(const Compact& c) {
    TrFragOffsets out;
#pragma unroll
    for (int second = 0; second < 2; ++second)
#pragma unroll
      for (int cb = 0; cb < 4; ++cb)
        out.ptr[second][cb] = c.row_base[second] + (((unsigned)(cb * 4) << 4) ^ c.y16[second]);
    return out;
  }
  TrFragOffsets() = default;
  CT_DEVICE bf16x8 load(int tile_off, int ks, int cb) const {
    const int off = tile_off + ks * kStepBytes + (cb >> 2) * 256;
    const bf16x4_vs lo = lds_load_tr(ptr[0][cb & 3] + off);
    const bf16x4_vs hi = lds_load_tr(ptr[1][cb & 3] + off);
    bf16x8 out;
    out[0] = lo[0]; out[1] = lo[1]; out[2] = lo[2]; out[3] = lo[3];
    out[4] = hi[0]; out[5] = hi[1]; out[6] = hi[2]; out[7] = hi[3];
    return out;
  }
};

// Register-lean variants of the two structures above for kernels that cannot afford 8 address
// registers per operand: the swizzle is an XOR of the chunk index with a lane constant, and the
// chunk index of a fragment is (compile-time constant) XOR (lane constant), so a fragment
// address is (constant ^ lane term) + lane base: one v_xad_u32 per read instead of a register
// held for the whole kernel. CPR >= 16 only (the 4-bit swizzle).
template <int CPR>
struct RowFragCompact {
  static_assert(CPR >= 16, "compact offsets need the 4-bit swizzle");
  static constexpr int kRowBlockBytes = 32 * CPR * 16;
  lds_addr row_base;  // start of this lane's row
  unsigned x16;       // (half ^ swizzle(row)) * 16
  CT_DEVICE explicit RowFragCompact(lds_addr base) : RowFragCompact(base, lane_id()) {}
  CT_DEVICE RowFragCompact(lds_addr base, int l) {
    const int row = l & 31, half = l >> 5;
    row_base = base + row * CPR * 16;
    x16 = (unsigned)((half ^ swizzle<CPR>(row)) << 4);
  }
  CT_DEVICE lds_addr addr(int tile_off, int rb, int ks) const {
    const unsigned chunk_bytes = ((unsigned)(2 * ks) << 4) ^ x16;
    return row_base + chunk_bytes + (tile_off + rb * kRowBlockBytes);
  }
  CT_DEVICE bf16x8 load(int tile_off, int rb, int ks) const {
    return lds_load<bf16x8>(addr(tile_off, rb, ks));
  }
};

template <int CPR, KSlots MAP>
struct TrFragCompact {
  static_assert(CPR >= 16, "compact offsets need the 4-bit swizzle");
  static constexpr int kStepBytes = 16 * CPR * 16;
  lds_addr row_base[2];  // per read of the pair: row start + the 8-byte half inside the chunk
  unsigned y16[2];       // ((chunk bits below the column block) ^ swizzle(row)) * 16
  CT_DEVICE explicit TrFragCompact(lds_addr base) : TrFragCompact(base, lane_id()) {}
  CT_DEVICE TrFragCompact(lds_addr base, int l) {
    const int p = l & 15, q16 = (l >> 4) & 1, half = l >> 5;
#pragma unroll
    for (int second = 0; second < 2; ++second) {
      const int row = (MAP == KSlots::kNatural ? 8 * half + 4 * second : 4 * half + 8 * second) +
                      (p >> 2);
      const int col_low = 16 * q16 + 4 * (p & 3);  // column inside the 32-column block
      row_base[second] = base + row * CPR * 16 + (col_low & 4) * 2;
      y16[second] = (unsigned)(((col_low >> 3) ^ swizzle<CPR>(row)) << 4);
    }
  }
  // The same addresses rebuilt at the point of use: nothing lane-dependent is then live
  // across the caller's loop (where, once spilled, each such value costs a scratch reload
  // whose wait also drains the asynchronous copies in flight).
  CT_DEVICE static TrFragCompact fresh(lds_addr base) { return TrFragCompact(base, lane_id_here()); }
  CT_DEVICE bf16x8 load(int tile_off, int ks, int cb) const {
    const int off = tile_off + ks * kStepBytes + (cb >> 2) * 256;
    const unsigned block = (unsigned)((cb & 3) * 4) << 4;
    const bf16x4_vs lo = lds_load_tr(row_base[0] + (block ^ y16[0]) + off);
    const bf16x4_vs hi = lds_load_tr(row_base[1] + (block ^ y16[1]) + off);
    bf16x8 out;
    out[0] = lo[0]; out[1] = lo[1]; out[2] = lo[2]; out[3] = lo[3];
    out[4] = hi[0]; out[5] = hi[1]; out[6] = hi[2]; out[7] = hi[3];
    return out;
  }
};

// Pack accumulator registers 8t .. 8t+7 into a bf16 operand (round to nearest even).
CT_DEVICE bf16x8 pack_acc8(const f32x16& c, int t) {
  bf16x8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (bf16)c[8 * t + e];
  return out;
}

CT_DEVICE u32x4 load_global16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
CT_DEVICE void store_global16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }

// The 32 rows of a wavefront (one head, D elements each) as the k-contiguous MFMA fragments of its
// lanes: row l % 32, chunks 2 ks + l / 32. Loaded directly in that form an instruction touches 32
// rows with 32 bytes each, and the address unit of a compute unit, which handles a few cache lines
// per cycle, needs 8-12 k cycles for the three tensors of a dQ tile (measured: a tenth of that
// kernel at short segments). Here the lanes run along the rows instead (an instruction covers 64 /
// CPR whole rows), and the chunks go through the wavefront's LDS patch (swizzled tile layout) to
// the lanes that need them.
template <int D>
struct RowBlockLoader {
  static constexpr int CPR = D / 8;              // 16-byte chunks per row
  static constexpr int kRowsPerLoad = 64 / CPR;  // rows one instruction covers
  static constexpr int kLoads = 32 / kRowsPerLoad;
  u32x4 raw[kLoads];
  // `first_row`: row 0 of the block for this wavefront's head; row stride in elements
  CT_DEVICE void request(const bf16* first_row, size_t row_stride) {
    const int l = lane_id_here();
    const bf16* mine = first_row + (size_t)(l / CPR) * row_stride + (l % CPR) * 8;
#pragma unroll
    for (int n = 0; n < kLoads; ++n) raw[n] = load_global16(mine + (size_t)(n * kRowsPerLoad) * row_stride);
  }
  // (LDS operations of one wavefront complete in order: the reads see the writes, and the next
  // block's writes come after these reads)
  template <class Fragment>
  CT_DEVICE void to_fragments(lds_addr patch, Fragment* fragments) {
    const int l = lane_id_here();
#pragma unroll
    for (int n = 0; n < kLoads; ++n)
      lds_store<u32x4>(patch + tile_byte_offset<CPR>(l / CPR + n * kRowsPerLoad, l % CPR), raw[n]);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks)
      fragments[ks] = lds_load<Fragment>(patch + tile_byte_offset<CPR>(l & 31, 2 * ks + (l >> 5)));
    __builtin_amdgcn_wave_barrier();
  }
};

// 4-byte store to uniform_base + lane_offset + IMM bytes (scalar base, 32-bit lane offset): no
// per-store vector address arithmetic. The scalar base may have just been written by a vector
// instruction (v_readfirstlane): a memory instruction that reads such a register needs 5 wait
// states after the write, and the compiler does not add them in front of an asm statement, so
// each of these stores carries them itself (s_nop 4). A store of more than 8 bytes has a second
// hazard the compiler cannot see through an asm statement: a vector instruction must not write
// the registers that hold the store's data for 2 wait states after it (the data is read late),
// so the 16-byte form ends with s_nop 1.
template <int IMM>
CT_DEVICE void store_global4_s(void* uniform_base, unsigned lane_offset, float value) {
  static_assert(IMM >= 0 && IMM < 4096, "immediate offset out of range");
  const unsigned long long b = (unsigned long long)(uintptr_t)uniform_base;
  const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)b);
  const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
  const unsigned long long base = ((unsigned long long)hi << 32) | (unsigned long long)lo;
  asm volatile("s_nop 4\n\tglobal_store_dword %0, %1, %2 offset:%3" : : "v"(lane_offset), "v"(value), "s"(base), "n"(IMM) : "memory");
}

// 16- and 8-byte stores of the same form.
template <int IMM>
CT_DEVICE void store_global16_s(void* uniform_base, unsigned lane_offset, f32x4 value) {
  static_assert(IMM >= 0 && IMM < 4096, "immediate offset out of range");
  const unsigned long long b = (unsigned long long)(uintptr_t)uniform_base;
  const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)b);
  const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
  const unsigned long long base = ((unsigned long long)hi << 32) | (unsigned long long)lo;
  asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 offset:%3\n\ts_nop 1" : : "v"(lane_offset), "v"(value), "s"(base), "n"(IMM) : "memory");
}
template <int IMM>
CT_DEVICE void store_global8_s(void* uniform_base, unsigned lane_offset, bf16x4 value) {
  static_assert(IMM >= 0 && IMM < 4096, "immediate offset out of range");
  const unsigned long long b = (unsigned long long)(uintptr_t)uniform_base;
  const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)b);
  const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
  const unsigned long long base = ((unsigned long long)hi << 32) | (unsigned long long)lo;
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  const u32x2 bits = __builtin_bit_cast(u32x2, value);
  asm volatile("s_nop 4\n\tglobal_store_dwordx2 %0, %1, %2 offset:%3" : : "v"(lane_offset), "v"(bits), "s"(base), "n"(IMM) : "memory");
}

// The write and read addresses of a wavefront's 32 x D patch (swizzled tile layout) when an
// accumulator leaves through it, with the lane-dependent part formed once: the swizzle is bitwise,
// so the chunk index of a store (a constant) or the row step of a load (a constant) enters as one
// exclusive-or with a constant, and the rows go to memory through a scalar base that advances on
// the scalar unit plus one 32-bit lane offset. (Formed per element from row and chunk numbers, the
// same addresses cost the forward 280 vector instructions per query tile, beside 160 of arithmetic.)
template <int D>
struct PatchRows {
  static constexpr int CPR = D / 8;
  static constexpr int kRowsPerLoad = 64 / CPR;
  static constexpr int kLoads = 32 / kRowsPerLoad;
  // 8-byte store of elements 4 * half .. + 3 of chunk `chunk` (a constant) of row `row`:
  // store_base(patch, row, half) + chunk_term<chunk>(row_swizzle(row))
  static CT_DEVICE lds_addr store_base(lds_addr patch, int row, int half) { return patch + (row * (CPR * 16) + half * 8); }
  static CT_DEVICE unsigned row_swizzle(int row) { return (unsigned)swizzle<CPR>(row) << 4; }
  template <int CHUNK>
  static CT_DEVICE unsigned chunk_term(unsigned swizzle16) { return (unsigned)(CHUNK << 4) ^ swizzle16; }
  // all 32 rows out: lane l takes chunk l % CPR of rows l / CPR + kRowsPerLoad n
  static CT_DEVICE void to_global(lds_addr patch, int l, bf16* first_row, size_t row_stride) {
    const int row0 = l / CPR, c = l % CPR;
    const lds_addr row_base = patch + row0 * (CPR * 16);
    const unsigned chunk16 = (unsigned)((c ^ swizzle<CPR>(row0)) << 4);
    const unsigned lane_offset = (unsigned)(row0 * row_stride * 2) + (unsigned)(c * 16);
    char* base = reinterpret_cast<char*>(first_row);
    const size_t step = (size_t)kRowsPerLoad * row_stride * 2;
#pragma unroll
    for (int n = 0; n < kLoads; ++n) {
      // rows row0 and kRowsPerLoad n have no set bit in common: swizzle(row0 + kRowsPerLoad n) is
      // the exclusive-or of their swizzles
      const unsigned term = chunk16 ^ ((unsigned)swizzle<CPR>(kRowsPerLoad * n) << 4);
      const u32x4 val = lds_load<u32x4>(row_base + term + n * (kRowsPerLoad * CPR * 16));
      store_global16_s<0>(base + n * step, lane_offset, __builtin_bit_cast(f32x4, val));
    }
  }
};


CT_DEVICE bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }
CT_DEVICE u32x4 as_u32x4(bf16x8 v) { return __builtin_bit_cast(u32x4, v); }

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
