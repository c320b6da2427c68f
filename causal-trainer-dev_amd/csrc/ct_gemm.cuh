// 256 x 256 workgroup-tile bf16 GEMM core for gfx950, used by the cut
// cross-entropy kernels.
//
// 4 wavefronts in a 2 x 2 arrangement, 128 x 128 outputs per wavefront held
// as 4 x 4 mfma32 accumulator blocks (256 f32 registers per lane). Operand
// tiles of BK contraction steps are staged global -> registers -> swizzled
// LDS, double buffered with one barrier per step.
//
// An operand comes in one of two memory layouts:
//   KcLoader  "k-contiguous": matrix rows are the M (or N) index, the
//             contraction index is contiguous. LDS tile [256][BK], MFMA
//             fragments read with ds_read_b128.
//   McLoader  "m-contiguous": matrix rows are the contraction index, the M
//             (or N) index is contiguous. LDS tile [BK][256], fragments read
//             with transposed LDS reads.
// Rows can be addressed through an index list (gather), everything out of
// range is zero filled, and unaligned leading dimensions fall back to
// element-wise loads.
#pragma once

#include <type_traits>

#include "ct_common.cuh"

namespace ct {

constexpr int kGemmTile = 256;

CT_DEVICE u32x4 load_chunk_guarded(const bf16* p, int count, bool aligned) {
  if (count >= 8 && aligned) return load_global16(p);
  bf16x8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = e < count ? p[e] : (bf16)0.f;
  return as_u32x4(v);
}

// Both loaders have a straight-line fast path (every row / column / k of the
// step in range and 16-byte aligned: unconditional 16-byte loads at
// uniform-base + 32-bit lane offsets) and a guarded element-wise path that
// zero fills; the choice is uniform over the workgroup.
template <int BK>
struct KcLoader {
  static constexpr int CPR = BK / 8;
  static constexpr int NCH = BK / 8;          // 16-byte chunks per thread per step
  static constexpr int kRowStep = 256 / CPR;  // rows between a thread's chunks
  const char* base;    // uniform
  unsigned voff[NCH];  // byte offset of this thread's chunk n from base (k = 0)
  u32x4 regs[NCH];
  int lds_off, k_valid, row_mask;
  bool fast;

  // rows m0 .. m0+255 of `base_` (leading dimension ld elements), optionally
  // gathered through row_index. Rows >= rows_valid read as zero, or, with
  // alias_invalid_rows, as a copy of the first row (for callers that discard
  // those rows); k >= k_valid reads as zero.
  CT_DEVICE void init(const bf16* base_, long ld, const int* row_index, int m0, int rows_valid,
                      int k_valid_, bool aligned, bool alias_invalid_rows) {
    const int tid = threadIdx.x, chunk = tid % CPR, row0 = tid / CPR;
    k_valid = k_valid_;
    lds_off = tile_byte_offset<CPR>(row0, chunk);
    const bool gathered = row_index != nullptr;
    base = reinterpret_cast<const char*>(gathered ? base_ : base_ + (size_t)m0 * ld);
    row_mask = 0;
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      const int r = row0 + n * kRowStep;
      const bool ok = m0 + r < rows_valid;
      if (ok || alias_invalid_rows) row_mask |= 1 << n;
      const long src = gathered ? row_index[ok ? m0 + r : 0] : (ok ? r : 0);
      voff[n] = (unsigned)((src * ld + chunk * 8) * 2);
    }
    fast = aligned && (alias_invalid_rows || m0 + kGemmTile <= rows_valid);
  }
  CT_DEVICE void fetch(int k0) {
    if (fast && k0 + BK <= k_valid) {
      const char* p = base + (size_t)k0 * 2;
#pragma unroll
      for (int n = 0; n < NCH; ++n) regs[n] = load_global16(p + voff[n]);
    } else {
      const int k = k0 + (threadIdx.x % CPR) * 8;
      const int count = min(max(k_valid - k, 0), 8);
#pragma unroll
      for (int n = 0; n < NCH; ++n) {
        const bool ok = (row_mask >> n) & 1;
        regs[n] = (ok && count) ? load_chunk_guarded(reinterpret_cast<const bf16*>(
                                                         base + (size_t)k0 * 2 + voff[n]),
                                                     count, false)
                                : u32x4{0u, 0u, 0u, 0u};
      }
    }
  }
  CT_DEVICE void commit(lds_addr tile) const {
#pragma unroll
    for (int n = 0; n < NCH; ++n)
      lds_store<u32x4>(tile + lds_off + n * (kRowStep * CPR * 16), regs[n]);
  }
  // fragment for the wavefront's 32-row block i, contraction steps 16*ks .. 16*ks+15;
  // `wave_first` (multiple of 128) is the wavefront's first row.
  typedef RowFragOffsets<CPR> FragOffsets;
  static CT_DEVICE bf16x8 frag(int tile_off, const FragOffsets& fo, int ks, int wave_first, int i) {
    return fo.load(tile_off + (wave_first / 32) * FragOffsets::kRowBlockBytes, i, ks);
  }
};

template <int BK>
struct McLoader {
  static constexpr int CPR = kGemmTile / 8;  // 32
  static constexpr int NCH = BK / 8;
  const char* base;  // uniform: column m0 of row 0
  const int* row_index;
  long ld;
  unsigned voff[NCH];
  int lds_off[NCH];
  u32x4 regs[NCH];
  int count, k_valid;
  bool fast;

  // columns m0 .. m0+255 of `base_`; contraction rows optionally gathered.
  // Columns >= cols_valid and rows >= k_valid read as zero.
  CT_DEVICE void init(const bf16* base_, long ld_, const int* row_index_, int m0, int cols_valid,
                      int k_valid_, bool aligned) {
    const int tid = threadIdx.x, col = (tid % CPR) * 8, row0 = tid / CPR;
    base = reinterpret_cast<const char*>(base_ + m0);
    row_index = row_index_;
    ld = ld_;
    k_valid = k_valid_;
    count = min(max(cols_valid - m0 - col, 0), 8);
    fast = aligned && m0 + kGemmTile <= cols_valid;
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      const int r = row0 + 8 * n;
      lds_off[n] = tile_byte_offset<CPR>(r, tid % CPR);
      voff[n] = (unsigned)(((row_index ? 0 : (long)r * ld) + col) * 2);
    }
  }
  CT_DEVICE void fetch(int k0) {
    const int row0 = threadIdx.x / CPR;
    if (fast && k0 + BK <= k_valid) {
      if (row_index) {
#pragma unroll
        for (int n = 0; n < NCH; ++n)
          regs[n] = load_global16(base + (size_t)row_index[k0 + row0 + 8 * n] * ld * 2 + voff[n]);
      } else {
        const char* p = base + (size_t)k0 * ld * 2;
#pragma unroll
        for (int n = 0; n < NCH; ++n) regs[n] = load_global16(p + voff[n]);
      }
    } else {
#pragma unroll
      for (int n = 0; n < NCH; ++n) {
        const int k = k0 + row0 + 8 * n;
        if (k < k_valid && count) {
          const size_t src = row_index ? (size_t)row_index[k] : (size_t)k0;
          const char* p = base + src * ld * 2 + voff[n];
          regs[n] = load_chunk_guarded(reinterpret_cast<const bf16*>(p), count, false);
        } else {
          regs[n] = u32x4{0u, 0u, 0u, 0u};
        }
      }
    }
  }
  CT_DEVICE void commit(lds_addr tile) const {
#pragma unroll
    for (int n = 0; n < NCH; ++n) lds_store<u32x4>(tile + lds_off[n], regs[n]);
  }
  typedef TrFragOffsets<CPR, KSlots::kNatural> FragOffsets;
  static CT_DEVICE bf16x8 frag(int tile_off, const FragOffsets& fo, int ks, int wave_first, int i) {
    return fo.load(tile_off + (wave_first / 128) * 256, ks, i);
  }
};

template <int BK>
struct GemmSmem {
  static constexpr int kTileBytes = kGemmTile * BK * 2;
  static constexpr int kStageBytes = 2 * kTileBytes;
  static constexpr size_t kBytes = 2 * kStageBytes;
};

struct GemmAcc {
  f32x16 c[4][4];
  CT_DEVICE void clear() {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) c[a][b] = zero16();
  }
};

// acc += A[m-tile, k_begin:k_end] * B[n-tile, k_begin:k_end]^T. Must be called by
// all 256 threads; ends with the LDS tiles free for reuse.
template <int BK, class ALoader, class BLoader>
CT_DEVICE void gemm_tile(ALoader& A, BLoader& B, int k_begin, int k_end, lds_addr smem,
                         GemmAcc& acc) {
  const int w = threadIdx.x >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  constexpr int kTile = GemmSmem<BK>::kTileBytes, kStage = GemmSmem<BK>::kStageBytes;
  if (k_begin >= k_end) return;
  const typename ALoader::FragOffsets afo(smem);
  const typename BLoader::FragOffsets bfo(smem);
  A.fetch(k_begin);
  B.fetch(k_begin);
  A.commit(smem);
  B.commit(smem + kTile);
  __syncthreads();
  int cur = 0, nxt = kStage;
  for (int k0 = k_begin; k0 < k_end; k0 += BK) {
    const int a_tile = cur, b_tile = cur + kTile;
    const bool more = k0 + BK < k_end;
    if (more) {
      A.fetch(k0 + BK);
      B.fetch(k0 + BK);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 af[4], bfr[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        af[i] = ALoader::frag(a_tile, afo, ks, wm, i);
        bfr[i] = BLoader::frag(b_tile, bfo, ks, wn, i);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int jn = 0; jn < 4; ++jn) acc.c[i][jn] = mfma32(af[i], bfr[jn], acc.c[i][jn]);
    }
    if (more) {
      A.commit(smem + nxt);
      B.commit(smem + nxt + kTile);
    }
    __syncthreads();
    const int tmp = cur;
    cur = nxt;
    nxt = tmp;
  }
}

}  // namespace ct
