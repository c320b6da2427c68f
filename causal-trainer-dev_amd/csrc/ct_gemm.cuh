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

template <int BK>
struct KcLoader {
  static constexpr int CPR = BK / 8;
  static constexpr int NCH = BK / 8;          // 16-byte chunks per thread per step
  static constexpr int kRowStep = 256 / CPR;  // rows between a thread's chunks
  static constexpr int kTileElems = kGemmTile * BK;
  const bf16* row_ptr[NCH];
  u32x4 regs[NCH];
  int chunk, k_valid;
  bool aligned;

  // rows m0 .. m0+255 of `base` (leading dimension ld), optionally gathered
  // through row_index; rows >= rows_valid and k >= k_valid read as zero.
  CT_DEVICE void init(const bf16* base, long ld, const int* row_index, int m0, int rows_valid,
                      int k_valid_, bool aligned_) {
    const int tid = threadIdx.x;
    chunk = tid % CPR;
    k_valid = k_valid_;
    aligned = aligned_;
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      const int gm = m0 + tid / CPR + n * kRowStep;
      const bool ok = gm < rows_valid;
      const long src = ok ? (row_index ? row_index[gm] : gm) : 0;
      row_ptr[n] = ok ? base + src * ld : nullptr;
    }
  }
  CT_DEVICE void fetch(int k0) {
    const int k = k0 + chunk * 8;
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      const int count = row_ptr[n] ? min(max(k_valid - k, 0), 8) : 0;
      regs[n] = count ? load_chunk_guarded(row_ptr[n] + k, count, aligned) : u32x4{0u, 0u, 0u, 0u};
    }
  }
  CT_DEVICE void commit(lds_addr tile) const {
    const int tid = threadIdx.x;
#pragma unroll
    for (int n = 0; n < NCH; ++n)
      lds_store<u32x4>(tile + tile_byte_offset<CPR>(tid / CPR + n * kRowStep, chunk), regs[n]);
  }
  // fragment for MFMA rows/cols first .. first+31, contraction steps 16*ks .. 16*ks+15
  typedef RowFragOffsets<CPR> FragOffsets;
  // `wave_first` (multiple of 128) is the wavefront's first row, `i` its 32-row block.
  static CT_DEVICE bf16x8 frag(lds_addr tile, const FragOffsets& fo, int ks, int wave_first, int i) {
    return lds_load<bf16x8>(tile + (wave_first / 32 + i) * FragOffsets::kRowBlockBytes + fo.off[ks]);
  }
};

template <int BK>
struct McLoader {
  static constexpr int CPR = kGemmTile / 8;  // 32
  static constexpr int NCH = BK / 8;
  static constexpr int kTileElems = kGemmTile * BK;
  const bf16* base;
  const int* row_index;
  long ld;
  u32x4 regs[NCH];
  int m0, cols_valid, k_valid;
  bool aligned;

  // columns m0 .. m0+255 of `base`; contraction rows optionally gathered.
  CT_DEVICE void init(const bf16* base_, long ld_, const int* row_index_, int m0_, int cols_valid_,
                      int k_valid_, bool aligned_) {
    base = base_;
    ld = ld_;
    row_index = row_index_;
    m0 = m0_;
    cols_valid = cols_valid_;
    k_valid = k_valid_;
    aligned = aligned_;
  }
  CT_DEVICE void fetch(int k0) {
    const int tid = threadIdx.x;
    const int m = m0 + (tid % CPR) * 8;
    const int count = min(max(cols_valid - m, 0), 8);
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      const int k = k0 + tid / CPR + 8 * n;
      if (k < k_valid && count) {
        const long src = row_index ? row_index[k] : k;
        regs[n] = load_chunk_guarded(base + src * ld + m, count, aligned);
      } else {
        regs[n] = u32x4{0u, 0u, 0u, 0u};
      }
    }
  }
  CT_DEVICE void commit(lds_addr tile) const {
    const int tid = threadIdx.x;
#pragma unroll
    for (int n = 0; n < NCH; ++n)
      lds_store<u32x4>(tile + tile_byte_offset<CPR>(tid / CPR + 8 * n, tid % CPR), regs[n]);
  }
  typedef TrFragOffsets<CPR, KSlots::kNatural> FragOffsets;
  static CT_DEVICE bf16x8 frag(lds_addr tile, const FragOffsets& fo, int ks, int wave_first, int i) {
    return fo.load(tile + (wave_first / 128) * 256, ks, i);
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
  const typename ALoader::FragOffsets afo;
  const typename BLoader::FragOffsets bfo;
  A.fetch(k_begin);
  B.fetch(k_begin);
  A.commit(smem);
  B.commit(smem + kTile);
  __syncthreads();
  lds_addr cur = smem, nxt = smem + kStage;
  for (int k0 = k_begin; k0 < k_end; k0 += BK) {
    const lds_addr a_tile = cur, b_tile = cur + kTile;
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
      A.commit(nxt);
      B.commit(nxt + kTile);
    }
    __syncthreads();
    const lds_addr tmp = cur;
    cur = nxt;
    nxt = tmp;
  }
}

}  // namespace ct
