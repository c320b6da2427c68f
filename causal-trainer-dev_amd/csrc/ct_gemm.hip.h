// 256 x 256 workgroup-tile bf16 GEMM core for gfx950, used by the cut
// cross-entropy kernels.
//
// 4 wavefronts in a 2 x 2 arrangement, 128 x 128 outputs per wavefront held
// as 4 x 4 mfma32 accumulator blocks (256 f32 registers per lane). The
// contraction runs in steps of BK = 32.
//
// An operand comes in one of two memory layouts:
//   KcLoader  "k-contiguous": matrix rows are the M (or N) index, the
//             contraction index is contiguous. LDS tile [256][BK], MFMA
//             fragments read with ds_read_b128.
//   McLoader  "m-contiguous": matrix rows are the contraction index, the M
//             (or N) index is contiguous. LDS tile [BK][256], fragments read
//             with transposed LDS reads.
// Rows can be addressed through an index list (gather).
//
// Two main loops share the loaders:
//   pipelined  every row / column / k of the tile is in range and 16-byte
//              aligned: tiles are copied global -> LDS asynchronously, three
//              steps ahead, into a ring of 4 LDS stages; MFMA fragments are
//              double buffered in registers so that LDS reads of the next
//              half step overlap the 16 MFMAs of the current one; one
//              barrier per step.
//   guarded    anything ragged or unaligned: element-wise guarded loads that
//              zero fill, staged through registers, 2 LDS stages.
// The choice is uniform over the workgroup.
#pragma once

#include <type_traits>

#include "ct_common.hip.h"
#include "ct_gemm_asm.inc"

namespace ct {

constexpr int kGemmTile = 256;
constexpr int kGemmBK = 32;

CT_DEVICE u32x4 load_chunk_guarded(const bf16* p, int count) {
  bf16x8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = e < count ? p[e] : (bf16)0.f;
  return as_u32x4(v);
}

struct GemmSmem {
  static constexpr int kTileBytes = kGemmTile * kGemmBK * 2;  // 16 KB
  static constexpr int kStageBytes = 2 * kTileBytes;          // A tile then B tile
  static constexpr int kStages = 4;
  static constexpr size_t kBytes = (size_t)kStages * kStageBytes;  // 128 KB
};

// In both loaders thread t owns the 16-byte LDS slots t + 256 n of the tile
// (n < 4): slot P holds physical chunk P % CPR of row P / CPR, i.e. logical
// chunk (P % CPR) ^ swizzle(row); voff[n] is the byte offset of that chunk
// from `base` at k = 0.
struct KcLoader {
  static constexpr int CPR = kGemmBK / 8;  // 4
  static constexpr int NCH = 4;
  const char* base;    // uniform
  unsigned voff[NCH];
  u32x4 regs[NCH];
  int chunk, k_valid, row_mask;
  bool fast;

  // rows m0 .. m0+255 of `base_` (leading dimension ld elements), optionally
  // gathered through row_index. Rows >= rows_valid read as zero, or, with
  // alias_invalid_rows, as a copy of the first row (for callers that discard
  // those rows); k >= k_valid reads as zero.
  // With interleave_rows, tile row 128 w + 32 nb + j holds matrix row m0 + 128 w + 4 j + nb:
  // in the accumulator layout lane j of a wavefront then owns 4 consecutive matrix rows (its
  // column blocks nb = 0..3), which an epilogue can store with one 8- or 16-byte access.
  CT_DEVICE void init(const bf16* base_, long ld, const int* row_index, int m0, int rows_valid,
                      int k_valid_, bool aligned, bool alias_invalid_rows,
                      bool interleave_rows = false) {
    const int t = threadIdx.x;
    k_valid = k_valid_;
    const bool gathered = row_index != nullptr;
    base = reinterpret_cast<const char*>(gathered ? base_ : base_ + (size_t)m0 * ld);
    row_mask = 0;
    const int r0 = t / CPR;
    chunk = (t % CPR) ^ swizzle<CPR>(r0);  // rows r0 + 64 n share the swizzle
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      const int tile_row = r0 + 64 * n;
      const int r = interleave_rows ? ((tile_row & 128) | ((tile_row & 31) << 2) | ((tile_row >> 5) & 3))
                                    : tile_row;
      const bool ok = m0 + r < rows_valid;
      if (ok || alias_invalid_rows) row_mask |= 1 << n;
      const long src = gathered ? row_index[ok ? m0 + r : 0] : (ok ? r : 0);
      voff[n] = (unsigned)((src * ld + chunk * 8) * 2);
    }
    fast = aligned && (alias_invalid_rows || m0 + kGemmTile <= rows_valid) && k_valid % kGemmBK == 0;
  }
  // copies N0 .. N1-1 of the thread's NCH 16-byte slots
  template <int N0 = 0, int N1 = NCH>
  CT_DEVICE void dma(int k0, lds_addr tile) const {
    const int wave = uniform(threadIdx.x >> 6);
    const char* p = base + (size_t)k0 * 2;
#pragma unroll
    for (int n = N0; n < N1; ++n) dma16_s(p, voff[n], tile + (n * 256 + wave * 64) * 16);
  }
  CT_DEVICE void fetch(int k0) {
    const int k = k0 + chunk * 8;
    const int count = min(max(k_valid - k, 0), 8);
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      const bool ok = (row_mask >> n) & 1;
      regs[n] = (ok && count) ? load_chunk_guarded(reinterpret_cast<const bf16*>(
                                                       base + (size_t)k0 * 2 + voff[n]),
                                                   count)
                              : u32x4{0u, 0u, 0u, 0u};
    }
  }
  CT_DEVICE void commit(lds_addr tile) const {
#pragma unroll
    for (int n = 0; n < NCH; ++n) lds_store<u32x4>(tile + (n * 256 + (int)threadIdx.x) * 16, regs[n]);
  }
  // fragment for the wavefront's 32-row block i, contraction steps 16*ks .. 16*ks+15;
  // `wave_first` (multiple of 128) is the wavefront's first row.
  typedef RowFragOffsets<CPR> FragOffsets;
  static CT_DEVICE bf16x8 frag(int tile_off, const FragOffsets& fo, int ks, int wave_first, int i) {
    return fo.load(tile_off + (wave_first / 32) * FragOffsets::kRowBlockBytes, i, ks);
  }
};

struct McLoader {
  static constexpr int CPR = kGemmTile / 8;  // 32
  static constexpr int NCH = 4;
  const char* base;  // uniform: column m0 of row 0
  const int* row_index;
  long ld;
  unsigned voff[NCH];
  u32x4 regs[NCH];
  int col[2];  // first column of the chunk fetched in even / odd passes
  int cols_left, k_valid;
  bool fast;

  // columns m0 .. m0+255 of `base_`; contraction rows optionally gathered.
  // Columns >= cols_valid and rows >= k_valid read as zero.
  CT_DEVICE void init(const bf16* base_, long ld_, const int* row_index_, int m0, int cols_valid,
                      int k_valid_, bool aligned) {
    const int t = threadIdx.x;
    base = reinterpret_cast<const char*>(base_ + m0);
    row_index = row_index_;
    ld = ld_;
    k_valid = k_valid_;
    cols_left = cols_valid - m0;
    fast = aligned && m0 + kGemmTile <= cols_valid && k_valid % kGemmBK == 0;
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      const int r = t / CPR + 8 * n;
      const int c = ((t % CPR) ^ swizzle<CPR>(r)) * 8;
      col[n & 1] = c;
      voff[n] = (unsigned)(((row_index ? 0 : (long)r * ld) + c) * 2);
    }
  }
  // copies N0 .. N1-1 of the thread's NCH 16-byte slots (N0 even, N1 = N0 + 2 or NCH)
  template <int N0 = 0, int N1 = NCH>
  CT_DEVICE void dma(int k0, lds_addr tile) const {
    const int wave = uniform(threadIdx.x >> 6);
    if (row_index) {
      // A wavefront covers rows k0 + 2 wave + {0, 1} + 8 n: read the two row indices
      // with scalar loads (tracked by lgkmcnt, so they do not force the copies
      // still in flight to drain the way a vector load would).
      typedef int i32x2 __attribute__((ext_vector_type(2)));
      const int* ip = row_index + k0 + 2 * wave + 8 * N0;
      const bool upper = lane_id() >= 32;
#pragma unroll
      for (int n = N0; n < N1; n += 2) {
        i32x2 p0, p1;
        asm volatile(
            "s_load_dwordx2 %0, %2, 0x0\n\ts_load_dwordx2 %1, %2, 0x20\n\ts_waitcnt lgkmcnt(0)"
            : "=&s"(p0), "=&s"(p1)
            : "s"(ip + 8 * (n - N0))
            : "memory");
        dma16(base + (size_t)(upper ? p0[1] : p0[0]) * ld * 2 + voff[n],
              tile + (n * 256 + wave * 64) * 16);
        dma16(base + (size_t)(upper ? p1[1] : p1[0]) * ld * 2 + voff[n + 1],
              tile + ((n + 1) * 256 + wave * 64) * 16);
      }
    } else {
      const char* p = base + (size_t)k0 * ld * 2;
#pragma unroll
      for (int n = N0; n < N1; ++n) dma16_s(p, voff[n], tile + (n * 256 + wave * 64) * 16);
    }
  }
  CT_DEVICE void fetch(int k0) {
    const int r0 = (int)threadIdx.x / CPR;
#pragma unroll
    for (int n = 0; n < NCH; ++n) {
      const int k = k0 + r0 + 8 * n;
      const int count = min(max(cols_left - col[n & 1], 0), 8);
      if (k < k_valid && count) {
        const size_t src = row_index ? (size_t)row_index[k] : (size_t)k0;
        regs[n] = load_chunk_guarded(reinterpret_cast<const bf16*>(base + src * ld * 2 + voff[n]),
                                     count);
      } else {
        regs[n] = u32x4{0u, 0u, 0u, 0u};
      }
    }
  }
  CT_DEVICE void commit(lds_addr tile) const {
#pragma unroll
    for (int n = 0; n < NCH; ++n) lds_store<u32x4>(tile + (n * 256 + (int)threadIdx.x) * 16, regs[n]);
  }
  typedef TrFragOffsets<CPR, KSlots::kNatural> FragOffsets;
  static CT_DEVICE bf16x8 frag(int tile_off, const FragOffsets& fo, int ks, int wave_first, int i) {
    return fo.load(tile_off + (wave_first / 128) * 256, ks, i);
  }
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

struct GemmFrags {
  bf16x8 a[4], b[4];
};

template <class ALoader, class BLoader>
CT_DEVICE void load_frags(GemmFrags& f, int stage_off, const typename ALoader::FragOffsets& afo,
                          const typename BLoader::FragOffsets& bfo, int ks, int wm, int wn) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f.a[i] = ALoader::frag(stage_off, afo, ks, wm, i);
    f.b[i] = BLoader::frag(stage_off + GemmSmem::kTileBytes, bfo, ks, wn, i);
  }
}

CT_DEVICE void mfma_block(const GemmFrags& f, GemmAcc& acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int jn = 0; jn < 4; ++jn) acc.c[i][jn] = mfma32(f.a[i], f.b[jn], acc.c[i][jn]);
}

template <int I0, int I1>
CT_DEVICE void mfma_rows(const GemmFrags& f, GemmAcc& acc) {
#pragma unroll
  for (int i = I0; i < I1; ++i)
#pragma unroll
    for (int jn = 0; jn < 4; ++jn) acc.c[i][jn] = mfma32(f.a[i], f.b[jn], acc.c[i][jn]);
}

// s_waitcnt vmcnt(N) for N in {0, 8, 12, 16} (expcnt / lgkmcnt left at "no wait").
CT_DEVICE void wait_vmcnt(int outstanding) {
  if (outstanding >= 16)
    __builtin_amdgcn_s_waitcnt(0x0F70 | (1 << 14));  // vmcnt = 16
  else if (outstanding >= 12)
    __builtin_amdgcn_s_waitcnt(0x0F70 | 12);
  else if (outstanding >= 8)
    __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
  else
    __builtin_amdgcn_s_waitcnt(0x0F70);
}
CT_DEVICE void wait_lds() { __builtin_amdgcn_s_waitcnt(0xC07F); }  // lgkmcnt(0) only
// Execution barrier without the memory fence of __syncthreads() (which would wait for
// every copy in flight); callers order their own LDS traffic with the waits above.
CT_DEVICE void workgroup_barrier() { __builtin_amdgcn_s_barrier(); }

// The pipelined main loop with a fixed instruction order (see gen_gemm_asm.py), for an
// m-contiguous A without row gather, a k-contiguous B and a step count that is a positive
// multiple of 4. Entered with the copies of steps 0..2 issued and step 0 landed for every
// wavefront; returns with nothing in flight and the LDS tiles free.
CT_DEVICE unsigned long long uniform64(const void* p) {
  const unsigned long long b = (unsigned long long)(uintptr_t)p;
  const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)b);
  const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
  return ((unsigned long long)hi << 32) | (unsigned long long)lo;
}
CT_DEVICE void gemm_loop_scheduled(const McLoader& A, const KcLoader& B, int k_begin, int steps,
                                   lds_addr smem, const McLoader::FragOffsets& afo,
                                   const KcLoader::FragOffsets& bfo, int wm, int wn, GemmAcc& acc) {
  const int wave = uniform(threadIdx.x >> 6);
  // sources of the copies of step 3
  const unsigned long long src_a =
      uniform64(A.base + (size_t)(k_begin + 3 * kGemmBK) * (size_t)A.ld * 2);
  const unsigned long long src_b = uniform64(B.base + (size_t)(k_begin + 3 * kGemmBK) * 2);
  const unsigned stride_a = (unsigned)uniform((int)(kGemmBK * A.ld * 2));
  const unsigned steps_u = (unsigned)uniform(steps);
  const unsigned lds_wave = (unsigned)uniform((int)(uintptr_t)(smem + wave * 1024));
  const int a_off = (wm / 128) * 256;
  const int b_off = GemmSmem::kTileBytes + (wn / 32) * KcLoader::FragOffsets::kRowBlockBytes;
  asm volatile(CT_GEMM_LOOP
               : "+a"(acc.c[0][0]), "+a"(acc.c[0][1]), "+a"(acc.c[0][2]), "+a"(acc.c[0][3]),
                 "+a"(acc.c[1][0]), "+a"(acc.c[1][1]), "+a"(acc.c[1][2]), "+a"(acc.c[1][3]),
                 "+a"(acc.c[2][0]), "+a"(acc.c[2][1]), "+a"(acc.c[2][2]), "+a"(acc.c[2][3]),
                 "+a"(acc.c[3][0]), "+a"(acc.c[3][1]), "+a"(acc.c[3][2]), "+a"(acc.c[3][3])
               : "s"(src_a), "s"(src_b), "s"(stride_a), "s"(steps_u), "s"(lds_wave),
                 "v"(afo.ptr[0][0] + a_off), "v"(afo.ptr[0][1] + a_off), "v"(afo.ptr[0][2] + a_off),
                 "v"(afo.ptr[0][3] + a_off), "v"(afo.ptr[1][0] + a_off), "v"(afo.ptr[1][1] + a_off),
                 "v"(afo.ptr[1][2] + a_off), "v"(afo.ptr[1][3] + a_off), "v"(bfo.ptr[0] + b_off),
                 "v"(bfo.ptr[1] + b_off), "v"(A.voff[0]), "v"(A.voff[1]), "v"(A.voff[2]),
                 "v"(A.voff[3]), "v"(B.voff[0]), "v"(B.voff[1]), "v"(B.voff[2]), "v"(B.voff[3])
               : "memory", "m0", "scc", CT_GEMM_LOOP_CLOBBERS);
}

// acc += A[m-tile, k_begin:k_end] * B[n-tile, k_begin:k_end]^T. Must be called by
// all 256 threads; ends with the LDS tiles free for reuse.
template <class ALoader, class BLoader>
CT_DEVICE void gemm_tile(ALoader& A, BLoader& B, int k_begin, int k_end, lds_addr smem,
                         GemmAcc& acc) {
  constexpr int BK = kGemmBK, kTile = GemmSmem::kTileBytes, kStage = GemmSmem::kStageBytes;
  constexpr int kRing = GemmSmem::kStages * kStage;
  constexpr int kLoadsPerStep = ALoader::NCH + BLoader::NCH;  // 8 per thread
  static_assert(kLoadsPerStep == 8, "wait_vmcnt assumes 8 copies per thread per step");
  const int w = threadIdx.x >> 6;
  const int wm = (w >> 1) * 128, wn = (w & 1) * 128;
  if (k_begin >= k_end) return;
  const typename ALoader::FragOffsets afo(smem);
  const typename BLoader::FragOffsets bfo(smem);
  const int steps = (k_end - k_begin + BK - 1) / BK;

  if (A.fast && B.fast) {
    dma_wait_all();  // nothing of ours may still be in flight when counting copies below
    for (int i = 0; i < 3 && i < steps; ++i) {
      A.dma(k_begin + i * BK, smem + i * kStage);
      B.dma(k_begin + i * BK, smem + i * kStage + kTile);
    }
    wait_vmcnt((min(steps, 3) - 1) * kLoadsPerStep);
    workgroup_barrier();
    if constexpr (std::is_same<ALoader, McLoader>::value && std::is_same<BLoader, KcLoader>::value) {
      if (steps % 4 == 0 && !A.row_index) {  // uniform
        gemm_loop_scheduled(A, B, k_begin, steps, smem, afo, bfo, wm, wn, acc);
        return;
      }
    }
    GemmFrags f0, f1;
    load_frags<ALoader, BLoader>(f0, 0, afo, bfo, 0, wm, wn);
    int stage = 0;
    for (int k = 0; k < steps; ++k) {
      // The copies of step k+3 go into the stage read during step k-1 (free since the
      // last barrier); the B half is issued between the MFMAs so that a shorter burst of
      // copies stalls the matrix pipe.
      const int dst = (stage + 3 * kStage) & (kRing - 1);
      const int k_next = k_begin + (k + 3) * BK;
      const bool more = k + 3 < steps;
      load_frags<ALoader, BLoader>(f1, stage, afo, bfo, 1, wm, wn);
      mfma_rows<0, 1>(f0, acc);
      if (more) A.dma(k_next, smem + dst);
      mfma_rows<1, 3>(f0, acc);
      if (more) B.dma(k_next, smem + dst + kTile);
      mfma_rows<3, 4>(f0, acc);
      // step k+1 must have landed: at most the copies of steps k+2, k+3 may be in flight
      wait_vmcnt(min(max(steps - k - 2, 0), 2) * kLoadsPerStep);
      wait_lds();  // our reads of this stage are done before anyone recycles it
      workgroup_barrier();
      stage = (stage + kStage) & (kRing - 1);
      if (k + 1 < steps) load_frags<ALoader, BLoader>(f0, stage, afo, bfo, 0, wm, wn);
      mfma_rows<0, 4>(f1, acc);
    }
    wait_lds();
    __syncthreads();
    return;
  }

  A.fetch(k_begin);
  B.fetch(k_begin);
  A.commit(smem);
  B.commit(smem + kTile);
  __syncthreads();
  int cur = 0, nxt = kStage;
  for (int k0 = k_begin; k0 < k_end; k0 += BK) {
    const bool more = k0 + BK < k_end;
    if (more) {
      A.fetch(k0 + BK);
      B.fetch(k0 + BK);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      GemmFrags f;
      load_frags<ALoader, BLoader>(f, cur, afo, bfo, ks, wm, wn);
      mfma_block(f, acc);
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
