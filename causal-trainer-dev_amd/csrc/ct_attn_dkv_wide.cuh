// dK / dV, wide form (head dimension 128): one wavefront per SIMD with the whole register file.
//
// A workgroup is two wavefronts; each owns 64 keys of the 128-key tile (two 32-key blocks): their K
// fragments in vector registers, their V rows in LDS, the 2 x (dK, dV) accumulators in the 256
// accumulation registers. Two workgroups share a compute unit, one wavefront per SIMD, so nothing
// else runs beside a wavefront: a step (one query block of one head) whose pairs are all allowed is
// one generated instruction stream (gen_attn_asm.py, CT_DKVW_FAST_SEQUENCE) in which the exponent /
// dS arithmetic of one key block sits between the MFMAs of the other. Steps with masked pairs take
// the 32-key sequences of the narrow kernel, block by block.
//
// Work list, split chunks, partial sums and the reduction kernel are those of attn_dkv_kernel
// (wavefront w here covers the 32-key blocks 2w and 2w + 1 of the tile).
#pragma once

#include "ct_attn_bwd_kernels.cuh"

namespace ct {

// Copy of a 32 x 128 bf16 tile into its swizzled LDS layout by 128 threads: thread t owns the
// 16-byte slots t + 128 n (n = 0..3), i.e. chunk t % 16 of rows t / 16 + 8 n. The swizzle
// depends on row bits 0..3, so a thread needs one source offset per pass.
struct TileDma128 {
  unsigned lane_off[4];
  CT_DEVICE explicit TileDma128(size_t row_stride_bytes) {
    const int t = threadIdx.x;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int row = t / 16 + 8 * n;
      lane_off[n] = (unsigned)((size_t)row * row_stride_bytes + (((t % 16) ^ swizzle<16>(row)) * 16));
    }
  }
  CT_DEVICE void issue(const char* origin, lds_addr tile) const {
    const int wave = uniform(threadIdx.x >> 6);
#pragma unroll
    for (int n = 0; n < 4; ++n) dma16_s(origin, lane_off[n], tile + (n * 128 + wave * 64) * 16);
  }
};

struct DkvWideLds {
  static constexpr int kStage = QdoStage<128>::kBytes;
  static constexpr int kVResident = 2 * kStage;          // 2 wavefronts x 64 rows x 256 bytes
  static constexpr int kTotalBytes = kVResident + 2 * 64 * 256;
};

// Q / dO rows and statistics of query block qb of head h into `stage` (see qdo_fetch): wavefront 0
// fetches lse2 and delta, wavefront 1 the segment ids and visible ends.
CT_DEVICE void qdo_fetch_wide(const TileDma128& dma, const AttnParams& p, int b, int h, int qb, lds_addr stage) {
  constexpr int D = 128;
  const size_t origin = (((size_t)b * p.S + qb * kQueryTile) * p.Hq + h) * D;
  dma.issue(reinterpret_cast<const char*>(p.q + origin), stage + QdoStage<D>::kQ);
  dma.issue(reinterpret_cast<const char*>(p.dout + origin), stage + QdoStage<D>::kDo);
  const int wave = uniform(threadIdx.x >> 6);
  const size_t head_major = ((size_t)b * p.Hq + h) * p.S + qb * kQueryTile;
  const size_t row_major = (size_t)b * p.S + qb * kQueryTile;
  const unsigned lane = (unsigned)lane_id_here();  // (not kept in a register across the caller's loop)
  const char* first = wave == 0 ? reinterpret_cast<const char*>(p.lse2 + head_major)
                                : reinterpret_cast<const char*>(p.seg + row_major);
  const char* second = wave == 0 ? reinterpret_cast<const char*>(p.delta + head_major)
                                 : reinterpret_cast<const char*>(p.end + row_major);
  const lds_addr dst = stage + QdoStage<D>::kLse + wave * (2 * kQueryTile * 4);
  if (lane < 8) dma16_s(first, lane * 16, dst);
  if ((wave == 0 || p.end != nullptr) && lane < 8) dma16_s(second, lane * 16, dst + kQueryTile * 4);
}

// The (dK, dV) sums of a wavefront's 64 keys fill the 256 accumulation registers. They are named
// inside the assembly statements only (accumulator i = a[16 i : 16 i + 15], see gen_attn_asm.py:
// w_acc) and never handed to the compiler, which would otherwise move them between statements;
// every statement that touches them lists all of them as clobbered, and the compiler keeps nothing
// of its own there (checked on the generated code: no accumulation-register instruction outside
// these statements).
CT_DEVICE void dkvw_zero_accumulators() { asm volatile(CT_DKVW_ZERO : : : CT_DKVW_ACCUMULATORS); }

template <int INDEX>
CT_DEVICE f32x16 dkvw_read_accumulator() {
  float v[16];
  asm volatile(CT_DKVW_READ
               : "=v"(v[0]), "=v"(v[1]), "=v"(v[2]), "=v"(v[3]), "=v"(v[4]), "=v"(v[5]), "=v"(v[6]), "=v"(v[7]),
                 "=v"(v[8]), "=v"(v[9]), "=v"(v[10]), "=v"(v[11]), "=v"(v[12]), "=v"(v[13]), "=v"(v[14]), "=v"(v[15])
               : "i"(16 * INDEX));
  f32x16 out;
#pragma unroll
  for (int e = 0; e < 16; ++e) out[e] = v[e];
  return out;
}

// What the stream needs to issue the copies of the next item (all scalar except the lane offsets).
struct DkvWideCopies {
  const char* q;       // Q rows of the next item
  const char* dout;    // dO rows
  const char* stat0;   // the two statistics arrays this wavefront fetches
  const char* stat1;
  unsigned tile_dst;   // LDS address of this wavefront's first slot of the other stage's Q tile
  unsigned stat_dst;   // LDS address of its first statistics array in the other stage
};

#define CT_DKVW_COPY_OPERANDS                                                                          \
  "v"(dma.lane_off[0]), "v"(dma.lane_off[1]), "v"(dma.lane_off[2]), "v"(dma.lane_off[3]), "s"(cp.q),    \
      "s"(cp.dout), "s"(cp.stat0), "s"(cp.stat1), "s"(cp.tile_dst), "s"(cp.stat_dst), "v"(lane16)

template <int STAGE_OFF>
CT_DEVICE void dkvw_fast_step(const bf16x8 (*kf)[8], const RowFragOffsets<16>& rp,
                              const TrFragOffsets<16, KSlots::kAccum>& tp, lds_addr stat_ptr, float scale_log2e,
                              unsigned v_off, const TileDma128& dma, const DkvWideCopies& cp, unsigned lane16) {
  asm volatile(CT_DKVW_FAST_SEQUENCE
               :
               : "v"(kf[0][0]), "v"(kf[0][1]), "v"(kf[0][2]), "v"(kf[0][3]), "v"(kf[0][4]), "v"(kf[0][5]),
                 "v"(kf[0][6]), "v"(kf[0][7]), "v"(kf[1][0]), "v"(kf[1][1]), "v"(kf[1][2]), "v"(kf[1][3]),
                 "v"(kf[1][4]), "v"(kf[1][5]), "v"(kf[1][6]), "v"(kf[1][7]),
                 "v"(rp.ptr[0]), "v"(rp.ptr[1]), "v"(rp.ptr[2]), "v"(rp.ptr[3]), "v"(rp.ptr[4]), "v"(rp.ptr[5]),
                 "v"(rp.ptr[6]), "v"(rp.ptr[7]),
                 "v"(tp.ptr[0][0]), "v"(tp.ptr[0][1]), "v"(tp.ptr[0][2]), "v"(tp.ptr[0][3]),
                 "v"(tp.ptr[1][0]), "v"(tp.ptr[1][1]), "v"(tp.ptr[1][2]), "v"(tp.ptr[1][3]),
                 "v"(stat_ptr), "s"(scale_log2e), "s"(v_off), "i"(STAGE_OFF), CT_DKVW_COPY_OPERANDS
               : "memory", "m0", "scc", CT_DKVW_ASM_SCRATCH, CT_DKVW_ACCUMULATORS);
}

// The same step with the starting values of the two S blocks handed over in registers (-lse /
// scale of the row where the pair is allowed, -inf where it is not).
template <int STAGE_OFF>
CT_DEVICE void dkvw_masked_step(const bf16x8 (*kf)[8], const RowFragOffsets<16>& rp,
                                const TrFragOffsets<16, KSlots::kAccum>& tp, lds_addr stat_ptr, float scale_log2e,
                                unsigned v_off, const TileDma128& dma, const DkvWideCopies& cp, unsigned lane16,
                                const f32x16& s_init0, const f32x16& s_init1) {
  asm volatile(CT_DKVW_MASKED_SEQUENCE
               :
               : "v"(kf[0][0]), "v"(kf[0][1]), "v"(kf[0][2]), "v"(kf[0][3]), "v"(kf[0][4]), "v"(kf[0][5]),
                 "v"(kf[0][6]), "v"(kf[0][7]), "v"(kf[1][0]), "v"(kf[1][1]), "v"(kf[1][2]), "v"(kf[1][3]),
                 "v"(kf[1][4]), "v"(kf[1][5]), "v"(kf[1][6]), "v"(kf[1][7]),
                 "v"(rp.ptr[0]), "v"(rp.ptr[1]), "v"(rp.ptr[2]), "v"(rp.ptr[3]), "v"(rp.ptr[4]), "v"(rp.ptr[5]),
                 "v"(rp.ptr[6]), "v"(rp.ptr[7]),
                 "v"(tp.ptr[0][0]), "v"(tp.ptr[0][1]), "v"(tp.ptr[0][2]), "v"(tp.ptr[0][3]),
                 "v"(tp.ptr[1][0]), "v"(tp.ptr[1][1]), "v"(tp.ptr[1][2]), "v"(tp.ptr[1][3]),
                 "v"(stat_ptr), "s"(scale_log2e), "s"(v_off), "i"(STAGE_OFF), CT_DKVW_COPY_OPERANDS, "v"(s_init0),
                 "v"(s_init1)
               : "memory", "m0", "scc", CT_DKVW_ASM_SCRATCH, CT_DKVW_ACCUMULATORS);
}

__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_dkv_wide_kernel(AttnParams p) {
  constexpr int D = 128;
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr lds0 = lds_address_of(smem_raw);
  constexpr int kStage = DkvWideLds::kStage;

  const int l = lane_id(), j = l & 31, half = l >> 5, w = uniform(threadIdx.x >> 6);
  const int nrb = p.S / 32;
  const int kvh = blockIdx.x % p.Hkv, entry = blockIdx.x / p.Hkv;
  if (entry >= uniform(p.dkv_header[0])) return;
  const int2 work_entry = p.dkv_entries[entry];
  const int tile = uniform(work_entry.x), packed = uniform(work_entry.y);
  const int chunk = packed & 255, nsplit = (packed >> 8) & 255, slot0 = (unsigned)packed >> 16;
  const int b = tile / (nrb / 4), kt = tile % (nrb / 4);
  const int g = p.Hq / p.Hkv;
  const int* meta_b = p.meta + (size_t)b * nrb * kMetaW;

  int q_lo = INT_MAX, q_hi = -1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const MetaPtr m = meta_const(meta_b + (kt * 4 + i) * kMetaW);
    q_lo = min(q_lo, uniform(m[kQFirst]));
    q_hi = max(q_hi, uniform(m[kQLast]));
  }
  // this wavefront's two 32-key blocks
  const int rb0 = kt * 4 + 2 * w;
  int my_min[2], my_max[2], my_uni[2], seg_k[2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    my_min[kb] = uniform(meta_const(meta_b)[(rb0 + kb) * kMetaW + kMinNz]);
    my_max[kb] = uniform(meta_const(meta_b)[(rb0 + kb) * kMetaW + kMaxId]);
    my_uni[kb] = uniform(meta_const(meta_b)[(rb0 + kb) * kMetaW + kUniform]);
    seg_k[kb] = p.seg[(size_t)b * p.S + (rb0 + kb) * 32 + j];
  }
  const bool has_end = p.end != nullptr;
  const size_t kv_row_stride = (size_t)p.Hkv * D;

  // pointers of the row fragments and transposed fragments (held for the whole kernel: a lone
  // wavefront has the registers)
  const RowFragOffsets<16> rp(lds0);
  const TrFragOffsets<16, KSlots::kAccum> tp(lds0);
  const unsigned v_off = DkvWideLds::kVResident + w * (64 * 256);  // this wavefront's V rows
  const lds_addr stat_ptr = lds0 + 16 * half;

  bf16x8 kf[2][8];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    const size_t kv_off = (((size_t)b * p.S + (rb0 + kb) * 32 + j) * p.Hkv + kvh) * D;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      kf[kb][ks] = as_bf16x8(load_global16(p.k + kv_off + 16 * ks + 8 * half));
      lds_store<u32x4>(rp.ptr[ks] + v_off + kb * 8192, load_global16(p.v + kv_off + 16 * ks + 8 * half));
    }
  }
  dkvw_zero_accumulators();
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) asm volatile("" : "+v"(kf[kb][ks]));

  const float scale_log2e = p.scale * kLog2e;

  const int nq = (q_lo <= q_hi) ? (q_hi - q_lo + 1) : 0;
  const int per_chunk = (nq * g + nsplit - 1) / nsplit;
  int it = chunk * per_chunk;
  const int items = min(nq * g, it + per_chunk);
  int qb = q_lo, head = kvh * g;
  if (it < items) {
    head += it / nq;
    qb += it % nq;
  }
  const TileDma128 dma((size_t)p.Hq * D * 2);
  if (it < items) {
    qdo_fetch_wide(dma, p, b, head, qb, lds0);
    dma_wait_all();
  }
  __syncthreads();

  QueryBlockBounds qb_bounds = query_block_bounds(meta_b, min(qb, nrb - 1));
  auto step = [&](auto stage_tag) {
    constexpr int CUR = decltype(stage_tag)::value;
    const lds_addr stage = lds0 + CUR * kStage;
    const bool more = it + 1 < items;
    int qb_next = qb + 1, head_next = head;
    if (qb_next > q_hi) {
      qb_next = q_lo;
      ++head_next;
    }
    // The streams below issue the copies of the next item themselves (behind their first MFMAs); a
    // step that has nothing to compute issues them here. Past the last item the current one is
    // fetched again, into the stage nobody reads any more.
    const int h_cp = more ? head_next : head, qb_cp = more ? qb_next : qb;
    DkvWideCopies cp;
    {
      const size_t origin = (((size_t)b * p.S + qb_cp * kQueryTile) * p.Hq + h_cp) * D;
      const size_t head_major = ((size_t)b * p.Hq + h_cp) * p.S + qb_cp * kQueryTile;
      const size_t row_major = (size_t)b * p.S + qb_cp * kQueryTile;
      cp.q = reinterpret_cast<const char*>(p.q + origin);
      cp.dout = reinterpret_cast<const char*>(p.dout + origin);
      cp.stat0 = w == 0 ? reinterpret_cast<const char*>(p.lse2 + head_major) : reinterpret_cast<const char*>(p.seg + row_major);
      cp.stat1 = w == 0 ? reinterpret_cast<const char*>(p.delta + head_major)
                        : reinterpret_cast<const char*>(has_end ? p.end + row_major : p.seg + row_major);
      const unsigned other = (unsigned)(uintptr_t)(lds0 + (CUR ^ 1) * kStage);
      cp.tile_dst = uniform(other + w * 1024);
      cp.stat_dst = uniform(other + QdoStage<D>::kLse + w * 256);
    }
    const unsigned lane16 = (unsigned)lane_id_here() * 16;
    const int q_min = qb_bounds.min_nz, q_max = qb_bounds.max_id, q_end_max = qb_bounds.end_max,
              q_end_min = qb_bounds.end_min, q_uni = qb_bounds.uniform;
    if (more) qb_bounds = query_block_bounds(meta_b, qb_next);
    bool visit[2], interior[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      visit[kb] = blocks_interact(q_min, q_max, q_end_max, my_min[kb], my_max[kb], (rb0 + kb) * 32);
      interior[kb] = tile_is_interior(q_uni, q_end_min, my_uni[kb], (rb0 + kb) * 32 + 31);
    }
    if (visit[0] && visit[1] && interior[0] && interior[1]) {
      dkvw_fast_step<CUR * kStage>(kf, rp, tp, stat_ptr, scale_log2e, v_off, dma, cp, lane16);
    } else if (visit[0] || visit[1]) {
      // Some pair of the step is not allowed (or one block has nothing to do with this query
      // block): the S blocks start from -inf there.
      f32x16 s_init[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const int key = (rb0 + kb) * 32 + j;
        const int seg_k_or_never = seg_k[kb] != 0 ? seg_k[kb] : -1;
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          const int r0 = 8 * qd + 4 * half;
          const f32x4 lse4 = lds_load<f32x4>(stage + QdoStage<D>::kLse + r0 * 4);
          const i32x4 seg4 = lds_load<i32x4>(stage + QdoStage<D>::kSeg + r0 * 4);
          i32x4 end4;
          if (has_end) {
            end4 = lds_load<i32x4>(stage + QdoStage<D>::kEnd + r0 * 4);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) end4[e] = qb * kQueryTile + r0 + e;
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const bool ok = visit[kb] & (interior[kb] | ((seg4[e] == seg_k_or_never) & (key <= end4[e])));
            s_init[kb][4 * qd + e] = ok ? lse4[e] : kNegInf;
          }
        }
      }
      dkvw_masked_step<CUR * kStage>(kf, rp, tp, stat_ptr, scale_log2e, v_off, dma, cp, lane16, s_init[0], s_init[1]);
    } else if (more) {
      qdo_fetch_wide(dma, p, b, head_next, qb_next, lds0 + (CUR ^ 1) * kStage);
    }
    dma_wait_all();
    __syncthreads();
    ++it;
    qb = qb_next;
    head = head_next;
  };
  while (it < items) {
    step(std::integral_constant<int, 0>{});
    if (it >= items) break;
    step(std::integral_constant<int, 1>{});
  }

  // Accumulators out of their registers, one 32-key block at a time.
  const lds_addr patch = lds0 + v_off;  // V rows are no longer needed
  auto finish = [&](auto kb_tag) {
    constexpr int kb = decltype(kb_tag)::value;
    f32x16 dvacc[4] = {dkvw_read_accumulator<4 * kb + 0>(), dkvw_read_accumulator<4 * kb + 1>(),
                       dkvw_read_accumulator<4 * kb + 2>(), dkvw_read_accumulator<4 * kb + 3>()};
    f32x16 dkacc[4] = {dkvw_read_accumulator<8 + 4 * kb + 0>(), dkvw_read_accumulator<8 + 4 * kb + 1>(),
                       dkvw_read_accumulator<8 + 4 * kb + 2>(), dkvw_read_accumulator<8 + 4 * kb + 3>()};
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int e = 0; e < 16; ++e) dkacc[db][e] *= p.scale;
    if (nsplit > 1) {
      // A chunk of a split tile leaves its sums as f32 for attn_dkv_reduce_kernel (same layout as
      // the narrow kernel: this block is its wavefront 2 w + kb).
      float* mine = p.dkv_partials + dkv_partial_offset<D>(slot0 + chunk, p.Hkv, kvh, 2 * w + kb) + l * 4;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          f32x4 a, c;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            a[e] = dkacc[db][4 * q4 + e];
            c[e] = dvacc[db][4 * q4 + e];
          }
          *reinterpret_cast<f32x4*>(mine + (db * 4 + q4) * 256) = a;
          *reinterpret_cast<f32x4*>(mine + DkvPartial<D>::kPerTensor + (db * 4 + q4) * 256) = c;
        }
    } else {
      const size_t out_off = (((size_t)b * p.S + (rb0 + kb) * 32) * p.Hkv + kvh) * D;
      store_rows<D>(dkacc, patch, p.dk + out_off, kv_row_stride);
      __builtin_amdgcn_wave_barrier();
      store_rows<D>(dvacc, patch, p.dv + out_off, kv_row_stride);
      __builtin_amdgcn_wave_barrier();
    }
  };
  finish(std::integral_constant<int, 0>{});
  finish(std::integral_constant<int, 1>{});
}

}  // namespace ct
