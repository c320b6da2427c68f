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

#include "ct_attn_bwd_kernels.hip.h"

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

// What a stream needs to issue the copies of the next item, besides this thread's source offsets:
// all wave-uniform.
struct DkvWideCopies {
  const char* q;       // Q rows of the next item
  const char* dout;    // dO rows
  const char* stat0;   // the two statistics arrays this wavefront fetches
  const char* stat1;
};

// Everything that stays the same from step to step.
struct DkvWideFrame {
  bf16x8 kf[2][8];                          // K fragments of the two key blocks
  RowFragOffsets<16> rp;                    // row-fragment pointers
  TrFragOffsets<16, KSlots::kAccum> tp;     // transposed-fragment pointers
  lds_addr stat_ptr;                        // LDS base + 16 * (lane / 32)
  float scale_log2e;
  unsigned v_off;                           // byte offset of this wavefront's V rows
  unsigned tile_base, stat_base;            // LDS addresses of this wavefront's copy slots at stage offset 0
};

#define CT_DKVW_FRAME_OPERANDS                                                                                   \
  "v"(f.kf[0][0]), "v"(f.kf[0][1]), "v"(f.kf[0][2]), "v"(f.kf[0][3]), "v"(f.kf[0][4]), "v"(f.kf[0][5]),           \
      "v"(f.kf[0][6]), "v"(f.kf[0][7]), "v"(f.kf[1][0]), "v"(f.kf[1][1]), "v"(f.kf[1][2]), "v"(f.kf[1][3]),       \
      "v"(f.kf[1][4]), "v"(f.kf[1][5]), "v"(f.kf[1][6]), "v"(f.kf[1][7]), "v"(f.rp.ptr[0]), "v"(f.rp.ptr[1]),     \
      "v"(f.rp.ptr[2]), "v"(f.rp.ptr[3]), "v"(f.rp.ptr[4]), "v"(f.rp.ptr[5]), "v"(f.rp.ptr[6]), "v"(f.rp.ptr[7]), \
      "v"(f.tp.ptr[0][0]), "v"(f.tp.ptr[0][1]), "v"(f.tp.ptr[0][2]), "v"(f.tp.ptr[0][3]), "v"(f.tp.ptr[1][0]),    \
      "v"(f.tp.ptr[1][1]), "v"(f.tp.ptr[1][2]), "v"(f.tp.ptr[1][3]), "v"(f.stat_ptr), "s"(f.scale_log2e),         \
      "s"(f.v_off), "s"(cp.q), "s"(cp.dout), "s"(cp.stat0), "s"(cp.stat1), "s"(f.tile_base), "s"(f.stat_base)

// One step whose pairs are all allowed. STAGE: byte offset of the stage that is read; the next item
// is copied into the other one.
template <int STAGE, int OTHER>
CT_DEVICE void dkvw_fast_step(const DkvWideFrame& f, const DkvWideCopies& cp, const TileDma128& dma, unsigned lane16) {
  asm volatile(CT_DKVW_FAST_SEQUENCE
               :
               : CT_DKVW_FRAME_OPERANDS, "i"(STAGE), "i"(OTHER), "v"(dma.lane_off[0]), "v"(dma.lane_off[1]),
                 "v"(dma.lane_off[2]), "v"(dma.lane_off[3]), "v"(lane16)
               : "memory", "m0", "scc", CT_DKVW_ASM_SCRATCH, CT_DKVW_ACCUMULATORS);
}

// The same step with the starting values of the two S blocks handed over in registers (-lse /
// scale of the row where the pair is allowed, -inf where it is not).
template <int STAGE, int OTHER>
CT_DEVICE void dkvw_masked_step(const DkvWideFrame& f, const DkvWideCopies& cp, const TileDma128& dma, unsigned lane16,
                                const f32x16& s_init0, const f32x16& s_init1) {
  asm volatile(CT_DKVW_MASKED_SEQUENCE
               :
               : CT_DKVW_FRAME_OPERANDS, "v"(s_init0), "v"(s_init1), "i"(STAGE), "i"(OTHER), "v"(dma.lane_off[0]),
                 "v"(dma.lane_off[1]), "v"(dma.lane_off[2]), "v"(dma.lane_off[3]), "v"(lane16)
               : "memory", "m0", "scc", CT_DKVW_ASM_SCRATCH, CT_DKVW_ACCUMULATORS);
}

// `steps` all-allowed steps over consecutive query blocks of one head, starting on STAGE, with the
// copy waits and workgroup barriers between them inside the statement. `cp` names the rows of the
// item after the first; every step moves one query block (`q_stride` bytes of Q / dO rows, 128
// bytes of statistics) further.
template <int STAGE, int OTHER>
CT_DEVICE void dkvw_run(const DkvWideFrame& f, const DkvWideCopies& cp, const TileDma128& dma, unsigned lane16,
                        unsigned steps, unsigned q_stride) {
  unsigned o0 = dma.lane_off[0], o1 = dma.lane_off[1], o2 = dma.lane_off[2], o3 = dma.lane_off[3], l16 = lane16;
  asm volatile(CT_DKVW_RUN_SEQUENCE
               : "+s"(steps), "+v"(o0), "+v"(o1), "+v"(o2), "+v"(o3), "+v"(l16)
               : CT_DKVW_FRAME_OPERANDS, "s"(q_stride), "i"(STAGE), "i"(OTHER)
               : "memory", "m0", "scc", CT_DKVW_ASM_SCRATCH, CT_DKVW_ACCUMULATORS);
}

__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_dkv_wide_kernel(AttnParams p) {
  constexpr int D = 128;
  extern __shared__ __align__(16) char smem_raw[];
  const lds_addr lds0 = lds_address_of(smem_raw);
  constexpr int kStage = DkvWideLds::kStage;

  const int l = lane_id(), j = l & 31, half = l >> 5, w = uniform(threadIdx.x >> 6);
  const int nrb = p.S / 32;
  const int kvh = p.kvh_base + blockIdx.x % p.kvh_count, entry = blockIdx.x / p.kvh_count;
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

  // Fragment pointers and K fragments are held for the whole kernel: a lone wavefront has the registers.
  DkvWideFrame f;
  f.rp = RowFragOffsets<16>(lds0);
  f.tp = TrFragOffsets<16, KSlots::kAccum>(lds0);
  f.v_off = DkvWideLds::kVResident + w * (64 * 256);  // this wavefront's V rows
  f.stat_ptr = lds0 + 16 * half;
  f.scale_log2e = exponent_scale(p.scale) * kLog2e;
  const float masked = masked_score(p.scale);
  f.tile_base = uniform((unsigned)(uintptr_t)lds0 + w * 1024);
  f.stat_base = uniform((unsigned)(uintptr_t)lds0 + QdoStage<D>::kLse + w * 256);
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    const size_t kv_off = (((size_t)b * p.S + (rb0 + kb) * 32 + j) * p.Hkv + kvh) * D;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      f.kf[kb][ks] = as_bf16x8(load_global16(p.k + kv_off + 16 * ks + 8 * half));
      lds_store<u32x4>(f.rp.ptr[ks] + f.v_off + kb * 8192, load_global16(p.v + kv_off + 16 * ks + 8 * half));
    }
  }
  dkvw_zero_accumulators();
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) asm volatile("" : "+v"(f.kf[kb][ks]));

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
  const unsigned q_stride = (unsigned)(kQueryTile * p.Hq * D * 2);  // bytes between the rows of consecutive query blocks
  if (it < items) {
    qdo_fetch_wide(dma, p, b, head, qb, lds0);
    dma_wait_all();
  }
  __syncthreads();

  // Rows an item's copies read: Q / dO rows and the two statistics arrays of this wavefront.
  auto rows_of = [&](int h, int q_block) {
    DkvWideCopies cp;
    const size_t origin = (((size_t)b * p.S + q_block * kQueryTile) * p.Hq + h) * D;
    const size_t head_major = ((size_t)b * p.Hq + h) * p.S + q_block * kQueryTile;
    const size_t row_major = (size_t)b * p.S + q_block * kQueryTile;
    cp.q = reinterpret_cast<const char*>(p.q + origin);
    cp.dout = reinterpret_cast<const char*>(p.dout + origin);
    cp.stat0 = w == 0 ? reinterpret_cast<const char*>(p.lse2 + head_major) : reinterpret_cast<const char*>(p.seg + row_major);
    cp.stat1 = w == 0 ? reinterpret_cast<const char*>(p.delta + head_major)
                      : reinterpret_cast<const char*>(has_end ? p.end + row_major : p.seg + row_major);
    return cp;
  };
  auto all_allowed = [&](const QueryBlockBounds& q) {
    bool yes = true;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
      yes = yes && blocks_interact(q.min_nz, q.max_id, q.end_max, my_min[kb], my_max[kb], (rb0 + kb) * 32) &&
            tile_is_interior(q.uniform, q.end_min, my_uni[kb], (rb0 + kb) * 32 + 31);
    return yes;
  };
  // Number of consecutive query blocks from `first` on (at most 64, not beyond q_hi) whose steps
  // are all-allowed for this wavefront: lane i looks at block first + i. The answer depends on the
  // keys and the query block only, so it is remembered for the other heads of the group.
  int run_first = -1, run_length = 0;
  auto allowed_run = [&](int first) {
    if (first == run_first) return run_length;
    const int mine = first + lane_id_here();
    bool yes = false;
    if (mine <= q_hi) {
      const int* m = meta_b + (size_t)mine * kMetaW;
      QueryBlockBounds q;
      q.min_nz = m[kMinNz];
      q.max_id = m[kMaxId];
      q.uniform = m[kUniform];
      q.end_min = m[kEndMin];
      q.end_max = m[kEndMax];
      yes = all_allowed(q);
    }
    const unsigned long long stops = ~__ballot(yes);
    run_first = first;
    run_length = stops == 0 ? 64 : uniform(__builtin_ctzll(stops));
    return run_length;
  };

  QueryBlockBounds qb_bounds = query_block_bounds(meta_b, min(qb, nrb - 1));
  auto step = [&](auto stage_tag) {
    constexpr int CUR = decltype(stage_tag)::value;
    constexpr int kThis = CUR * kStage, kOther = (CUR ^ 1) * kStage;
    const lds_addr stage = lds0 + kThis;
    const unsigned lane16 = (unsigned)lane_id_here() * 16;

    // A run of all-allowed steps within this head and chunk goes through one statement that loops
    // by itself; an even number of steps, so that the stages are back where this step expects
    // them, and the run's last block is left to the single step below (it copies whatever item
    // comes next, which need not be the next query block).
    if (all_allowed(qb_bounds)) {
      const int within = min(min(allowed_run(qb), q_hi - qb + 1), items - it);
      const int steps = (within - 1) & ~1;
      if (steps >= 2) {
        dkvw_run<kThis, kOther>(f, rows_of(head, qb + 1), dma, lane16, (unsigned)steps, q_stride);
        it += steps;
        qb += steps;
        qb_bounds = query_block_bounds(meta_b, qb);
      }
    }

    const bool more = it + 1 < items;
    int qb_next = qb + 1, head_next = head;
    if (qb_next > q_hi) {
      qb_next = q_lo;
      ++head_next;
    }
    // The streams below issue the copies of the next item themselves (behind their first MFMAs); a
    // step that has nothing to compute issues them here. Past the last item the current one is
    // fetched again, into the stage nobody reads any more.
    const DkvWideCopies cp = rows_of(more ? head_next : head, more ? qb_next : qb);
    const QueryBlockBounds q = qb_bounds;
    if (more) qb_bounds = query_block_bounds(meta_b, qb_next);
    bool visit[2], interior[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      visit[kb] = blocks_interact(q.min_nz, q.max_id, q.end_max, my_min[kb], my_max[kb], (rb0 + kb) * 32);
      interior[kb] = tile_is_interior(q.uniform, q.end_min, my_uni[kb], (rb0 + kb) * 32 + 31);
    }
    if (visit[0] && visit[1] && interior[0] && interior[1]) {
      dkvw_fast_step<kThis, kOther>(f, cp, dma, lane16);
    } else if (visit[0] || visit[1]) {
      // Some pair of the step is not allowed (or one block has nothing to do with this query
      // block): the S blocks start from the infinity that the exponent turns into -inf there.
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
            s_init[kb][4 * qd + e] = ok ? lse4[e] : masked;
          }
        }
      }
      dkvw_masked_step<kThis, kOther>(f, cp, dma, lane16, s_init[0], s_init[1]);
    } else if (more) {
      qdo_fetch_wide(dma, p, b, head_next, qb_next, lds0 + kOther);
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
  const lds_addr patch = lds0 + f.v_off;  // V rows are no longer needed
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
