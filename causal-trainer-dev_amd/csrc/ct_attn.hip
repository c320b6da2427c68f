// C ABI of the attention hot path: argument validation and launches.
#include <atomic>
#include <algorithm>

#include "ct_attn_bwd_kernels.hip.h"
#include "ct_attn_dkv_wide.hip.h"
#include "ct_attn_kernels.hip.h"
#include "ct_error.h"

#include <string.h>

#include <initializer_list>

namespace ct {

// ---------------------------------------------------------------------------
// Tile bounds. One workgroup per batch row; phase 1 summarises every
// 32-position block, phase 2 turns the summaries into visit ranges.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void attn_prepare_kernel(const int* seg, const int* end, int S,
                                                            int* meta, int* sched_all,
                                                            int* global_scratch) {
  // [nrb][3]: min_nz, max_id, end_max; later schedule_ints(nrb) work counts. In LDS when the
  // row fits, else this batch row's part of the scratch region (3 * nrb ints per row).
  extern __shared__ int lds_meta_shared[];
  const int b = blockIdx.x;
  int* lds_meta = global_scratch ? global_scratch + (size_t)b * 3 * (S / 32) : lds_meta_shared;
  const int nrb = S / 32, nt = S / kKeyTile;
  const int* segb = seg + (size_t)b * S;
  const int* endb = end ? end + (size_t)b * S : nullptr;
  int* mb = meta + (size_t)b * nrb * kMetaW;
  int* sched = sched_all + (size_t)b * schedule_ints(nrb);

  for (int rb = threadIdx.x; rb < nrb; rb += blockDim.x) {
    int min_nz = INT_MAX, max_id = 0, end_min = INT_MAX, end_max = -1;
    const int first_id = segb[rb * 32];
    bool same = true;
    for (int i = 0; i < 32; ++i) {
      const int pos = rb * 32 + i;
      const int id = segb[pos];
      same &= (id == first_id);
      if (id != 0) {
        min_nz = min(min_nz, id);
        max_id = max(max_id, id);
        const int e = endb ? endb[pos] : pos;
        end_min = min(end_min, e);
        end_max = max(end_max, e);
      }
    }
    if (max_id == 0) min_nz = 0;  // reference: all-padding block -> (0, 0)
    int* m = mb + rb * kMetaW;
    m[kMinNz] = min_nz;
    m[kMaxId] = max_id;
    m[kUniform] = (same && first_id != 0) ? first_id : 0;
    m[kEndMin] = end_min;
    m[kEndMax] = end_max;
    m[9] = 0;
    m[10] = 0;
    m[11] = 0;
    lds_meta[rb * 3 + 0] = min_nz;
    lds_meta[rb * 3 + 1] = max_id;
    lds_meta[rb * 3 + 2] = end_max;
  }
  __threadfence();
  __syncthreads();

  for (int rb = threadIdx.x; rb < nrb; rb += blockDim.x) {
    const int my_min = lds_meta[rb * 3 + 0], my_max = lds_meta[rb * 3 + 1],
              my_end = lds_meta[rb * 3 + 2];
    // As queries: which 64-key tiles?
    int kv_first = INT_MAX, kv_last = -1;
    if (my_min != 0) {
      const int t_hi = min(my_end / kKeyTile, nt - 1);
      for (int t = 0; t <= t_hi; ++t) {
        const int a_min = lds_meta[(2 * t) * 3], c_min = lds_meta[(2 * t + 1) * 3];
        const int k_min = a_min == 0 ? c_min : (c_min == 0 ? a_min : min(a_min, c_min));
        const int k_max = max(lds_meta[(2 * t) * 3 + 1], lds_meta[(2 * t + 1) * 3 + 1]);
        if (blocks_interact(my_min, my_max, my_end, k_min, k_max, t * kKeyTile)) {
          kv_first = min(kv_first, t);
          kv_last = t;
        }
      }
    }
    // As keys: which 32-row query blocks?
    int q_first = INT_MAX, q_last = -1;
    if (my_min != 0) {
      for (int qb = 0; qb < nrb; ++qb) {
        if (blocks_interact(lds_meta[qb * 3], lds_meta[qb * 3 + 1], lds_meta[qb * 3 + 2], my_min,
                            my_max, rb * 32)) {
          q_first = min(q_first, qb);
          q_last = qb;
        }
      }
    }
    int* m = mb + rb * kMetaW;
    m[kKvFirst] = kv_first;
    m[kKvLast] = kv_last;
    m[kQFirst] = q_first;
    m[kQLast] = q_last;
  }
  __threadfence();  // the table and (for long rows) the scratch arrays are re-read through global memory
  __syncthreads();

  // Where the dS blocks of each key block start (kDsOff): exclusive prefix sum of the lengths of
  // the query-block ranges. Every thread sums a contiguous run of row blocks, the runs are
  // scanned across the workgroup, and each thread then walks its run again.
  {
    __shared__ long long scan_buf[1024];
    const int per = (nrb + (int)blockDim.x - 1) / (int)blockDim.x;
    const int lo = min(nrb, (int)threadIdx.x * per), hi = min(nrb, lo + per);
    auto pairs_of = [&](int rb) {
      const int* m = mb + rb * kMetaW;
      return m[kQLast] >= m[kQFirst] ? (long long)(m[kQLast] - m[kQFirst] + 1) : 0ll;
    };
    long long local = 0;
    for (int rb = lo; rb < hi; ++rb) local += pairs_of(rb);
    scan_buf[threadIdx.x] = local;
    __syncthreads();
    for (int off = 1; off < (int)blockDim.x; off <<= 1) {
      const long long below = (int)threadIdx.x >= off ? scan_buf[threadIdx.x - off] : 0ll;
      __syncthreads();
      scan_buf[threadIdx.x] += below;
      __syncthreads();
    }
    long long run = scan_buf[threadIdx.x] - local;
    for (int rb = lo; rb < hi; ++rb) {
      mb[rb * kMetaW + kDsOff] = (int)min(run, (long long)INT_MAX);
      run += pairs_of(rb);
    }
  }

  // Phase 3: amount of work per tile, for the four schedules, into LDS (the
  // summaries are no longer needed): [0, nrb) query tiles of 1 row block,
  // then tiles of 2, of 4, then 128-key tiles.
  int* work = lds_meta;
  const int off2 = nrb, off4 = nrb + nrb / 2, offk = nrb + nrb / 2 + nrb / 4;
  for (int i = threadIdx.x; i < nrb; i += blockDim.x) {
    const int* m = mb + i * kMetaW;
    work[i] = m[kKvLast] >= m[kKvFirst] ? m[kKvLast] - m[kKvFirst] + 1 : 0;
  }
  for (int pb = 2; pb <= 4; pb *= 2) {
    int* dst = work + (pb == 2 ? off2 : off4);
    for (int i = threadIdx.x; i < nrb / pb; i += blockDim.x) {
      int first = INT_MAX, last = -1;
      for (int k = 0; k < pb; ++k) {
        const int* m = mb + (i * pb + k) * kMetaW;
        first = min(first, m[kKvFirst]);
        last = max(last, m[kKvLast]);
      }
      dst[i] = last >= first ? last - first + 1 : 0;
    }
  }
  for (int i = threadIdx.x; i < nrb / 4; i += blockDim.x) {
    int first = INT_MAX, last = -1;
    for (int k = 0; k < 4; ++k) {
      const int* m = mb + (i * 4 + k) * kMetaW;
      first = min(first, m[kQFirst]);
      last = max(last, m[kQLast]);
    }
    work[offk + i] = last >= first ? last - first + 1 : 0;
  }
  const int off8 = 2 * nrb, n8 = (nrb + 7) / 8;
  for (int i = threadIdx.x; i < n8; i += blockDim.x) {
    int first = INT_MAX, last = -1;
    for (int k = 0; k < 8 && i * 8 + k < nrb; ++k) {
      const int* m = mb + (i * 8 + k) * kMetaW;
      first = min(first, m[kKvFirst]);
      last = max(last, m[kKvLast]);
    }
    work[off8 + i] = last >= first ? last - first + 1 : 0;
  }
  __threadfence();
  __syncthreads();

  // Phase 4: rank sort (descending work, ties by index) -> schedules.
  const int counts[5] = {nrb, nrb / 2, nrb / 4, nrb / 4, n8};
  const int offsets[5] = {0, off2, off4, offk, off8};
  for (int sidx = 0; sidx < 5; ++sidx) {
    const int n = counts[sidx];
    const int* wk = work + offsets[sidx];
    int* out = sched + offsets[sidx];
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const int wi = wk[i];
      int rank = 0;
      for (int k = 0; k < n; ++k) {
        const int wv = wk[k];
        rank += (wv > wi) || (wv == wi && k < i);
      }
      out[rank] = i;
    }
  }
}

// Packs the query tiles of the whole batch into kBins bins of near equal work
// (longest processing time first). One workgroup per tile size (2, 4, 8 row blocks);
// the greedy pass runs on one wavefront, lane j keeping the load of bin j.
__global__ __launch_bounds__(1024) void attn_bins_kernel(int* meta, int B, int S,
                                                         int* global_scratch) {
  // work[n], order[n], bin_of[n]: in LDS when they fit, else this workgroup's third of the
  // scratch region (3 * B * tiles(2) ints per workgroup)
  extern __shared__ int lds_bins_shared[];
  __shared__ int counts[kBins];
  const int nrb = S / 32;
  const int pb = 2 << blockIdx.x;
  const int tpr = bin_tiles_per_row(nrb, pb), n = B * tpr;
  int* lds_bins = global_scratch
                      ? global_scratch + (size_t)blockIdx.x * 3 * B * bin_tiles_per_row(nrb, 2)
                      : lds_bins_shared;
  int* work = lds_bins;
  int* order = lds_bins + n;
  int* bin_of = lds_bins + 2 * n;
  int* region = meta + bin_region_offset(B, nrb, pb);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int b = i / tpr, qt = i % tpr;
    const int* mb = meta + (size_t)b * nrb * kMetaW;
    int first = INT_MAX, last = -1;
    for (int k = 0; k < pb && qt * pb + k < nrb; ++k) {
      first = min(first, mb[(qt * pb + k) * kMetaW + kKvFirst]);
      last = max(last, mb[(qt * pb + k) * kMetaW + kKvLast]);
    }
    // a tile without keys still costs a launch of the prologue; +3 ~ prologue and store
    work[i] = (last >= first ? last - first + 1 : 0) + 3;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int wi = work[i];
    int rank = 0;
    for (int k = 0; k < n; ++k) {
      const int wv = work[k];
      rank += (wv > wi) || (wv == wi && k < i);
    }
    order[rank] = i;
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    int load = lane < kBins ? 0 : INT_MAX;
    for (int r = 0; r < n; ++r) {
      // argmin over lanes (ties to the lowest bin): reduce (load, lane) keys
      long long key = ((long long)load << 8) | lane;
      for (int off = 32; off > 0; off >>= 1) {
        const long long other = __shfl_xor(key, off, 64);
        key = other < key ? other : key;
      }
      const int target = (int)(key & 0xff);
      const int item = order[r];
      if (lane == target) {
        load += work[item];
        bin_of[r] = target;
      }
    }
  }
  __syncthreads();
  // offsets by counting, then a stable scatter in rank order (heaviest first inside a bin)
  if (threadIdx.x < kBins) {
    int count = 0;
    for (int r = 0; r < n; ++r) count += bin_of[r] == (int)threadIdx.x;
    counts[threadIdx.x] = count;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int j = 0; j < kBins; ++j) {
      region[j] = run;
      run += counts[j];
    }
    region[kBins] = run;
  }
  __syncthreads();
  if (threadIdx.x < kBins) {
    int pos = region[threadIdx.x];
    for (int r = 0; r < n; ++r)
      if (bin_of[r] == (int)threadIdx.x) region[kBins + 1 + pos++] = order[r];
  }
}

__global__ void attn_block_summary_kernel(const int* seg, const int* end, int S, int block,
                                          int nblocks, int width, int* out) {
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= nblocks) return;
  const int per_row = S / block;
  const int b = gid / per_row, blk = gid % per_row;
  const int* segb = seg + (size_t)b * S + (size_t)blk * block;
  int min_nz = INT_MAX, max_id = 0, end_max = 0;
  for (int i = 0; i < block; ++i) {
    const int id = segb[i];
    if (id != 0) {
      min_nz = min(min_nz, id);
      max_id = max(max_id, id);
    }
    if (end) end_max = max(end_max, id != 0 ? end[(size_t)b * S + (size_t)blk * block + i] : 0);
  }
  if (max_id == 0) min_nz = 0;
  out[(size_t)gid * width + 0] = min_nz;
  out[(size_t)gid * width + 1] = max_id;
  if (end) out[(size_t)gid * width + 2] = end_max;
}

static float round_to_bf16(float x) {
  uint32_t u;
  ::memcpy(&u, &x, 4);
  const uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  u &= 0xffff0000u;
  float y;
  ::memcpy(&y, &u, 4);
  return y;
}

static int validate_shape(const char* fn, int B, int S, int Hq, int Hkv, int D) {
  CT_REQUIRE(B > 0 && S > 0 && Hq > 0 && Hkv > 0, "%s: dimensions must be positive", fn);
  CT_REQUIRE(S % 128 == 0, "%s: sequence length %d has no 128-aligned tiling", fn, S);
  CT_REQUIRE(Hq % Hkv == 0,
             "%s: query head count must be divisible by the KV head count, got Hq=%d, Hkv=%d", fn,
             Hq, Hkv);
  if (D != 64 && D != 128) return fail(CT_UNSUPPORTED, "%s: head_dim must be 64 or 128, got %d", fn, D);
  // (block tables and work lists index 32-position blocks of the whole batch with 32-bit ints)
  if ((long long)B * S > (1ll << 26))
    return fail(CT_UNSUPPORTED, "%s: batch %d x sequence %d exceeds 2^26 positions", fn, B, S);
  // (the tile ranking of ct_attn_prepare is quadratic in the row blocks of one batch row: rows up to
  // 2^20 positions are what it is built and tested for)
  if (S > (1 << 20))
    return fail(CT_UNSUPPORTED, "%s: sequence %d exceeds 2^20 positions per batch row", fn, S);
  return CT_OK;
}

// Tiles move by 16-byte asynchronous copies, so every tensor base must be 16-byte aligned.
static bool aligned16(std::initializer_list<const void*> ptrs) {
  for (const void* p : ptrs)
    if (reinterpret_cast<uintptr_t>(p) & 15u) return false;
  return true;
}

// Query heads of one KV head handled by a single workgroup.
static int heads_per_group(int Hq, int Hkv) {
  const int g = Hq / Hkv;
  return g % 4 == 0 ? 4 : (g % 2 == 0 ? 2 : 1);
}

// Kernels that need more than the default 64 KB of dynamic LDS say so once per kernel and device
// (the attribute belongs to the loaded code object of that device), not on every launch.
static int ensure_lds(const char* fn, const void* kernel, size_t bytes, std::atomic<unsigned>& done) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 32) device = -1;
  if (device >= 0 && (done.load(std::memory_order_acquire) >> device & 1u)) return CT_OK;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e != hipSuccess) return fail(CT_LAUNCH_FAILED, "%s: %s", fn, hipGetErrorString(e));
  if (device >= 0) done.fetch_or(1u << device, std::memory_order_release);
  return CT_OK;
}
#define CT_ENSURE_LDS(fn, kernel, bytes)                                                  \
  do {                                                                                    \
    static std::atomic<unsigned> done_{0};                                                \
    int rc_ = ensure_lds(fn, reinterpret_cast<const void*>(kernel), (bytes), done_);      \
    if (rc_) return rc_;                                                                  \
  } while (0)

template <int D, int HS>
static int launch_fwd(hipStream_t stream, const AttnParams& p) {
  const size_t smem = VkStage<D>::kTotalBytes;
  CT_ENSURE_LDS("ct_attn_fwd", (&attn_fwd_kernel<D, HS>), smem);
  const int grid = (p.Hq / HS) * kBins;  // (head slice, KV head) groups x work bins
  LaunchScope scope1("attn_fwd_kernel", stream);
  hipLaunchKernelGGL((attn_fwd_kernel<D, HS>), dim3(grid), dim3(kFwdWaves * 64), smem, stream, p);
  return scope1.done();
}

template <int D>
static int dispatch_fwd(hipStream_t stream, const AttnParams& p) {
  switch (heads_per_group(p.Hq, p.Hkv)) {
    case 4: return launch_fwd<D, 4>(stream, p);
    case 2: return launch_fwd<D, 2>(stream, p);
    default: return launch_fwd<D, 1>(stream, p);
  }
}

// Workgroups of the persistent dQ kernels: 64 per (head slice, KV head) group, two per compute
// unit when there are 8 groups; more per group when a pass has fewer groups than that.
static int dq_grid(const AttnParams& p, int hs) {
  const int groups = ((p.Hq / p.Hkv) / hs) * p.kvh_count;
  const int members = groups >= 8 ? 2 * kBins : (2 * kBins * 8 + groups - 1) / groups;
  return groups * members;
}

template <int D, int HS>
static int launch_dq(hipStream_t stream, const AttnParams& p) {
  const size_t smem = 2 * KvStage<D>::kBytes;
  CT_ENSURE_LDS("ct_attn_bwd", (&attn_dq_kernel<D, HS>), smem);
  LaunchScope scope2("attn_dq_kernel", stream);
  hipLaunchKernelGGL((attn_dq_kernel<D, HS>), dim3(dq_grid(p, HS)), dim3(256), smem, stream, p);
  return scope2.done();
}

template <int D, int HS>
static int launch_dq_blocks(hipStream_t stream, const AttnParams& p) {
  const size_t smem = DsStage<D>::kTotalBytes;
  CT_ENSURE_LDS("ct_attn_bwd", (&attn_dq_blocks_kernel<D, HS>), smem);
  LaunchScope scope("attn_dq_blocks_kernel", stream);
  hipLaunchKernelGGL((attn_dq_blocks_kernel<D, HS>), dim3(dq_grid(p, HS)), dim3(kDqbWaves * 64), smem, stream, p);
  return scope.done();
}

// Which dK/dV kernel runs for head dimension 128 when the caller leaves the choice open: the wide
// kernel's streams pay off where runs of all-allowed steps are long, which needs long segments;
// measured 8 % faster at S = 32768 with segments up to the whole row and 3 % slower at S = 4096
// with segments of 64 to 4096 positions.
constexpr int kWideDkvFromSeq = 16384;

// One pass of the dK/dV kernel over the KV heads p.kvh_base ... (all of them unless dS is stored).
template <int D>
static int launch_dkv(hipStream_t stream, const AttnParams& p, bool wide) {
  const size_t smem = QdoStage<D>::kTotalBytes;
  const int grid = p.dkv_max_entries * p.kvh_count;  // entries beyond the list's length exit at once
  if constexpr (D == 128) {
    if (wide) {
      CT_ENSURE_LDS("ct_attn_bwd", &attn_dkv_wide_kernel, DkvWideLds::kTotalBytes);
      LaunchScope scope("attn_dkv_wide_kernel", stream);
      hipLaunchKernelGGL(attn_dkv_wide_kernel, dim3(grid), dim3(128), DkvWideLds::kTotalBytes, stream, p);
      return scope.done();
    }
  }
  LaunchScope scope3("attn_dkv_kernel", stream);
  if (p.ds) {
    CT_ENSURE_LDS("ct_attn_bwd", (&attn_dkv_kernel<D, true>), smem);
    hipLaunchKernelGGL((attn_dkv_kernel<D, true>), dim3(grid), dim3(256), smem, stream, p);
  } else {
    CT_ENSURE_LDS("ct_attn_bwd", (&attn_dkv_kernel<D, false>), smem);
    hipLaunchKernelGGL((attn_dkv_kernel<D, false>), dim3(grid), dim3(256), smem, stream, p);
  }
  return scope3.done();
}

template <int D>
static int launch_dkv_reduce(hipStream_t stream, const AttnParams& p) {
  const int grid = p.dkv_max_entries * p.Hkv;
  LaunchScope scope9("attn_dkv_reduce_kernel", stream);
  hipLaunchKernelGGL((attn_dkv_reduce_kernel<D>), dim3(grid), dim3(256), 4 * 32 * D * 2, stream, p);
  return scope9.done();
}

// The delta pass on its own: delta in row order (b, s, h).
template <int D>
static int launch_delta(hipStream_t stream, const bf16* out, const bf16* dout, float* delta, long rows) {
  // 16 workgroups per compute unit, each walking 1024-chunk tiles with a grid stride
  const long tiles = (rows * (D / 8) + 1023) / 1024;
  const dim3 grid((unsigned)(tiles < 4096 ? tiles : 4096));
  LaunchScope scope4("attn_delta_kernel", stream);
  hipLaunchKernelGGL((attn_delta_kernel<D>), grid, dim3(256), 0, stream, out, dout, delta, rows);
  return scope4.done();
}

template <int D>
static int launch_schedule(hipStream_t stream, const AttnParams& p, int kvh_side_by_side) {
  LaunchScope scope7("attn_dkv_schedule_kernel", stream);
  hipLaunchKernelGGL(attn_dkv_schedule_kernel, dim3(1), dim3(1024), 0, stream, p.meta, p.B, p.S,
                     kvh_side_by_side, p.Hq / p.Hkv, p.dkv_max_entries, p.dkv_max_partials, p.dkv_header,
                     p.dkv_entries, p.dq_counters, kDqCounters);
  return scope7.done();
}

// Recompute form: the work list; dQ per query tile (evaluates S and dP itself and computes delta
// and -lse / scale for its rows on the way); dK/dV per key tile; the sum of split chunks.
template <int D>
static int dispatch_bwd_recompute(hipStream_t stream, const AttnParams& p, bool wide, bool list_kept) {
  int rc = list_kept ? 0 : launch_schedule<D>(stream, p, p.Hkv);
  if (rc) return rc;
  switch (heads_per_group(p.Hq, p.Hkv)) {
    case 4: rc = launch_dq<D, 4>(stream, p); break;
    case 2: rc = launch_dq<D, 2>(stream, p); break;
    default: rc = launch_dq<D, 1>(stream, p); break;
  }
  if (rc) return rc;
  rc = launch_dkv<D>(stream, p, wide);
  if (rc) return rc;
  return launch_dkv_reduce<D>(stream, p);
}

// Stored-dS form: row statistics; the work list; then per pass of KV heads the dK/dV kernel, which
// leaves its dS blocks in the region, and dQ as a product over those blocks; the sum of split chunks.
template <int D>
static int dispatch_bwd_blocks(hipStream_t stream, AttnParams p, int kvh_per_pass, bool wide, bool list_kept) {
  {
    const long tiles = (long)p.B * p.Hq * (p.S / (D == 128 ? 64 : 128));
    LaunchScope scope("attn_bwd_stats_kernel", stream);
    hipLaunchKernelGGL((attn_bwd_stats_kernel<D>), dim3((unsigned)(tiles < 8192 ? tiles : 8192)), dim3(256), 0,
                       stream, p.out, p.dout, p.lse, p.delta, p.lse2, p.B, p.S, p.Hq, exponent_scale(p.scale));
    int rc = scope.done();
    if (rc) return rc;
  }
  int rc = list_kept ? 0 : launch_schedule<D>(stream, p, kvh_per_pass);
  if (rc) return rc;
  for (int base = 0; base < p.Hkv; base += kvh_per_pass) {
    p.kvh_base = base;
    p.kvh_count = min(kvh_per_pass, p.Hkv - base);
    rc = launch_dkv<D>(stream, p, wide);
    if (rc) return rc;
    switch (heads_per_group(p.Hq, p.Hkv)) {
      case 4: rc = launch_dq_blocks<D, 4>(stream, p); break;
      case 2: rc = launch_dq_blocks<D, 2>(stream, p); break;
      default: rc = launch_dq_blocks<D, 1>(stream, p); break;
    }
    if (rc) return rc;
  }
  return launch_dkv_reduce<D>(stream, p);
}

}  // namespace ct

using namespace ct;

extern "C" size_t ct_attn_meta_bytes(int32_t batch, int32_t seq) {
  if (batch <= 0 || seq <= 0) return 0;
  return meta_total_ints(batch, seq / 32) * sizeof(int32_t);
}

static bool bwd_shape_ok(int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads, int32_t head_dim) {
  return batch > 0 && seq > 0 && q_heads > 0 && kv_heads > 0 && head_dim > 0 && seq % kDkvKeys == 0 &&
         q_heads % kv_heads == 0;
}

extern "C" size_t ct_attn_bwd_workspace_bytes(int32_t batch, int32_t seq, int32_t q_heads,
                                             int32_t kv_heads, int32_t head_dim) {
  if (!bwd_shape_ok(batch, seq, q_heads, kv_heads, head_dim)) return 0;
  return bwd_plan(batch, seq, q_heads, kv_heads, head_dim, false, 0, false).total;
}

extern "C" size_t ct_attn_bwd_workspace_bytes_from_ds(int32_t batch, int32_t seq, int32_t q_heads,
                                                     int32_t kv_heads, int32_t head_dim,
                                                     int32_t has_attention_end) {
  if (!bwd_shape_ok(batch, seq, q_heads, kv_heads, head_dim)) return 0;
  const BwdPlan plan = bwd_plan(batch, seq, q_heads, kv_heads, head_dim, has_attention_end != 0, 0, true);
  return plan.spill ? plan.total : 0;
}

extern "C" int32_t ct_attn_prepare(void* stream, const int32_t* segment_ids,
                                   const int32_t* attention_end, int32_t batch, int32_t seq,
                                   int32_t* tile_meta) {
  CT_REQUIRE(segment_ids && tile_meta, "ct_attn_prepare: null pointer");
  int rc = validate_shape("ct_attn_prepare", batch, seq, 1, 1, 128);
  if (rc) return rc;
  const int nrb = seq / 32;
  // working arrays: LDS when they fit, else the scratch region after the table
  int* scratch = tile_meta + meta_table_ints(batch, nrb);
  int* prepare_scratch = nullptr;
  if (!prepare_fits_lds(nrb)) {
    prepare_scratch = scratch;
    scratch += (size_t)batch * 3 * nrb;
  }
  int* bins_scratch = bins_fit_lds(batch, nrb) ? nullptr : scratch;
  const size_t smem = prepare_scratch ? 0 : (size_t)nrb * 3 * sizeof(int);
  {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prepare_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       kPrepareLdsRowBlocks * 3 * 4);
    if (e != hipSuccess) return fail(CT_LAUNCH_FAILED, "ct_attn_prepare: %s", hipGetErrorString(e));
  }
  const int threads = nrb >= 1024 ? 1024 : ((nrb + 63) / 64) * 64;
  LaunchScope scope5("attn_prepare_kernel", (hipStream_t)stream);
  hipLaunchKernelGGL(attn_prepare_kernel, dim3(batch), dim3(threads), smem, (hipStream_t)stream,
                     segment_ids, attention_end, seq, tile_meta,
                     tile_meta + (size_t)batch * nrb * kMetaW, prepare_scratch);
  rc = scope5.done();
  if (rc) return rc;
  const size_t bins_smem = bins_scratch ? 0 : (size_t)3 * batch * bin_tiles_per_row(nrb, 2) * sizeof(int);
  {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_bins_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kBinsLdsInts * 4);
    if (e != hipSuccess) return fail(CT_LAUNCH_FAILED, "ct_attn_prepare: %s", hipGetErrorString(e));
  }
  LaunchScope scope8("attn_bins_kernel", (hipStream_t)stream);
  hipLaunchKernelGGL(attn_bins_kernel, dim3(3), dim3(1024), bins_smem, (hipStream_t)stream, tile_meta,
                     batch, seq, bins_scratch);
  return scope8.done();
}

extern "C" int32_t ct_attn_block_summary(void* stream, const int32_t* segment_ids,
                                         const int32_t* attention_end, int32_t batch, int32_t seq,
                                         int32_t block, int32_t* out) {
  CT_REQUIRE(segment_ids && out, "ct_attn_block_summary: null pointer");
  CT_REQUIRE(batch > 0 && seq > 0 && block > 0, "ct_attn_block_summary: dimensions must be positive");
  CT_REQUIRE(seq % block == 0, "ct_attn_block_summary: sequence %d not divisible by block %d", seq,
             block);
  const int nblocks = batch * (seq / block);
  LaunchScope scope6("attn_block_summary_kernel", (hipStream_t)stream);
  hipLaunchKernelGGL(attn_block_summary_kernel, dim3((nblocks + 127) / 128), dim3(128), 0,
                     (hipStream_t)stream, segment_ids, attention_end, seq, block, nblocks,
                     attention_end ? 3 : 2, out);
  return scope6.done();
}

extern "C" int32_t ct_attn_fwd(void* stream, const ct_attn_fwd_args* a) {
  CT_REQUIRE(a, "ct_attn_fwd: null args");
  CT_REQUIRE(a->q && a->k && a->v && a->segment_ids && a->tile_meta && a->out && a->lse,
             "ct_attn_fwd: null pointer");
  int rc = validate_shape("ct_attn_fwd", a->batch, a->seq, a->q_heads, a->kv_heads, a->head_dim);
  if (rc) return rc;
  CT_REQUIRE(a->scale == a->scale && a->scale - a->scale == 0.f, "ct_attn_fwd: scale must be finite");
  CT_REQUIRE(aligned16({a->q, a->k, a->v, a->segment_ids, a->attention_end, a->tile_meta, a->out, a->lse}),
             "ct_attn_fwd: every device pointer must be 16-byte aligned");
  AttnParams p = {};
  p.q = reinterpret_cast<const bf16*>(a->q);
  p.k = reinterpret_cast<const bf16*>(a->k);
  p.v = reinterpret_cast<const bf16*>(a->v);
  p.seg = a->segment_ids;
  p.end = a->attention_end;
  p.meta = a->tile_meta;
  p.sched = a->tile_meta + (size_t)a->batch * (a->seq / 32) * kMetaW;
  p.out = reinterpret_cast<bf16*>(a->out);
  p.lse = a->lse;
  p.B = a->batch;
  p.S = a->seq;
  p.Hq = a->q_heads;
  p.Hkv = a->kv_heads;
  p.scale = round_to_bf16(a->scale);
  return a->head_dim == 128 ? dispatch_fwd<128>((hipStream_t)stream, p)
                            : dispatch_fwd<64>((hipStream_t)stream, p);
}

extern "C" int32_t ct_attn_delta(void* stream, const uint16_t* out, const uint16_t* dout,
                                 float* delta, int64_t rows, int32_t head_dim) {
  CT_REQUIRE(out && dout && delta, "ct_attn_delta: null pointer");
  CT_REQUIRE(rows > 0, "ct_attn_delta: rows must be positive");
  CT_REQUIRE(aligned16({out, dout, delta}), "ct_attn_delta: every device pointer must be 16-byte aligned");
  if (head_dim != 64 && head_dim != 128)
    return fail(CT_UNSUPPORTED, "ct_attn_delta: head_dim must be 64 or 128, got %d", head_dim);
  const bf16* o = reinterpret_cast<const bf16*>(out);
  const bf16* g = reinterpret_cast<const bf16*>(dout);
  return head_dim == 128 ? launch_delta<128>((hipStream_t)stream, o, g, delta, (long)rows)
                         : launch_delta<64>((hipStream_t)stream, o, g, delta, (long)rows);
}

extern "C" int32_t ct_attn_bwd(void* stream, const ct_attn_bwd_args* a) {
  CT_REQUIRE(a, "ct_attn_bwd: null args");
  CT_REQUIRE(a->q && a->k && a->v && a->segment_ids && a->tile_meta && a->out && a->lse &&
                 a->dout && a->dq && a->dk && a->dv && a->delta && a->workspace,
             "ct_attn_bwd: null pointer");
  int rc = validate_shape("ct_attn_bwd", a->batch, a->seq, a->q_heads, a->kv_heads, a->head_dim);
  if (rc) return rc;
  CT_REQUIRE(a->scale == a->scale && a->scale - a->scale == 0.f, "ct_attn_bwd: scale must be finite");
  CT_REQUIRE(aligned16({a->q, a->k, a->v, a->segment_ids, a->attention_end, a->tile_meta, a->out, a->lse,
                        a->dout, a->dq, a->dk, a->dv, a->delta, a->workspace}),
             "ct_attn_bwd: every device pointer must be 16-byte aligned");
  AttnParams p = {};
  p.q = reinterpret_cast<const bf16*>(a->q);
  p.k = reinterpret_cast<const bf16*>(a->k);
  p.v = reinterpret_cast<const bf16*>(a->v);
  p.seg = a->segment_ids;
  p.end = a->attention_end;
  p.meta = a->tile_meta;
  p.sched = a->tile_meta + (size_t)a->batch * (a->seq / 32) * kMetaW;
  p.out = const_cast<bf16*>(reinterpret_cast<const bf16*>(a->out));
  p.lse = const_cast<float*>(a->lse);
  p.dout = reinterpret_cast<const bf16*>(a->dout);
  p.delta = a->delta;
  p.dq = reinterpret_cast<bf16*>(a->dq);
  p.dk = reinterpret_cast<bf16*>(a->dk);
  p.dv = reinterpret_cast<bf16*>(a->dv);
  p.B = a->batch;
  p.S = a->seq;
  p.Hq = a->q_heads;
  p.Hkv = a->kv_heads;
  p.scale = round_to_bf16(a->scale);
  const int kernel_choice = a->variant & 0xf, path_choice = a->variant & 0xf0;
  const bool list_kept = (a->variant & CT_ATTN_BWD_WORK_LIST_KEPT) != 0;
  CT_REQUIRE((a->variant & ~(0xff | CT_ATTN_BWD_WORK_LIST_KEPT)) == 0 && kernel_choice <= CT_ATTN_BWD_DKV_WIDE &&
                 (path_choice == 0 || path_choice == CT_ATTN_BWD_DQ_RECOMPUTE || path_choice == CT_ATTN_BWD_DQ_FROM_DS),
             "ct_attn_bwd: unknown variant 0x%x", a->variant);
  // The wide dK/dV kernel does not store dS: asking for it settles the dQ form as well.
  const bool wide_forced = kernel_choice == CT_ATTN_BWD_DKV_WIDE && a->head_dim == 128;
  CT_REQUIRE(!(wide_forced && path_choice == CT_ATTN_BWD_DQ_FROM_DS),
             "ct_attn_bwd: the wide dK/dV kernel has no stored-dS form");
  // Left to the library (no form asked for), the stored-dS form runs where it measured faster and
  // costs nothing the caller has not offered: rows of up to kFromDsUpToSeq positions, the narrow
  // dK/dV kernel, and a workspace that holds the dS blocks of all KV heads at once.
  bool allow_blocks = path_choice == CT_ATTN_BWD_DQ_FROM_DS;
  if (path_choice == 0 && !wide_forced && a->seq <= kFromDsUpToSeq) {
    const BwdPlan offered = bwd_plan(a->batch, a->seq, a->q_heads, a->kv_heads, a->head_dim,
                                     a->attention_end != nullptr, a->workspace_bytes, true);
    allow_blocks = offered.spill && offered.kvh_per_pass == a->kv_heads && a->workspace_bytes >= offered.total;
  }
  const BwdPlan plan = bwd_plan(a->batch, a->seq, a->q_heads, a->kv_heads, a->head_dim,
                                a->attention_end != nullptr, a->workspace_bytes, allow_blocks);
  if (a->workspace_bytes < plan.total)
    return fail(CT_WORKSPACE_TOO_SMALL, "ct_attn_bwd: workspace %zu < %zu bytes", a->workspace_bytes,
                plan.total);
  if (path_choice == CT_ATTN_BWD_DQ_FROM_DS && !plan.spill)
    return fail(CT_WORKSPACE_TOO_SMALL,
                "ct_attn_bwd: the stored-dS form needs %zu bytes of workspace for one KV head, got %zu",
                plan.L.total + ds_bytes_per_kv_head(a->batch, a->seq, a->q_heads, a->kv_heads,
                                                    a->attention_end != nullptr),
                a->workspace_bytes);
  const DkvLayout& L = plan.L;
  char* ws = static_cast<char*>(a->workspace);
  p.dkv_header = reinterpret_cast<int*>(ws + L.header);
  p.dq_counters = p.dkv_header + 64;
  p.dkv_entries = reinterpret_cast<int2*>(ws + L.entries);
  p.dkv_partials = reinterpret_cast<float*>(ws + L.partials);
  p.lse2 = reinterpret_cast<float*>(ws + L.lse2);
  p.dkv_max_entries = L.max_entries;
  p.dkv_max_partials = L.max_partials;
  p.kvh_base = 0;
  p.kvh_count = a->kv_heads;
  hipStream_t s = (hipStream_t)stream;
  if (plan.spill) {
    p.ds = ws + plan.ds;
    p.ds_row_blocks = plan.row_blocks;
    return a->head_dim == 128 ? dispatch_bwd_blocks<128>(s, p, plan.kvh_per_pass, false, list_kept)
                              : dispatch_bwd_blocks<64>(s, p, plan.kvh_per_pass, false, list_kept);
  }
  const bool wide = a->head_dim == 128 &&
                    (wide_forced || (kernel_choice == 0 && a->seq >= kWideDkvFromSeq));
  return a->head_dim == 128 ? dispatch_bwd_recompute<128>(s, p, wide, list_kept)
                            : dispatch_bwd_recompute<64>(s, p, wide, list_kept);
}
