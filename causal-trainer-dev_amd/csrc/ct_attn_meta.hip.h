// Tile-bounds buffer shared by the attention kernels.
//
// The sequence is cut into 32-position blocks ("row blocks"). For each block
// the buffer holds kMetaW int32:
//   [0] min_nz   smallest nonzero segment id in the block, 0 if none
//   [1] max_id   largest id among nonzero ids, 0 if none
//   [2] uniform  the id shared by all 32 positions if they are equal and
//                nonzero, else 0
//   [3] end_min  min visible end over positions with id != 0 (INT_MAX if none)
//   [4] end_max  max visible end over positions with id != 0 (-1 if none)
//   [5] kv_first first 64-key tile this block (as queries) has to visit
//   [6] kv_last  last such tile (INT_MAX / -1 pair when there is none)
//   [7] q_first  first 32-row query block that has to visit this block (as keys)
//   [8] q_last   last such block
//   [9] ds_off   number of (key block, visiting query block) pairs of the key blocks before this
//                one in the same batch row, i.e. the exclusive prefix sum of
//                max(0, q_last - q_first + 1): where the dS blocks of this key block start in
//                the backward's dS region (saturates at INT_MAX)
// [0], [1] and the "has to visit" predicate follow the reference's block
// summaries and skip test (src/kernels/efficient_attention.py:313-323,
// :377-412): two blocks interact iff both hold a nonzero id, their id ranges
// overlap, and the key block starts at or before the query block's largest
// visible end.
//
// After the [batch][nrb][kMetaW] table come four work-sorted schedules per
// batch row, each a permutation that lists tiles by decreasing amount of
// work, so that the hardware's in-order workgroup dispatch places the longest
// tiles first:
//   query tiles of 1, 2 and 4 row blocks (by number of key tiles to visit),
//   128-key tiles (by number of query blocks to visit),
//   query tiles of 8 row blocks (the last one may be partial).
#pragma once

#include <limits.h>

#include "ct_common.hip.h"

namespace ct {

constexpr int kMetaW = 12;
enum MetaSlot {
  kMinNz = 0,
  kMaxId = 1,
  kUniform = 2,
  kEndMin = 3,
  kEndMax = 4,
  kKvFirst = 5,
  kKvLast = 6,
  kQFirst = 7,
  kQLast = 8,
  kDsOff = 9,
};

// ints of schedule data per batch row (nrb + nrb/2 + nrb/4 + nrb/4, then ceil(nrb/8) <= nrb/4)
__host__ __device__ inline int schedule_ints(int nrb) { return 2 * nrb + nrb / 4; }
// offset of the schedule for query tiles of pb row blocks (pb = 1, 2, 4, 8) inside a row's
// schedules; a row has ceil(nrb / pb) tiles of pb blocks
__host__ __device__ inline int query_schedule_offset(int nrb, int pb) {
  return pb == 1 ? 0 : (pb == 2 ? nrb : (pb == 4 ? nrb + nrb / 2 : 2 * nrb));
}
__host__ __device__ inline int key_schedule_offset(int nrb) { return nrb + nrb / 2 + nrb / 4; }

// ---------------------------------------------------------------------------
// Static work bins (after the schedules of the last batch row).
//
// A kernel that keeps one workgroup per compute unit cannot rely on the
// hardware dispatcher for balance: workgroups are dealt to the 8 XCDs round
// robin and in order, so one full XCD stalls the launch of every later
// workgroup. Instead the query tiles of the whole batch (items (batch row,
// tile), for tiles of 2, 4 and 8 row blocks) are packed once, by decreasing
// work onto the least loaded bin, into kBins bins of near equal work; a
// workgroup walks one bin for one (head slice, KV head) group. With 8 groups
// per 8 XCDs that is exactly one workgroup per compute unit, no atomics and a
// fixed assignment.
// Layout per tile size: kBins + 1 offsets, then the items (batch row * tiles
// per row + tile) bin after bin, heaviest first inside a bin.
// ---------------------------------------------------------------------------
constexpr int kBins = 32;
__host__ __device__ inline int bin_tiles_per_row(int nrb, int pb) { return (nrb + pb - 1) / pb; }
__host__ __device__ inline int bin_region_ints(int B, int nrb, int pb) {
  return kBins + 1 + B * bin_tiles_per_row(nrb, pb);
}
// offset (ints) of the bins for tiles of pb row blocks (pb = 2, 4, 8) from the start of the table
__host__ __device__ inline size_t bin_region_offset(int B, int nrb, int pb) {
  size_t off = (size_t)B * ((size_t)nrb * 12 + schedule_ints(nrb));
  if (pb >= 4) off += bin_region_ints(B, nrb, 2);
  if (pb >= 8) off += bin_region_ints(B, nrb, 4);
  return off;
}
// The metadata kernels keep their working arrays in LDS when they fit: 3 ints per row block
// of one batch row for the tile-bound kernel, 3 ints per 64-query tile of the whole batch for
// the bin packer. Larger shapes (a sequence beyond 262144 positions, or more than about 13 k
// query tiles in the batch) use a scratch region at the end of the caller's metadata buffer
// instead, so the buffer is only longer for the shapes that need it.
constexpr int kPrepareLdsRowBlocks = 8192;              // 96 KB of LDS
constexpr int kBinsLdsInts = (160 * 1024 - 1024) / 4;   // what attn_bins_kernel may take
__host__ __device__ inline size_t meta_table_ints(int B, int nrb) {
  return bin_region_offset(B, nrb, 8) + bin_region_ints(B, nrb, 8);
}
__host__ __device__ inline bool prepare_fits_lds(int nrb) { return nrb <= kPrepareLdsRowBlocks; }
__host__ __device__ inline bool bins_fit_lds(int B, int nrb) {
  return (size_t)3 * B * bin_tiles_per_row(nrb, 2) <= (size_t)kBinsLdsInts;
}
// scratch ints: [B][3 nrb] for the tile-bound kernel, then 3 regions of 3 * B * tiles(2) for the
// bin packer's three workgroups
__host__ __device__ inline size_t meta_scratch_ints(int B, int nrb) {
  size_t ints = 0;
  if (!prepare_fits_lds(nrb)) ints += (size_t)B * 3 * nrb;
  if (!bins_fit_lds(B, nrb)) ints += (size_t)3 * 3 * B * bin_tiles_per_row(nrb, 2);
  return ints;
}
__host__ __device__ inline size_t meta_total_ints(int B, int nrb) {
  return meta_table_ints(B, nrb) + meta_scratch_ints(B, nrb);
}

// ---------------------------------------------------------------------------
// dK/dV work list (backward workspace).
//
// A 128-key tile's work is the list of (query head of the group, visiting
// 32-row query block) items. Tiles at the start of a long segment carry many
// times the mean, so the list of a heavy tile is cut into up to kDkvMaxSplit
// chunks of about one compute slot's fair share (measured: finer chunks shorten the
// tail of the launch by less than their partial sums cost); every chunk is one
// workgroup, chunks are dispatched heaviest first, and the chunks of a split
// tile leave f32 partial sums that a small kernel adds up in chunk order
// (fixed order: results do not depend on timing).
// Workspace: header (entry count, chunk target), the sorted entries, lse * log2 e,
// the partial sums.
// ---------------------------------------------------------------------------
constexpr int kDkvSlots = 512;     // workgroups resident at once on the device (2 per CU)
constexpr int kDkvMinChunk = 16;   // items
constexpr int kDkvMaxSplit = 32;
constexpr int kDkvKeys = 128;      // keys per dK/dV tile

constexpr int kDqCounters = 448;  // one per (head slice, KV head) group of the dQ kernel

struct DkvLayout {
  int max_entries, max_partials;
  size_t header, entries, lse2, partials, total;
};

// Sum over tiles of the chunk count is at most tiles + total_items / target and the
// target is at least total_items * (KV heads that run side by side) / kDkvSlots.
__host__ inline DkvLayout dkv_layout(int B, int S, int Hq, int Hkv, int D, int kvh_per_pass) {
  DkvLayout L;
  const int tiles = B * (S / kDkvKeys);
  const int extra = (kDkvSlots + kvh_per_pass - 1) / kvh_per_pass + 1;
  L.max_entries = tiles + extra;
  L.max_partials = min(2 * extra, L.max_entries);
  auto up = [](size_t v) { return (v + 255) / 256 * 256; };
  L.header = 0;  // 64 ints of dK/dV list header, then kDqCounters work counters of the dQ kernel
  L.entries = (64 + kDqCounters) * sizeof(int);
  // -lse / scale, head-major [B, Hq, S] (the caller's delta scratch holds -delta the same way)
  L.lse2 = L.entries + up((size_t)L.max_entries * 2 * sizeof(int));
  L.partials = L.lse2 + up((size_t)B * S * Hq * sizeof(float));
  L.total = up(L.partials + (size_t)L.max_partials * Hkv * 2 * kDkvKeys * D * sizeof(float));
  return L;
}

// ---------------------------------------------------------------------------
// dS region (backward workspace, after the work list).
//
// The dK/dV kernel forms dS = P (dP - delta) for every (key block, visiting query block) pair
// anyway (its dK product consumes it as bf16). When the workspace has room it also stores these
// 32 x 32 bf16 blocks, and dQ = scale * dS K becomes a block-sparse product over stored blocks
// instead of a second evaluation of S and dP: 2 D flops per pair instead of 6 D, paid for with
// 2 bytes written and 2 bytes read per visited pair.
// Block (key block rb, query block qb) of query head h, batch row b sits at block index
//   ((h - first head of the pass) * B + b) * row_blocks + ds_off[rb] + qb - q_first[rb]
// (kDsBlockBytes each); row_blocks bounds the pairs of one batch row: nrb (nrb + 1) / 2 for plain
// causal masks (a key block is visited by query blocks at or after it), nrb^2 with visible ends.
// A block is stored as the dK/dV kernel's lanes hold it: two runs of 64 x 16 bytes; run t, lane
// (half, key j) holds key j's dS against the 8 query slots 16 half + 8 t + e, and slot s stands
// for query row 16 ((s >> 3) & 1) + 4 (s >> 4) + (s & 3) + 8 ((s >> 2) & 1) of the block.
// KV heads are processed in passes of kvh_per_pass heads so that the region stays bounded.
// ---------------------------------------------------------------------------
constexpr int kDsBlockBytes = 32 * 32 * 2;
constexpr size_t kDsRegionDefaultCap = (size_t)16 << 30;  // what ct_attn_bwd_workspace_bytes asks for at most
constexpr size_t kDsRegionHardCap = (size_t)64 << 30;

CT_DEVICE int ds_slot_row(int s) { return 16 * ((s >> 3) & 1) + 4 * (s >> 4) + (s & 3) + 8 * ((s >> 2) & 1); }

__host__ inline size_t ds_row_blocks(int S, bool has_end) {
  const size_t nrb = (size_t)S / 32;
  return has_end ? nrb * nrb : nrb * (nrb + 1) / 2;
}
// bytes of dS blocks of one KV head's query heads
__host__ inline size_t ds_bytes_per_kv_head(int B, int S, int Hq, int Hkv, bool has_end) {
  return (size_t)(Hq / Hkv) * B * ds_row_blocks(S, has_end) * kDsBlockBytes;
}

// Longest row for which the backward takes the stored-dS form by itself when the caller's
// workspace has room for it (measured 1-3 % faster than recomputing at 4096-token packed rows,
// 15 % slower at 32768).
constexpr int kFromDsUpToSeq = 4096;

struct BwdPlan {
  DkvLayout L;
  bool spill;         // dS goes through the region, dQ from stored blocks
  int kvh_per_pass;   // KV heads per pass (spill) or all of them
  size_t ds, ds_bytes, row_blocks, total;
};

// The plan for a workspace of `bytes` (bytes == 0: the recommended size, dS region capped at
// kDsRegionDefaultCap but never below one KV head; a KV head beyond kDsRegionHardCap, or
// allow_spill == false: no region).
__host__ inline BwdPlan bwd_plan(int B, int S, int Hq, int Hkv, int D, bool has_end, size_t bytes,
                                 bool allow_spill) {
  BwdPlan plan;
  const size_t per_kvh = ds_bytes_per_kv_head(B, S, Hq, Hkv, has_end);
  plan.row_blocks = ds_row_blocks(S, has_end);
  plan.spill = false;
  plan.kvh_per_pass = Hkv;
  plan.L = dkv_layout(B, S, Hq, Hkv, D, Hkv);
  plan.ds = plan.L.total;
  plan.ds_bytes = 0;
  plan.total = plan.L.total;
  // (block indices are 32-bit in the kernels' scalar arithmetic before the final widening)
  const bool indexable = (size_t)(Hq / Hkv) * B * plan.row_blocks < ((size_t)1 << 31);
  if (!allow_spill || per_kvh > kDsRegionHardCap || !indexable) return plan;
  for (int kpp = Hkv; kpp >= 1; --kpp) {
    const DkvLayout L = dkv_layout(B, S, Hq, Hkv, D, kpp);
    const size_t region = per_kvh * kpp;
    bool fits;
    if (bytes == 0) fits = region <= kDsRegionDefaultCap || kpp == 1;
    else fits = L.total + region <= bytes;
    if (fits && (size_t)(Hq / Hkv) * kpp * B * plan.row_blocks < ((size_t)1 << 31)) {
      plan.spill = true;
      plan.kvh_per_pass = kpp;
      plan.L = L;
      plan.ds = L.total;
      plan.ds_bytes = region;
      plan.total = L.total + region;
      return plan;
    }
  }
  return plan;
}

struct KeyTileBounds {
  int min_nz;
  int max_id;
  int uniform;
};

// The table is written by an earlier kernel and only read here. Reading it through the
// constant address space makes wave-uniform accesses scalar loads: they are counted by
// lgkmcnt, so waiting for them does not also wait for the asynchronous tile copies in
// flight (a vector load would, vmcnt completes in order).
typedef __attribute__((address_space(4))) const int* MetaPtr;
CT_DEVICE MetaPtr meta_const(const int* p) { return (MetaPtr)p; }

// Bounds of the 64-key tile `t` = row blocks 2t and 2t+1 (wave-uniform).
CT_DEVICE KeyTileBounds key_tile_bounds(const int* meta_b, int t) {
  const MetaPtr a = meta_const(meta_b + (2 * t) * kMetaW);
  const MetaPtr c = a + kMetaW;
  const int a_min = a[kMinNz], c_min = c[kMinNz];
  KeyTileBounds out;
  out.min_nz = a_min == 0 ? c_min : (c_min == 0 ? a_min : min(a_min, c_min));
  out.max_id = max(a[kMaxId], c[kMaxId]);
  out.uniform = (a[kUniform] == c[kUniform]) ? a[kUniform] : 0;
  return out;
}

// The same in two steps, for a caller that wants the loads to complete under a wait it has anyway:
// key_tile_words_request issues the scalar loads and returns at once (the compiler does not know
// that the registers are still in flight, so it neither waits nor moves the loads behind the
// caller's barrier); the caller calls key_tile_words_wait before key_tile_bounds.
struct KeyTileWords {
  i32x4 a, c;  // the first four words of the two row blocks' records
};
static_assert(kMinNz == 0 && kMaxId == 1 && kUniform == 2, "the words the requests below read");
CT_DEVICE KeyTileWords key_tile_words_request(const int* meta_b, int t) {
  const int* record = meta_b + (size_t)(2 * t) * kMetaW;
  const unsigned long long b = (unsigned long long)(uintptr_t)record;
  const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)b);
  const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
  const unsigned long long base = ((unsigned long long)hi << 32) | (unsigned long long)lo;
  KeyTileWords w;
  asm volatile("s_load_dwordx4 %0, %2, 0x0\n\ts_load_dwordx4 %1, %2, %3"
               : "=&s"(w.a), "=&s"(w.c)
               : "s"(base), "i"(kMetaW * 4));
  return w;
}
// The wait that goes with key_tile_words_request. It takes the words as operands: what is computed
// from them cannot be scheduled in front of it.
CT_DEVICE void key_tile_words_wait(KeyTileWords& w) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(w.a), "+s"(w.c));
}
CT_DEVICE KeyTileBounds key_tile_bounds(const KeyTileWords& w) {
  const int a_min = w.a[kMinNz], c_min = w.c[kMinNz];
  KeyTileBounds out;
  out.min_nz = a_min == 0 ? c_min : (c_min == 0 ? a_min : min(a_min, c_min));
  out.max_id = max(w.a[kMaxId], w.c[kMaxId]);
  out.uniform = (w.a[kUniform] == w.c[kUniform]) ? w.a[kUniform] : 0;
  return out;
}

struct QueryBlockBounds {
  int min_nz, max_id, uniform, end_min, end_max, kv_first, kv_last;
};

CT_DEVICE QueryBlockBounds query_block_bounds(const int* meta_b, int rb) {
  const MetaPtr m = meta_const(meta_b + rb * kMetaW);
  QueryBlockBounds q;
  q.min_nz = uniform(m[kMinNz]);
  q.max_id = uniform(m[kMaxId]);
  q.uniform = uniform(m[kUniform]);
  q.end_min = uniform(m[kEndMin]);
  q.end_max = uniform(m[kEndMax]);
  q.kv_first = uniform(m[kKvFirst]);
  q.kv_last = uniform(m[kKvLast]);
  return q;
}

// Does query block q have any allowed pair in a key range with bounds k that
// starts at key_start? (conservative: may say yes for a fully masked tile)
CT_DEVICE bool blocks_interact(int q_min, int q_max, int q_end_max, int k_min, int k_max,
                               int key_start) {
  return q_min != 0 && k_min != 0 && max(q_min, k_min) <= min(q_max, k_max) &&
         key_start <= q_end_max;
}

// Every (query, key) pair of the tile is allowed: one shared nonzero id and
// the last key is visible from every query of the block.
CT_DEVICE bool tile_is_interior(int q_uniform, int q_end_min, int k_uniform, int key_last) {
  return q_uniform != 0 && q_uniform == k_uniform && key_last <= q_end_min;
}

}  // namespace ct
