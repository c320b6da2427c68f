/*
 * ct_hotpath.h -- C ABI of the MI355X (gfx950) hot-path library.
 *
 * Two hot paths of the Causal Trainer reference are provided:
 *   1. segment-isolated causal attention with GQA and per-query visibility
 *      ends (forward, logsumexp residual, custom backward);
 *   2. projection-fused cut cross-entropy (forward statistics + loss,
 *      backward dHidden / dHead).
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless named host_*. All tensors are
 *     dense row-major with the last dimension contiguous, exactly the layouts
 *     the reference passes to its kernels.
 *   - `stream` is a hipStream_t passed as void*. Work is only enqueued on
 *     that stream. No entry point synchronises, allocates or frees device
 *     memory, or keeps state between calls (ct_last_error is thread local).
 *   - Return value: 0 on success, a negative ct_status otherwise; the text
 *     for the most recent failure on the calling thread is ct_last_error().
 *     Argument validation happens before anything is launched.
 *   - bf16 tensors are passed as uint16_t* (raw bfloat16 bits).
 *
 * Reference citations are relative to the reference repository root,
 * "src/" abbreviating src/causal_trainer/.
 */
#ifndef CT_HOTPATH_H_
#define CT_HOTPATH_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum ct_status {
  CT_OK = 0,
  CT_INVALID_ARGUMENT = -1, /* shape / dtype / alignment / null pointer */
  CT_UNSUPPORTED = -2,      /* valid request the kernels do not implement */
  CT_WORKSPACE_TOO_SMALL = -3,
  CT_LAUNCH_FAILED = -4     /* HIP reported an error at launch */
} ct_status;

/* Text of the last failure on this thread ("" if none). */
const char* ct_last_error(void);

/* Library ABI version (bumped on any signature change). */
int32_t ct_abi_version(void);

/*
 * Measurement hook, no counterpart in the reference. When set (per calling
 * thread), every kernel launch made by an entry point on that thread is
 * bracketed by hook(user, kernel_name, 0, stream) and hook(user, kernel_name,
 * 1, stream), called on the host, so a harness can record stream events
 * around individual kernels. NULL removes it. The hook must not call back
 * into this library.
 */
typedef void (*ct_launch_hook)(void* user, const char* kernel, int32_t phase, void* stream);
void ct_set_launch_hook(ct_launch_hook hook, void* user);

/* ------------------------------------------------------------------------
 * Attention
 * --------------------------------------------------------------------- */

/* Number of int32 per 32-position block in the per-block table that opens the
 * tile-bounds buffer; the table is followed by work-sorted tile schedules. */
#define CT_ATTN_META_WIDTH 12

/* Bytes of the tile-bounds buffer for [batch, seq] segment ids: the table, the work-sorted
 * schedules and work bins, and for very long rows a scratch tail that ct_attn_prepare works in. */
size_t ct_attn_meta_bytes(int32_t batch, int32_t seq);

/*
 * Per-tile segment / visibility bounds used by every attention kernel to
 * skip fully masked tiles and to drop the per-element mask on interior
 * tiles. Run once per forward, reuse for every layer and for the backward.
 *
 * Replaces: prepare_attention_metadata and _segment_block_summary
 * (src/kernels/efficient_attention.py:313-374) together with the skip
 * predicates _summary_should_run / _compute_tile_is_causally_reachable
 * (:377-434), evaluated ahead of time.
 *
 *   segment_ids   int32 [batch, seq]  canonical ids, 0 = padding
 *   attention_end int32 [batch, seq]  inclusive last visible key per query,
 *                                     or NULL for plain causal (end = q)
 *   tile_meta     int32 out, ct_attn_meta_bytes(batch, seq) bytes
 * seq must be a positive multiple of 128 (reference: :221-232).
 */
int32_t ct_attn_prepare(void* stream, const int32_t* segment_ids,
                        const int32_t* attention_end, int32_t batch, int32_t seq,
                        int32_t* tile_meta);

/*
 * Block summaries in the reference's own format, for callers that keep the
 * AttentionMetadata tuple: out[b, blk] = (min nonzero id, max id) and, when
 * attention_end != NULL, a third column max(end where id != 0).
 * Replaces: _segment_block_summary + the hybrid column
 * (src/kernels/efficient_attention.py:313-323, :359-365).
 *   out int32 [batch, seq / block, attention_end ? 3 : 2]
 */
int32_t ct_attn_block_summary(void* stream, const int32_t* segment_ids,
                              const int32_t* attention_end, int32_t batch, int32_t seq,
                              int32_t block, int32_t* out);

typedef struct ct_attn_fwd_args {
  const uint16_t* q;            /* bf16 [batch, seq, q_heads, head_dim] */
  const uint16_t* k;            /* bf16 [batch, seq, kv_heads, head_dim] */
  const uint16_t* v;            /* bf16 [batch, seq, kv_heads, head_dim] */
  const int32_t* segment_ids;   /* int32 [batch, seq] */
  const int32_t* attention_end; /* int32 [batch, seq] or NULL */
  const int32_t* tile_meta;     /* from ct_attn_prepare (same ids / ends) */
  uint16_t* out;                /* bf16 [batch, seq, q_heads, head_dim] */
  float* lse;                   /* f32  [batch, seq, q_heads], natural log of
                                   the scaled scores; 0.0 on rows with no
                                   visible key */
  int32_t batch, seq, q_heads, kv_heads, head_dim;
  float scale;                  /* rounded to bf16 and folded into q in bf16 */
} ct_attn_fwd_args;

/*
 * O, LSE = attention(q, k, v). Query head h reads KV head h / (q_heads /
 * kv_heads). allowed(q, key) = key <= end[q] && seg[q] == seg[key] &&
 * seg[q] != 0.
 * Replaces: _local_attention_forward / _attention_forward_kernel
 * (src/kernels/efficient_attention.py:560-770, :889-982); mask semantics of
 * _make_causal_segment_mask_precanonicalized (src/modeling/attention.py:67-97);
 * GQA head map of vanilla_attention (src/modeling/attention.py:115-118).
 * head_dim in {64, 128}; q_heads % kv_heads == 0; seq % 128 == 0.
 */
int32_t ct_attn_fwd(void* stream, const ct_attn_fwd_args* args);

/* ct_attn_bwd_args.variant: 0 leaves every choice to the library (what a trainer passes). The
 * other values pin a kernel or a form of the backward, for tests and measurements; they are
 * per call, nothing is process-wide. Low 4 bits, the dK/dV kernel at head dimension 128:
 * NARROW = two wavefronts per SIMD with 32 keys each, WIDE = one wavefront per SIMD with 64
 * keys, the (dK, dV) sums in the accumulation registers and each step one generated
 * instruction stream (left open: WIDE from 16384 positions on, NARROW below). Bits 4-7, how dQ
 * is formed: RECOMPUTE = a query-stationary kernel evaluates S and dP a second time (the
 * reference's _local_attention_dq, src/kernels/efficient_attention.py:985-1267); FROM_DS = the
 * dK/dV kernel (NARROW) stores its bf16 dS blocks in the workspace and dQ is the product of those
 * blocks with K: 14 D instead of 18 D executed flops per pair for 4 bytes of HBM traffic per
 * pair and head; measured 1-3 % faster than RECOMPUTE on packed 4096-token rows and 15 % slower
 * on 32768-token rows; needs ct_attn_bwd_workspace_bytes_from_ds. Left open (0): FROM_DS for
 * rows of at most 4096 positions if the caller's workspace holds the dS blocks of all KV heads
 * (workspace_bytes >= ct_attn_bwd_workspace_bytes_from_ds and that size is the one-pass size),
 * else RECOMPUTE: a caller chooses by the workspace it offers. All give the same results within
 * the operator's tolerances (not bitwise: summation orders differ). */
#define CT_ATTN_BWD_DKV_NARROW 1
#define CT_ATTN_BWD_DKV_WIDE 2
#define CT_ATTN_BWD_DQ_RECOMPUTE 0x10
#define CT_ATTN_BWD_DQ_FROM_DS 0x20
/* The dK/dV work list depends on the tile metadata, the head counts and the form of the backward
 * only, not on the tensors: a caller that runs the backward of several layers over one packing
 * (same tile_meta, shape, variant and workspace size) can keep the list. With this flag the call
 * does not build it: the head of `workspace` must be as the previous ct_attn_bwd call on this
 * workspace left it (every call leaves the list in place and the work counters of the dQ kernel at
 * zero). One launch and 0.01 ms less per call; anything else in the workspace may be overwritten
 * between the calls. */
#define CT_ATTN_BWD_WORK_LIST_KEPT 0x100

typedef struct ct_attn_bwd_args {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const int32_t* segment_ids;
  const int32_t* attention_end; /* or NULL */
  const int32_t* tile_meta;
  const uint16_t* out;          /* forward output (residual) */
  const float* lse;             /* forward logsumexp (residual) */
  const uint16_t* dout;         /* bf16 cotangent of out */
  uint16_t* dq;                 /* bf16 [batch, seq, q_heads, head_dim] */
  uint16_t* dk;                 /* bf16 [batch, seq, kv_heads, head_dim] */
  uint16_t* dv;                 /* bf16 [batch, seq, kv_heads, head_dim] */
  float* delta;                 /* f32 scratch, batch * seq * q_heads elements (private layout) */
  void* workspace;              /* scratch, ct_attn_bwd_workspace_bytes(); contents need not be kept */
  size_t workspace_bytes;
  int32_t batch, seq, q_heads, kv_heads, head_dim;
  float scale;
  int32_t variant;              /* 0, or CT_ATTN_BWD_* values or-ed together */
} ct_attn_bwd_args;

/* Bytes of scratch ct_attn_bwd needs: the dK/dV work list (key tiles whose list of visiting
 * query blocks is long are cut into chunks that run as separate workgroups), the f32 partial
 * sums of such chunks and the row statistics. 0 for an unsupported shape. No reference
 * counterpart (the reference's dK/dV kernel accumulates in its f32 output window,
 * src/kernels/efficient_attention.py:1545-1549). */
size_t ct_attn_bwd_workspace_bytes(int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads,
                                   int32_t head_dim);

/* Bytes of scratch for variant CT_ATTN_BWD_DQ_FROM_DS: the above plus the dS region, 2 KB per
 * (32-key block, visiting 32-row query block, query head), reserved for the worst case of the
 * mask family (causal: S/32 (S/32 + 1) / 2 blocks per batch row and head; with attention_end:
 * (S/32)^2), for all KV heads if that is at most 16 GiB, else for as many KV heads as fit (the
 * backward then runs its kernels in passes over the KV heads), never less than one KV head; 0
 * if one KV head alone exceeds 64 GiB (that form is then unavailable). Any workspace between
 * one KV head's worth and this is used for as many KV heads per pass as it holds. */
size_t ct_attn_bwd_workspace_bytes_from_ds(int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads,
                                           int32_t head_dim, int32_t has_attention_end);

/*
 * dq, dk, dv from the saved (q, k, v, out, lse) and dout. Four launches: the dK/dV work list;
 * dq per query tile, which also computes the row statistics (-delta = -rowsum(out * dout) and
 * -lse / scale) for its rows; dk/dv per key tile; the sum of the chunks of split key tiles (in
 * a fixed order, so the result is deterministic). With CT_ATTN_BWD_DQ_FROM_DS: the row
 * statistics as a pass of their own, the work list, then per pass of KV heads dk/dv (which
 * stores its dS blocks) and dq as the product of those blocks with K, and the sum.
 * Replaces: delta at src/kernels/efficient_attention.py:1735-1738,
 * _local_attention_dq (:985-1267), _local_attention_dkv (:1270-1602) and the
 * f32 -> bf16 cast at :1774.
 */
int32_t ct_attn_bwd(void* stream, const ct_attn_bwd_args* args);

/* The delta pass as a pass of its own, delta[row] = rowsum(out * dout) in row order (the
 * backward forms it in the private layout its kernels want; this entry exists so that the
 * HBM-bound pass can be measured and tested by itself). */
int32_t ct_attn_delta(void* stream, const uint16_t* out, const uint16_t* dout,
                      float* delta, int64_t rows, int32_t head_dim);

/* ------------------------------------------------------------------------
 * Preparation steps directly in front of the hot paths (they define the
 * ignored-token sets, so they are bit-exact integer kernels)
 * --------------------------------------------------------------------- */

/*
 * canonical_ids[b, s] = one-based index of the contiguous valid run that holds
 * position s, 0 where attention_mask[b, s] == 0. A run starts at a valid
 * position whose predecessor is invalid or has a different segment id;
 * segment_ids may be NULL (all zero). int32 [batch, seq] in and out.
 * Replaces: canonicalize_segment_ids (src/modeling/rotary.py:13-50).
 */
int32_t ct_canonicalize_segment_ids(void* stream, const int32_t* attention_mask,
                                    const int32_t* segment_ids, int32_t batch, int32_t seq,
                                    int32_t* canonical_ids);

typedef struct ct_shifted_targets_args {
  const int32_t* input_ids;       /* int32 [batch, seq] */
  const int32_t* attention_mask;  /* int32 [batch, seq] or NULL (all valid); valid iff == 1 */
  const int32_t* segment_ids;     /* int32 [batch, seq] or NULL */
  const int32_t* assistant_mask;  /* int32 [batch, seq] or NULL; counts where != 0 */
  const float* loss_mask;         /* f32 [batch, seq] or NULL; may be fractional */
  const int32_t* labels;          /* int32 [batch, seq] or NULL (= input_ids) */
  int32_t* targets;               /* int32 out [batch, seq - 1]; 0 where the weight is not > 0 */
  float* weights;                 /* f32 out [batch, seq - 1] */
  void* scratch;                  /* ct_shifted_targets_scratch_bytes(), only read with segment_ids */
  size_t scratch_bytes;
  int32_t batch, seq;
  int32_t ignore_index;           /* the reference default is -100 */
} ct_shifted_targets_args;

size_t ct_shifted_targets_scratch_bytes(int32_t batch, int32_t seq);

/*
 * Shifted next-token targets and their loss weights: an edge s -> s + 1 counts
 * iff both tokens are valid, the label is not ignore_index and, with segment
 * ids, both lie in the same canonical run; assistant_mask and loss_mask are
 * read at the target position. The output feeds ct_cutce_fwd unchanged.
 * Replaces: _shifted_targets_and_weights (src/training/losses.py:21-85).
 */
int32_t ct_shifted_targets_and_weights(void* stream, const ct_shifted_targets_args* args);

/* ------------------------------------------------------------------------
 * Decoder-layer neighbours of the attention operator (single HBM passes)
 * --------------------------------------------------------------------- */

/*
 * position_ids[b, s] = distance of s from the start of its run of equal
 * canonical ids, 0 where attention_mask[b, s] == 0. canonical_ids are the
 * output of ct_canonicalize_segment_ids. int32 [batch, seq] in and out.
 * Replaces: _make_position_ids_precanonicalized (src/modeling/rotary.py:82-110).
 */
int32_t ct_position_ids(void* stream, const int32_t* attention_mask, const int32_t* canonical_ids,
                        int32_t batch, int32_t seq, int32_t* position_ids);

/*
 * cosine / sine [tokens, rotary_pairs] bf16 of f32(position) * inv_freq,
 * evaluated in f32 and rounded once; no maximum-position cache.
 * Replaces: rotary_cos_sin (src/modeling/rotary.py:132-157) with dtype bf16.
 */
int32_t ct_rotary_cos_sin(void* stream, const int32_t* position_ids, const float* inv_freq,
                          int64_t tokens, int32_t rotary_pairs, uint16_t* cosine, uint16_t* sine);

enum { CT_ROPE_GPT_J = 0 /* pairs (2i, 2i+1) */, CT_ROPE_GPT_NEOX = 1 /* pairs (i, i + R/2) */ };

typedef struct ct_rotary_args {
  const uint16_t* q_in;    /* bf16 [tokens, q_heads, head_dim] */
  const uint16_t* k_in;    /* bf16 [tokens, kv_heads, head_dim] */
  uint16_t* q_out;         /* may alias q_in */
  uint16_t* k_out;         /* may alias k_in */
  const uint16_t* cosine;  /* bf16 [tokens, rotary_pairs] */
  const uint16_t* sine;
  int64_t tokens;          /* batch * seq */
  int32_t q_heads, kv_heads, head_dim;
  int32_t rotary_pairs;    /* rotary_dim / 2; channels past rotary_dim pass through */
  int32_t rope_style;      /* CT_ROPE_GPT_J (the reference default) or CT_ROPE_GPT_NEOX */
  int32_t inverse;         /* 0: rotate (forward); 1: rotate back (gradients of q, k) */
  float q_scale;           /* 1.0: none. Otherwise Q is also multiplied by bf16(q_scale) in
                              bf16, after the rotation (forward) or before it (inverse):
                              the pre-scale of src/modeling/attention.py:124, so that the
                              attention operator can then be called with scale 1 */
} ct_rotary_args;

/*
 * Partial rotary embedding of Q and K from precomputed tables. The rotation is
 * evaluated in f32 from the bf16 operands and rounded once to bf16.
 * Supported: any head_dim and any even rotary_dim <= head_dim (head_dim % 8 == 0 with
 * rotary_dim % 16 == 0 takes the 16-byte kernel and needs 16-byte aligned pointers, other
 * shapes an element-wise one).
 * Replaces: apply_rotary_cos_sin (src/modeling/rotary.py:160-204) and its
 * transpose under autodiff.
 */
int32_t ct_apply_rotary(void* stream, const ct_rotary_args* args);

/*
 * y = bf16(bf16(x * r) * scale), r = 1 / sqrt(mean(x^2) + eps) with f32
 * statistics; x, y bf16 [rows, hidden], scale bf16 [hidden]; rstd (f32 [rows])
 * may be NULL. hidden % 8 == 0.
 * Replaces: rms_norm (src/modeling/architecture.py:155-162) with compute dtype bf16.
 */
int32_t ct_rms_norm_fwd(void* stream, const uint16_t* x, const uint16_t* scale, float eps,
                        int64_t rows, int32_t hidden, uint16_t* y, float* rstd);

size_t ct_rms_norm_bwd_workspace_bytes(int32_t hidden);

/*
 * Gradients of ct_rms_norm_fwd: dx bf16 [rows, hidden], dscale f32 [hidden]
 * (summed over rows in a fixed order). hidden % 8 == 0 (512 * {1, 2, 4, 8, 16}
 * keeps the row in registers; other sizes walk it three times).
 * Replaces: the autodiff transpose of rms_norm (src/modeling/architecture.py:155-162).
 */
int32_t ct_rms_norm_bwd(void* stream, const uint16_t* x, const uint16_t* scale, const uint16_t* dy,
                        float eps, int64_t rows, int32_t hidden, uint16_t* dx, float* dscale,
                        void* workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * Sparse cross-entropy on materialised logits (the non-fused loss backend)
 * --------------------------------------------------------------------- */

enum { CT_DTYPE_BF16 = 0, CT_DTYPE_F32 = 1 };

typedef struct ct_sparse_ce_args {
  const void* logits;      /* [rows, vocab], row-major, bf16 or f32 */
  const int32_t* targets;  /* int32 [rows] */
  const float* weights;    /* f32 [rows] */
  int64_t rows;
  int32_t vocab;
  int32_t logits_dtype;    /* CT_DTYPE_BF16 or CT_DTYPE_F32 */
  int32_t ignore_index;    /* the reference passes -100 */
} ct_sparse_ce_args;

/*
 * loss[r] = weights[r] * (logsumexp(logits[r, :]) - logits[r, targets[r]]) and
 * lse[r] = logsumexp(logits[r, :]) in f32 on rows with targets[r] != ignore_index
 * and weights[r] != 0; both 0 on the other rows (which are not read). A target
 * outside [0, vocab) on a counted row contributes a target logit of 0.
 * Replaces: _replicated_loss_and_lse / _ce_stats_pallas
 * (src/kernels/cross_entropy.py:99-251, :400-420).
 */
int32_t ct_sparse_ce_fwd(void* stream, const ct_sparse_ce_args* args, float* loss, float* lse);

/*
 * dlogits[r, v] = weights[r] * dy[r] * (exp(logits[r, v] - lse[r]) - [v == targets[r]])
 * on counted rows, 0 elsewhere, in the logits dtype; dy f32 [rows].
 * Replaces: _ce_bwd_pallas (src/kernels/cross_entropy.py:254-397).
 */
int32_t ct_sparse_ce_bwd(void* stream, const ct_sparse_ce_args* args, const float* lse,
                         const float* dy, void* dlogits);

/*
 * Measurement aid, no reference counterpart: copies `bytes` (a multiple of 16,
 * both pointers 16-byte aligned) device to device with a plain kernel. Run
 * under the same hardware counters as the hot-path kernels it gives the factor
 * between what FETCH_SIZE / WRITE_SIZE report and bytes actually moved.
 */
int32_t ct_calibration_copy(void* stream, void* dst, const void* src, size_t bytes);

/* ------------------------------------------------------------------------
 * Cut cross-entropy
 * --------------------------------------------------------------------- */

typedef struct ct_cutce_shape {
  int32_t rows;   /* N = flattened token rows */
  int32_t hidden; /* d, multiple of 128 */
  int32_t vocab;  /* V > 0 */
} ct_cutce_shape;

/* Bytes of workspace ct_cutce_fwd needs. */
size_t ct_cutce_fwd_workspace_bytes(const ct_cutce_shape* shape);
/*
 * Smallest and preferred workspace for ct_cutce_bwd. With the preferred size
 * the whole vocabulary is processed as one slab; with less, the vocabulary
 * is walked in slabs and dHidden is accumulated in f32 in the workspace.
 */
size_t ct_cutce_bwd_workspace_min_bytes(const ct_cutce_shape* shape);
size_t ct_cutce_bwd_workspace_bytes(const ct_cutce_shape* shape);
/*
 * Bytes of the optional logits cache (f32, vocabulary-major, rows and
 * vocabulary padded to 256). When the caller lends one to ct_cutce_fwd and
 * hands the same buffer to ct_cutce_bwd, the backward forms its bf16 dlogits
 * from the cached f32 logits instead of repeating the projection: 3 GEMMs per
 * step instead of 4 (the reference runs 5, src/kernels/cut_cross_entropy.py:258,
 * :383). No reference counterpart: the reference never keeps logits because a
 * TPU core has 32 GB; at N = 16384, V = 128256 the cache is 8.4 GB of 288 GB and
 * only lives from the forward of the loss to its backward, the adjacent step.
 * Both calls must use the same sparse_compaction flag (the cache is indexed by
 * the compacted row order).
 */
size_t ct_cutce_logits_cache_bytes(const ct_cutce_shape* shape);

typedef struct ct_cutce_fwd_args {
  const uint16_t* hidden;  /* bf16 [rows, hidden] */
  const uint16_t* head;    /* bf16 [hidden, vocab] (vocab contiguous) */
  const int32_t* targets;  /* int32 [rows]; never used to index memory */
  const float* weights;    /* f32 [rows]; a row is ignored iff weight == 0 */
  float* nll_sum;          /* f32 [1] */
  float* weight_sum;       /* f32 [1] */
  float* lse;              /* f32 [rows]; 0.0 on ignored rows */
  void* workspace;
  size_t workspace_bytes;
  ct_cutce_shape shape;
  int32_t sparse_compaction; /* gather active rows first (same results) */
  void* logits_cache;        /* NULL, or ct_cutce_logits_cache_bytes() of device memory to fill */
  size_t logits_cache_bytes;
} ct_cutce_fwd_args;

/*
 * nll_sum = sum_i w_i (logsumexp_v(hidden_i . head[:, v]) - hidden_i . head[:, t_i]),
 * weight_sum = sum_i w_i, lse_i saved for the backward. Logits are not
 * written to memory unless the caller lends a logits cache.
 * Replaces: _cut_stats_pallas + _loss_and_lse + _compact_active_rows
 * (src/kernels/cut_cross_entropy.py:85-222, :474-521, :673-694).
 */
int32_t ct_cutce_fwd(void* stream, const ct_cutce_fwd_args* args);

/*
 * ct_cutce_fwd for callers that cannot allocate device memory (code under HIP
 * graph capture, tight evaluation or serving loops, harnesses that forbid
 * hipMalloc). No counterpart in the reference. Same arguments, results and
 * kernels as ct_cutce_fwd, but args->workspace / workspace_bytes are ignored:
 * the workspace is a static device array inside the library,
 * ct_cutce_fwd_noalloc_max_bytes() (32 MiB) per GPU, held until the process
 * ends. Shapes whose ct_cutce_fwd_workspace_bytes() exceeds that are rejected
 * with CT_UNSUPPORTED before any launch (N = 16384, V = 128256 needs 25 MB and
 * fits). The call makes no hipMalloc / hipFree and no allocating library call.
 * All calls on one GPU share the array: calls that overlap on one GPU (two
 * streams, two threads) race; serialise them. Each call initialises what it
 * reads, so nothing carries over from the previous call.
 */
size_t ct_cutce_fwd_noalloc_max_bytes(void);
int32_t ct_cutce_fwd_noalloc(void* stream, const ct_cutce_fwd_args* args);

typedef struct ct_cutce_bwd_args {
  const uint16_t* hidden;
  const uint16_t* head;
  const int32_t* targets;
  const float* weights;
  const float* lse;        /* from ct_cutce_fwd */
  const float* dy;         /* f32 [1]: cotangent of nll_sum */
  uint16_t* dhidden;       /* bf16 [rows, hidden]; exactly 0 on ignored rows */
  uint16_t* dhead;         /* bf16 [hidden, vocab], or NULL when the head is
                              frozen (then the dHead kernel is never launched) */
  void* workspace;
  size_t workspace_bytes;
  ct_cutce_shape shape;
  int32_t sparse_compaction;
  const void* logits_cache;  /* NULL (logits are recomputed), or the buffer ct_cutce_fwd filled */
  size_t logits_cache_bytes;
} ct_cutce_bwd_args;

/*
 * G = w * dy * (softmax(logits) - onehot(target)) rounded to bf16,
 * dHidden = G @ head^T, dHead = hidden^T @ G, f32 accumulation.
 * Replaces: _cut_hidden_bwd_pallas and _cut_head_bwd_pallas
 * (src/kernels/cut_cross_entropy.py:225-471) and the scatter at :638-642.
 */
int32_t ct_cutce_bwd(void* stream, const ct_cutce_bwd_args* args);

#ifdef __cplusplus
}
#endif
#endif /* CT_HOTPATH_H_ */
