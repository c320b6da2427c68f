// XLA FFI handlers: a thin second entry into the C ABI of ct_hotpath.h.
//
// Built only where jaxlib's headers exist (jax.ffi.include_dir()); nothing in
// libct_hotpath.so depends on this file:
//   hipcc -O2 -fPIC -shared -std=c++17 -D__HIP_PLATFORM_AMD__ \
//         -I$(python -c "import jax.ffi; print(jax.ffi.include_dir())") \
//         -Iinclude causal-trainer-dev_amd/csrc/ct_ffi.cc \
//         -Lcausal-trainer-dev_amd -lct_hotpath -o causal-trainer-dev_amd/libct_ffi.so
// Every handler unpacks buffers, attributes and the platform stream and calls
// the C ABI; scratch memory is requested from XLA as extra results, so the
// handlers allocate nothing and are safe under command-buffer capture.
#include <hip/hip_runtime.h>

#include "ct_hotpath.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

ffi::Error status_to_error(int32_t status) {
  if (status == CT_OK) return ffi::Error::Success();
  const auto code = (status == CT_LAUNCH_FAILED) ? ffi::ErrorCode::kInternal
                                                 : ffi::ErrorCode::kInvalidArgument;
  return ffi::Error(code, ct_last_error());
}

template <typename T>
const uint16_t* bits(const T& buffer) {
  return reinterpret_cast<const uint16_t*>(buffer.untyped_data());
}
template <typename T>
uint16_t* bits_out(T& buffer) {
  return reinterpret_cast<uint16_t*>(buffer->untyped_data());
}

// segment ids / attention_end / tile bounds are int32 [B, S] (...); q is [B, S, Hq, D].
ffi::Error AttnPrepare(hipStream_t stream, ffi::Buffer<ffi::S32> segment_ids,
                       ffi::Buffer<ffi::S32> attention_end, ffi::ResultBuffer<ffi::S32> tile_meta,
                       bool has_end) {
  const auto dims = segment_ids.dimensions();
  if (dims.size() != 2) return ffi::Error::InvalidArgument("segment_ids must be [batch, sequence]");
  // ct_attn_prepare takes no buffer size: the table, its schedules and (for very long rows) the
  // scratch tail the kernels work in must all fit the result the caller asked XLA for
  if (tile_meta->size_bytes() < ct_attn_meta_bytes((int32_t)dims[0], (int32_t)dims[1]))
    return ffi::Error::InvalidArgument("tile_meta is smaller than ct_attn_meta_bytes(batch, sequence)");
  return status_to_error(ct_attn_prepare(stream, segment_ids.typed_data(),
                                         has_end ? attention_end.typed_data() : nullptr,
                                         (int32_t)dims[0], (int32_t)dims[1], tile_meta->typed_data()));
}

ffi::Error AttnFwd(hipStream_t stream, ffi::Buffer<ffi::BF16> q, ffi::Buffer<ffi::BF16> k,
                   ffi::Buffer<ffi::BF16> v, ffi::Buffer<ffi::S32> segment_ids,
                   ffi::Buffer<ffi::S32> attention_end, ffi::Buffer<ffi::S32> tile_meta,
                   ffi::ResultBuffer<ffi::BF16> out, ffi::ResultBuffer<ffi::F32> lse, float scale,
                   bool has_end) {
  const auto qd = q.dimensions();
  const auto kd = k.dimensions();
  if (qd.size() != 4 || kd.size() != 4)
    return ffi::Error::InvalidArgument("attention shapes must be [batch, sequence, heads, dim]");
  ct_attn_fwd_args a = {};
  a.q = bits(q);
  a.k = bits(k);
  a.v = bits(v);
  a.segment_ids = segment_ids.typed_data();
  a.attention_end = has_end ? attention_end.typed_data() : nullptr;
  a.tile_meta = tile_meta.typed_data();
  a.out = bits_out(out);
  a.lse = lse->typed_data();
  a.batch = (int32_t)qd[0];
  a.seq = (int32_t)qd[1];
  a.q_heads = (int32_t)qd[2];
  a.kv_heads = (int32_t)kd[2];
  a.head_dim = (int32_t)qd[3];
  a.scale = scale;
  return status_to_error(ct_attn_fwd(stream, &a));
}

ffi::Error AttnBwd(hipStream_t stream, ffi::Buffer<ffi::BF16> q, ffi::Buffer<ffi::BF16> k,
                   ffi::Buffer<ffi::BF16> v, ffi::Buffer<ffi::S32> segment_ids,
                   ffi::Buffer<ffi::S32> attention_end, ffi::Buffer<ffi::S32> tile_meta,
                   ffi::Buffer<ffi::BF16> out, ffi::Buffer<ffi::F32> lse,
                   ffi::Buffer<ffi::BF16> dout, ffi::ResultBuffer<ffi::BF16> dq,
                   ffi::ResultBuffer<ffi::BF16> dk, ffi::ResultBuffer<ffi::BF16> dv,
                   ffi::ResultBuffer<ffi::F32> delta_scratch, ffi::ResultBuffer<ffi::U8> workspace,
                   float scale, bool has_end) {
  const auto qd = q.dimensions();
  const auto kd = k.dimensions();
  if (qd.size() != 4 || kd.size() != 4)
    return ffi::Error::InvalidArgument("attention shapes must be [batch, sequence, heads, dim]");
  ct_attn_bwd_args a = {};
  a.q = bits(q);
  a.k = bits(k);
  a.v = bits(v);
  a.segment_ids = segment_ids.typed_data();
  a.attention_end = has_end ? attention_end.typed_data() : nullptr;
  a.tile_meta = tile_meta.typed_data();
  a.out = bits(out);
  a.lse = lse.typed_data();
  a.dout = bits(dout);
  a.dq = bits_out(dq);
  a.dk = bits_out(dk);
  a.dv = bits_out(dv);
  a.delta = delta_scratch->typed_data();
  a.workspace = workspace->untyped_data();
  a.workspace_bytes = workspace->size_bytes();
  a.batch = (int32_t)qd[0];
  a.seq = (int32_t)qd[1];
  a.q_heads = (int32_t)qd[2];
  a.kv_heads = (int32_t)kd[2];
  a.head_dim = (int32_t)qd[3];
  a.scale = scale;
  return status_to_error(ct_attn_bwd(stream, &a));
}

ct_cutce_shape cut_shape(const ffi::Buffer<ffi::BF16>& hidden, const ffi::Buffer<ffi::BF16>& head) {
  ct_cutce_shape s;
  s.rows = (int32_t)hidden.dimensions()[0];
  s.hidden = (int32_t)hidden.dimensions()[1];
  s.vocab = (int32_t)head.dimensions()[1];
  return s;
}

ffi::Error CutceFwd(hipStream_t stream, ffi::Buffer<ffi::BF16> hidden, ffi::Buffer<ffi::BF16> head,
                    ffi::Buffer<ffi::S32> targets, ffi::Buffer<ffi::F32> weights,
                    ffi::ResultBuffer<ffi::F32> nll_sum, ffi::ResultBuffer<ffi::F32> weight_sum,
                    ffi::ResultBuffer<ffi::F32> lse, ffi::ResultBuffer<ffi::U8> workspace,
                    ffi::ResultBuffer<ffi::U8> logits_cache, bool sparse_compaction) {
  if (hidden.dimensions().size() != 2 || head.dimensions().size() != 2)
    return ffi::Error::InvalidArgument("hidden must be [rows, hidden] and head [hidden, vocab]");
  ct_cutce_fwd_args a = {};
  a.hidden = bits(hidden);
  a.head = bits(head);
  a.targets = targets.typed_data();
  a.weights = weights.typed_data();
  a.nll_sum = nll_sum->typed_data();
  a.weight_sum = weight_sum->typed_data();
  a.lse = lse->typed_data();
  a.workspace = workspace->untyped_data();
  a.workspace_bytes = workspace->size_bytes();
  a.shape = cut_shape(hidden, head);
  a.sparse_compaction = sparse_compaction ? 1 : 0;
  // a cache result shorter than one tile means "no cache" (XLA has no optional results)
  if (logits_cache->size_bytes() >= 256 * 256 * sizeof(float)) {
    a.logits_cache = logits_cache->untyped_data();
    a.logits_cache_bytes = logits_cache->size_bytes();
  }
  return status_to_error(ct_cutce_fwd(stream, &a));
}

ffi::Error CutceBwd(hipStream_t stream, ffi::Buffer<ffi::BF16> hidden, ffi::Buffer<ffi::BF16> head,
                    ffi::Buffer<ffi::S32> targets, ffi::Buffer<ffi::F32> weights,
                    ffi::Buffer<ffi::F32> lse, ffi::Buffer<ffi::F32> dy,
                    ffi::Buffer<ffi::U8> logits_cache, ffi::ResultBuffer<ffi::BF16> dhidden, ffi::ResultBuffer<ffi::BF16> dhead,
                    ffi::ResultBuffer<ffi::U8> workspace, bool sparse_compaction,
                    bool head_trainable) {
  if (hidden.dimensions().size() != 2 || head.dimensions().size() != 2)
    return ffi::Error::InvalidArgument("hidden must be [rows, hidden] and head [hidden, vocab]");
  ct_cutce_bwd_args a = {};
  a.hidden = bits(hidden);
  a.head = bits(head);
  a.targets = targets.typed_data();
  a.weights = weights.typed_data();
  a.lse = lse.typed_data();
  a.dy = dy.typed_data();
  a.dhidden = bits_out(dhidden);
  a.dhead = head_trainable ? bits_out(dhead) : nullptr;  // frozen head: dHead never launched
  a.workspace = workspace->untyped_data();
  a.workspace_bytes = workspace->size_bytes();
  a.shape = cut_shape(hidden, head);
  a.sparse_compaction = sparse_compaction ? 1 : 0;
  if (logits_cache.size_bytes() >= 256 * 256 * sizeof(float)) {
    a.logits_cache = logits_cache.untyped_data();
    a.logits_cache_bytes = logits_cache.size_bytes();
  }
  return status_to_error(ct_cutce_bwd(stream, &a));
}

// ---- preparation steps in front of the hot paths (bit-exact integer kernels) ------------------

// An absent optional operand is passed as any int32 array of the right shape plus a false flag.
ffi::Error CanonicalizeSegmentIds(hipStream_t stream, ffi::Buffer<ffi::S32> attention_mask,
                                  ffi::Buffer<ffi::S32> segment_ids, ffi::ResultBuffer<ffi::S32> canonical,
                                  bool has_segments) {
  const auto dims = attention_mask.dimensions();
  if (dims.size() != 2) return ffi::Error::InvalidArgument("attention_mask must be [batch, sequence]");
  return status_to_error(ct_canonicalize_segment_ids(stream, attention_mask.typed_data(),
                                                     has_segments ? segment_ids.typed_data() : nullptr,
                                                     (int32_t)dims[0], (int32_t)dims[1], canonical->typed_data()));
}

ffi::Error ShiftedTargets(hipStream_t stream, ffi::Buffer<ffi::S32> input_ids, ffi::Buffer<ffi::S32> attention_mask,
                          ffi::Buffer<ffi::S32> segment_ids, ffi::Buffer<ffi::S32> assistant_mask,
                          ffi::Buffer<ffi::F32> loss_mask, ffi::Buffer<ffi::S32> labels,
                          ffi::ResultBuffer<ffi::S32> targets, ffi::ResultBuffer<ffi::F32> weights,
                          ffi::ResultBuffer<ffi::U8> scratch, bool has_mask, bool has_segments, bool has_assistant,
                          bool has_loss_mask, bool has_labels, int32_t ignore_index) {
  const auto dims = input_ids.dimensions();
  if (dims.size() != 2) return ffi::Error::InvalidArgument("input_ids must be [batch, sequence]");
  ct_shifted_targets_args a = {};
  a.input_ids = input_ids.typed_data();
  a.attention_mask = has_mask ? attention_mask.typed_data() : nullptr;
  a.segment_ids = has_segments ? segment_ids.typed_data() : nullptr;
  a.assistant_mask = has_assistant ? assistant_mask.typed_data() : nullptr;
  a.loss_mask = has_loss_mask ? loss_mask.typed_data() : nullptr;
  a.labels = has_labels ? labels.typed_data() : nullptr;
  a.targets = targets->typed_data();
  a.weights = weights->typed_data();
  a.scratch = scratch->untyped_data();
  a.scratch_bytes = scratch->size_bytes();
  a.batch = (int32_t)dims[0];
  a.seq = (int32_t)dims[1];
  a.ignore_index = ignore_index;
  return status_to_error(ct_shifted_targets_and_weights(stream, &a));
}

// ---- decoder-layer neighbours and the logits-level loss ----------------------------------

ffi::Error PositionIds(hipStream_t stream, ffi::Buffer<ffi::S32> attention_mask,
                       ffi::Buffer<ffi::S32> canonical_ids, ffi::ResultBuffer<ffi::S32> positions) {
  const auto dims = attention_mask.dimensions();
  if (dims.size() != 2) return ffi::Error::InvalidArgument("attention_mask must be [batch, sequence]");
  return status_to_error(ct_position_ids(stream, attention_mask.typed_data(), canonical_ids.typed_data(),
                                         (int32_t)dims[0], (int32_t)dims[1], positions->typed_data()));
}

ffi::Error RotaryCosSin(hipStream_t stream, ffi::Buffer<ffi::S32> positions, ffi::Buffer<ffi::F32> inv_freq,
                        ffi::ResultBuffer<ffi::BF16> cosine, ffi::ResultBuffer<ffi::BF16> sine) {
  const auto dims = positions.dimensions();
  if (dims.size() != 2) return ffi::Error::InvalidArgument("position_ids must be [batch, sequence]");
  return status_to_error(ct_rotary_cos_sin(stream, positions.typed_data(), inv_freq.typed_data(),
                                           (int64_t)dims[0] * dims[1], (int32_t)inv_freq.element_count(),
                                           bits_out(cosine), bits_out(sine)));
}

// forward (inverse = false) and the transpose used for the gradients (inverse = true)
ffi::Error ApplyRotary(hipStream_t stream, ffi::Buffer<ffi::BF16> q, ffi::Buffer<ffi::BF16> k,
                       ffi::Buffer<ffi::BF16> cosine, ffi::Buffer<ffi::BF16> sine,
                       ffi::ResultBuffer<ffi::BF16> q_out, ffi::ResultBuffer<ffi::BF16> k_out,
                       int32_t rope_style, bool inverse, float q_scale) {
  const auto qd = q.dimensions();
  const auto kd = k.dimensions();
  const auto cd = cosine.dimensions();
  if (qd.size() != 4 || kd.size() != 4 || cd.size() != 3)
    return ffi::Error::InvalidArgument("query and key must be [batch, sequence, heads, head_dim], tables [batch, sequence, pairs]");
  ct_rotary_args a = {};
  a.q_in = bits(q);
  a.k_in = bits(k);
  a.q_out = bits_out(q_out);
  a.k_out = bits_out(k_out);
  a.cosine = bits(cosine);
  a.sine = bits(sine);
  a.tokens = (int64_t)qd[0] * qd[1];
  a.q_heads = (int32_t)qd[2];
  a.kv_heads = (int32_t)kd[2];
  a.head_dim = (int32_t)qd[3];
  a.rotary_pairs = (int32_t)cd[2];
  a.rope_style = rope_style;
  a.inverse = inverse ? 1 : 0;
  a.q_scale = q_scale;
  return status_to_error(ct_apply_rotary(stream, &a));
}

ffi::Error RmsNormFwd(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::Buffer<ffi::BF16> scale,
                      ffi::ResultBuffer<ffi::BF16> y, float eps) {
  const auto dims = x.dimensions();
  if (dims.empty()) return ffi::Error::InvalidArgument("rms_norm needs at least one axis");
  const int64_t hidden = dims.back();
  return status_to_error(ct_rms_norm_fwd(stream, bits(x), bits(scale), eps,
                                         hidden ? (int64_t)x.element_count() / hidden : 0, (int32_t)hidden,
                                         bits_out(y), nullptr));
}

ffi::Error RmsNormBwd(hipStream_t stream, ffi::Buffer<ffi::BF16> x, ffi::Buffer<ffi::BF16> scale,
                      ffi::Buffer<ffi::BF16> dy, ffi::ResultBuffer<ffi::BF16> dx,
                      ffi::ResultBuffer<ffi::F32> dscale, ffi::ResultBuffer<ffi::U8> workspace, float eps) {
  const auto dims = x.dimensions();
  if (dims.empty()) return ffi::Error::InvalidArgument("rms_norm needs at least one axis");
  const int64_t hidden = dims.back();
  return status_to_error(ct_rms_norm_bwd(stream, bits(x), bits(scale), bits(dy), eps,
                                         hidden ? (int64_t)x.element_count() / hidden : 0, (int32_t)hidden,
                                         bits_out(dx), dscale->typed_data(), workspace->untyped_data(),
                                         workspace->size_bytes()));
}

ct_sparse_ce_args sparse_ce_args(const ffi::AnyBuffer& logits, const ffi::Buffer<ffi::S32>& targets,
                                 const ffi::Buffer<ffi::F32>& weights) {
  ct_sparse_ce_args a = {};
  const auto dims = logits.dimensions();
  a.logits = logits.untyped_data();
  a.targets = targets.typed_data();
  a.weights = weights.typed_data();
  a.vocab = dims.empty() ? 0 : (int32_t)dims.back();
  a.rows = a.vocab ? (int64_t)logits.element_count() / a.vocab : 0;
  a.logits_dtype = logits.element_type() == ffi::BF16 ? CT_DTYPE_BF16
                   : logits.element_type() == ffi::F32 ? CT_DTYPE_F32 : -1;
  a.ignore_index = -100;
  return a;
}

ffi::Error SparseCeFwd(hipStream_t stream, ffi::AnyBuffer logits, ffi::Buffer<ffi::S32> targets,
                       ffi::Buffer<ffi::F32> weights, ffi::ResultBuffer<ffi::F32> loss,
                       ffi::ResultBuffer<ffi::F32> lse) {
  const ct_sparse_ce_args a = sparse_ce_args(logits, targets, weights);
  return status_to_error(ct_sparse_ce_fwd(stream, &a, loss->typed_data(), lse->typed_data()));
}

ffi::Error SparseCeBwd(hipStream_t stream, ffi::AnyBuffer logits, ffi::Buffer<ffi::S32> targets,
                       ffi::Buffer<ffi::F32> weights, ffi::Buffer<ffi::F32> lse, ffi::Buffer<ffi::F32> dy,
                       ffi::Result<ffi::AnyBuffer> dlogits) {
  const ct_sparse_ce_args a = sparse_ce_args(logits, targets, weights);
  return status_to_error(ct_sparse_ce_bwd(stream, &a, lse.typed_data(), dy.typed_data(),
                                          dlogits->untyped_data()));
}

}  // namespace

#define CT_STREAM Ctx<ffi::PlatformStream<hipStream_t>>()

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_attn_prepare, AttnPrepare,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Attr<bool>("has_end"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_attn_fwd, AttnFwd,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Attr<float>("scale")
                                  .Attr<bool>("has_end"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_attn_bwd, AttnBwd,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<float>("scale")
                                  .Attr<bool>("has_end"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_cutce_fwd, CutceFwd,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<bool>("sparse_compaction"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_cutce_bwd, CutceBwd,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::U8>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<bool>("sparse_compaction")
                                  .Attr<bool>("head_trainable"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_canonicalize_segment_ids, CanonicalizeSegmentIds,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Attr<bool>("has_segments"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_shifted_targets, ShiftedTargets,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<bool>("has_mask")
                                  .Attr<bool>("has_segments")
                                  .Attr<bool>("has_assistant")
                                  .Attr<bool>("has_loss_mask")
                                  .Attr<bool>("has_labels")
                                  .Attr<int32_t>("ignore_index"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_position_ids, PositionIds,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Ret<ffi::Buffer<ffi::S32>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_rotary_cos_sin, RotaryCosSin,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_apply_rotary, ApplyRotary,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Attr<int32_t>("rope_style")
                                  .Attr<bool>("inverse")
                                  .Attr<float>("q_scale"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_rms_norm_fwd, RmsNormFwd,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Attr<float>("eps"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_rms_norm_bwd, RmsNormBwd,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Arg<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::BF16>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::U8>>()
                                  .Attr<float>("eps"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_sparse_ce_fwd, SparseCeFwd,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(ct_ffi_sparse_ce_bwd, SparseCeBwd,
                              ffi::Ffi::Bind()
                                  .CT_STREAM.Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::AnyBuffer>());
