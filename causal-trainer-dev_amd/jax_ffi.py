"""JAX binding of the hot paths through XLA FFI custom calls (needs jax + jaxlib on ROCm).

Reference-side glue with the reference's operator interfaces:

  AttentionMetadata, prepare_attention_metadata(canonical_segment_ids, *, mesh, profile,
      attention_end=None)                        src/causal_trainer/kernels/efficient_attention.py:63-74, :326-374
  efficient_attention(query, key, value, metadata, *, mesh, profile=None, scale=None,
      causal=True)                               :1807-1967 (custom VJP, residual (q, k, v, metadata, O, LSE))
  pallas_cut_linear_cross_entropy(hidden_states, lm_head_kernel, targets, weights, *, mesh,
      sparse_compaction=False, lm_head_trainable=True, local_chunk_size=0)
                                                 src/causal_trainer/kernels/cut_cross_entropy.py:524-670, :828-958
  canonicalize_segment_ids, make_position_ids, rotary_cos_sin, apply_rotary_cos_sin,
      apply_rotary_embedding                     src/causal_trainer/modeling/rotary.py:13-50, :63-234
  rms_norm(x, scale, eps, compute_dtype)         src/causal_trainer/modeling/architecture.py:155-162
  shifted_targets_and_weights (= _shifted_targets_and_weights)
                                                 src/causal_trainer/training/losses.py:21-85
  pallas_fused_sparse_cross_entropy(logits, targets, weights, *, mesh)
                                                 src/causal_trainer/kernels/cross_entropy.py:600-643

so that the call sites at src/causal_trainer/modeling/attention.py:435-444,
src/causal_trainer/modeling/architecture.py:691-696 and
src/causal_trainer/kernels/fused_cross_entropy.py:189-198 keep their arguments. What differs
from the reference: ``AttentionMetadata`` has one more field at the end, ``tile_bounds`` (the
opaque table the HIP kernels read, built by ``prepare_attention_metadata``); K/V may have any
head count that divides the query head count, head_dim may be 64 or 128; every mesh axis must
have size 1 (one GPU); cut cross-entropy computes in bfloat16 only; the backend guard asks for a
GPU instead of a TPU.

Every custom call goes through ``_call``, which checks operand, result and attribute counts
against ``HANDLERS``, the table of the handlers that csrc/ct_ffi.cc defines
(tests/test_host_and_abi.py keeps the two, and the documented list of handlers, in step).

jax is not installed in the build environment of this repository: this module has never been
executed. Importing it does not import jax; the C ABI underneath it is exercised through ctypes.
"""

from __future__ import annotations

import ctypes
import functools
import math
from pathlib import Path
from typing import Any, NamedTuple

import numpy as np

from . import _lib
from .attention_profile import (AttentionKernelProfile, _Axes, _integer, _positive, _validate_qkv_shapes,
                                default_attention_scale, resolve_attention_profile, validate_attention_profile)

_FFI_LIBRARY = Path(__file__).resolve().parent / "libct_ffi.so"
_SUPPORTED_HEAD_DIMS = (64, 128)
_HIDDEN_ALIGN = 128
# Largest f32 logits cache the cut cross-entropy VJP may keep between forward and backward.
# 0 keeps the reference's residual (hidden, head, targets, weights, lse) and nothing else.
LOGITS_CACHE_LIMIT_BYTES = 0


class Handler(NamedTuple):
    operands: int
    results: int
    attributes: tuple[str, ...]


# name -> what csrc/ct_ffi.cc binds for it (XLA_FFI_DEFINE_HANDLER_SYMBOL)
HANDLERS = {
    "ct_ffi_attn_prepare": Handler(2, 1, ("has_end",)),
    "ct_ffi_attn_fwd": Handler(6, 2, ("scale", "has_end")),
    "ct_ffi_attn_bwd": Handler(9, 5, ("scale", "has_end")),
    "ct_ffi_cutce_fwd": Handler(4, 5, ("sparse_compaction",)),
    "ct_ffi_cutce_bwd": Handler(7, 3, ("sparse_compaction", "head_trainable")),
    "ct_ffi_canonicalize_segment_ids": Handler(2, 1, ("has_segments",)),
    "ct_ffi_shifted_targets": Handler(6, 3, ("has_mask", "has_segments", "has_assistant", "has_loss_mask",
                                             "has_labels", "ignore_index")),
    "ct_ffi_position_ids": Handler(2, 1, ()),
    "ct_ffi_rotary_cos_sin": Handler(2, 2, ()),
    "ct_ffi_apply_rotary": Handler(4, 2, ("rope_style", "inverse", "q_scale")),
    "ct_ffi_rms_norm_fwd": Handler(2, 1, ("eps",)),
    "ct_ffi_rms_norm_bwd": Handler(3, 3, ("eps",)),
    "ct_ffi_sparse_ce_fwd": Handler(3, 2, ()),
    "ct_ffi_sparse_ce_bwd": Handler(5, 1, ()),
}


@functools.lru_cache(maxsize=1)
def register() -> None:
    """Registers every handler of libct_ffi.so for platform ROCM (once per process)."""

    import jax

    if not _FFI_LIBRARY.exists():
        raise RuntimeError(f"{_FFI_LIBRARY} is missing: build csrc/ct_ffi.cc against jaxlib's FFI headers")
    library = ctypes.CDLL(str(_FFI_LIBRARY))
    for name in HANDLERS:
        jax.ffi.register_ffi_target(name, jax.ffi.pycapsule(getattr(library, name)), platform="ROCM")


def _call(name: str, results, *operands, **attributes):
    """One custom call; counts are checked against HANDLERS before anything reaches XLA."""

    import jax

    handler = HANDLERS[name]
    if (len(operands), len(results), tuple(attributes)) != handler:
        raise TypeError(f"{name} takes {handler}, got {len(operands)} operands, {len(results)} results, "
                        f"attributes {tuple(attributes)}")
    register()
    return jax.ffi.ffi_call(name, tuple(results))(*operands, **attributes)


def _struct(shape, dtype):
    import jax

    return jax.ShapeDtypeStruct(tuple(shape), dtype)


def _require_gpu(operator_name: str) -> None:
    import jax

    if jax.default_backend() not in ("gpu", "rocm"):
        raise RuntimeError(f"{operator_name} is available only on a ROCm GPU")


def _require_one_device(mesh, operator_name: str) -> None:
    if mesh is None:
        raise ValueError(f"{operator_name} requires the training Mesh")
    active = _Axes(mesh).beyond_one_device()
    if active:
        raise ValueError(f"this build runs on one GPU; mesh axes larger than 1: {active}")


# ------------------------------------------------------------------------------------------
# attention
# ------------------------------------------------------------------------------------------
class AttentionMetadata(NamedTuple):
    """Packed metadata reused across layers, optionally with per-query end keys (inclusive global
    key indices). Hybrid query summaries carry the maximum visible end as a third column.
    ``tile_bounds`` is this build's addition: the int32 table the HIP kernels read."""

    query_segment_ids: Any
    kv_segment_ids: Any
    q_block_segments: Any
    kv_block_segments: Any
    attention_end: Any = None
    tile_bounds: Any = None


def _block_summary(segments, block: int):
    """(smallest nonzero id, largest id) of every block of ``block`` positions; (0, 0) for a block
    of padding (efficient_attention.py:313-323)."""

    import jax.numpy as jnp

    batch, sequence = segments.shape
    tiles = segments.reshape(batch, sequence // block, block)
    largest = tiles.max(axis=-1)
    smallest = jnp.where(tiles == 0, jnp.iinfo(jnp.int32).max, tiles).min(axis=-1)
    return jnp.stack((jnp.where(largest == 0, 0, smallest), largest), axis=-1).astype(jnp.int32)


def prepare_attention_metadata(canonical_segment_ids, *, mesh, profile, attention_end=None) -> AttentionMetadata:
    """Build the per-block summaries and the kernels' tile table once, before the decoder loop."""

    import jax.numpy as jnp

    if mesh is None:
        raise ValueError("attention metadata preparation requires the training mesh")
    if not isinstance(profile, AttentionKernelProfile):
        raise TypeError("profile must be an AttentionKernelProfile")
    _require_one_device(mesh, "prepare_attention_metadata")
    segments = jnp.asarray(canonical_segment_ids, dtype=jnp.int32)
    if segments.ndim != 2:
        raise ValueError(f"canonical_segment_ids must be [batch, sequence], got {segments.shape}")
    if segments.shape[0] == 0 or segments.shape[1] == 0:
        raise ValueError("canonical_segment_ids must have non-empty batch and sequence dimensions")
    block_q = _positive(profile.block_q, "profile.block_q")
    outer = _positive(profile.block_kv_outer, "profile.block_kv_outer")
    batch, sequence = segments.shape
    if sequence % block_q or sequence % outer:
        raise ValueError(f"metadata sequence must be divisible by profile blocks, got shape={segments.shape}, "
                         f"profile={profile}")
    q_summary, kv_summary = _block_summary(segments, block_q), _block_summary(segments, outer)
    has_end = attention_end is not None
    if has_end:
        attention_end = jnp.asarray(attention_end, dtype=jnp.int32)
        if attention_end.shape != segments.shape:
            raise ValueError("attention_end must match canonical_segment_ids")
        reach = jnp.where(segments != 0, attention_end, 0).reshape(batch, -1, block_q).max(axis=-1)
        q_summary = jnp.concatenate((q_summary, reach[..., None]), axis=-1)
    words = int(_lib.load().ct_attn_meta_bytes(batch, sequence)) // 4
    (tile_bounds,) = _call("ct_ffi_attn_prepare", [_struct((words,), jnp.int32)],
                           segments, attention_end if has_end else segments, has_end=has_end)
    return AttentionMetadata(segments, segments, q_summary, kv_summary, attention_end, tile_bounds)


def _validate_metadata(metadata, query_shape, profile) -> None:
    import jax.numpy as jnp

    if not isinstance(metadata, AttentionMetadata):
        raise TypeError("metadata must be AttentionMetadata")
    batch, sequence = query_shape[:2]
    hybrid = metadata.attention_end is not None
    expected = {
        "query_segment_ids": (batch, sequence),
        "kv_segment_ids": (batch, sequence),
        "q_block_segments": (batch, sequence // profile.block_q, 3 if hybrid else 2),
        "kv_block_segments": (batch, sequence // profile.block_kv_outer, 2),
    }
    if hybrid:
        expected["attention_end"] = (batch, sequence)
    for name, shape in expected.items():
        value = getattr(metadata, name)
        if value.shape != shape:
            raise ValueError(f"metadata.{name} must have shape {shape}, got {value.shape}")
        if value.dtype != jnp.int32:
            raise TypeError(f"metadata.{name} must have dtype int32, got {value.dtype}")
    words = int(_lib.load().ct_attn_meta_bytes(batch, sequence)) // 4
    if metadata.tile_bounds is None or metadata.tile_bounds.shape != (words,):
        raise ValueError("metadata.tile_bounds is missing; build it with prepare_attention_metadata")


def _attention_forward(query, key, value, metadata, scale):
    import jax.numpy as jnp

    has_end = metadata.attention_end is not None
    return _call("ct_ffi_attn_fwd",
                 [_struct(query.shape, jnp.bfloat16), _struct(query.shape[:3], jnp.float32)],
                 query, key, value, metadata.query_segment_ids,
                 metadata.attention_end if has_end else metadata.query_segment_ids, metadata.tile_bounds,
                 scale=np.float32(scale), has_end=has_end)


def _attention_backward(query, key, value, metadata, output, lse, output_cotangent, scale):
    import jax.numpy as jnp

    has_end = metadata.attention_end is not None
    batch, sequence, q_heads, head_dim = query.shape
    scratch = int(_lib.load().ct_attn_bwd_workspace_bytes(batch, sequence, q_heads, key.shape[2], head_dim))
    dq, dk, dv, _, _ = _call(
        "ct_ffi_attn_bwd",
        [_struct(query.shape, jnp.bfloat16), _struct(key.shape, jnp.bfloat16), _struct(value.shape, jnp.bfloat16),
         _struct((batch, q_heads, sequence), jnp.float32),      # delta scratch, head-major
         _struct((scratch,), jnp.uint8)],
        query, key, value, metadata.query_segment_ids,
        metadata.attention_end if has_end else metadata.query_segment_ids, metadata.tile_bounds, output, lse,
        output_cotangent.astype(jnp.bfloat16), scale=np.float32(scale), has_end=has_end)
    return dq, dk, dv


@functools.lru_cache(maxsize=1)
def _efficient_attention_impl():
    """The custom-VJP function (built on first use so that importing this module needs no jax)."""

    import jax

    @functools.partial(jax.custom_vjp, nondiff_argnums=(4, 5, 6, 7))
    def impl(query, key, value, metadata, mesh, profile, scale, causal):
        return _attention_forward(query, key, value, metadata, scale)[0]

    def impl_fwd(query, key, value, metadata, mesh, profile, scale, causal):
        output, lse = _attention_forward(query, key, value, metadata, scale)
        return output, (query, key, value, metadata, output, lse)

    def impl_bwd(mesh, profile, scale, causal, residual, output_cotangent):
        query, key, value, metadata, output, lse = residual
        dq, dk, dv = _attention_backward(query, key, value, metadata, output, lse, output_cotangent, scale)
        return dq, dk, dv, None

    impl.defvjp(impl_fwd, impl_bwd)
    return impl


def efficient_attention(query, key, value, metadata: AttentionMetadata, *, mesh, profile=None, scale=None,
                        causal: bool = True):
    """Segment-isolated causal (or ``attention_end``-bounded) attention with its analytic VJP."""

    import jax
    import jax.numpy as jnp

    query, key, value = jnp.asarray(query), jnp.asarray(key), jnp.asarray(value)
    _require_one_device(mesh, "efficient_attention")
    if not isinstance(causal, bool):
        raise TypeError("causal must be a compile-time bool")
    if not causal:
        raise ValueError("the efficient backend implements causal attention only")
    if key.shape != value.shape:
        raise ValueError(f"key and value shapes differ: {key.shape} and {value.shape}")
    query_shape, key_shape, _, _ = _validate_qkv_shapes(query.shape, key.shape, mesh)
    if query_shape[-1] not in _SUPPORTED_HEAD_DIMS:
        raise ValueError(f"the efficient attention kernel requires head_dim in {_SUPPORTED_HEAD_DIMS}; "
                         f"got head_dim={query_shape[-1]}")
    if not (query.dtype == key.dtype == value.dtype == jnp.bfloat16):
        raise TypeError(f"efficient_attention requires BF16 query/key/value, got {query.dtype}, {key.dtype}, "
                        f"{value.dtype}")
    _require_gpu("efficient_attention")
    if profile is None:
        profile = resolve_attention_profile(query_shape, key_shape, mesh,
                                            has_attention_end=metadata.attention_end is not None)
    validate_attention_profile(profile, query_shape, key_shape, mesh)
    _validate_metadata(metadata, query_shape, profile)
    if scale is None:
        scale = default_attention_scale(query_shape[-1])
    else:
        if isinstance(scale, (jax.Array, jax.core.Tracer)):
            raise TypeError("scale must be a compile-time Python scalar")
        try:
            scale = float(scale)
        except (TypeError, ValueError) as error:
            raise TypeError("scale must be a compile-time Python scalar") from error
        if not math.isfinite(scale):
            raise ValueError(f"scale must be finite, got {scale}")
    return _efficient_attention_impl()(query, key, value, metadata, mesh, profile, scale, causal)


# ------------------------------------------------------------------------------------------
# cut cross-entropy
# ------------------------------------------------------------------------------------------
def _cutce_shape(rows: int, hidden: int, vocab: int):
    return _lib.CutceShape(rows=rows, hidden=hidden, vocab=vocab)


def backward_workspace_bytes(rows: int, hidden: int, vocab: int, local_chunk_size: int) -> int:
    """Workspace of the backward. Without chunking the dlogits slab spans the vocabulary; with
    ``local_chunk_size`` rows per chunk the slab is as large as the dlogits of one chunk of rows
    would be (never below the kernels' minimum), and the vocabulary is walked in slabs."""

    lib = _lib.load()
    shape = _cutce_shape(rows, hidden, vocab)
    full, least = int(lib.ct_cutce_bwd_workspace_bytes(shape)), int(lib.ct_cutce_bwd_workspace_min_bytes(shape))
    if local_chunk_size <= 0 or local_chunk_size >= rows:
        return full
    return max(least, min(full, least + (full - least) * local_chunk_size // rows))


@functools.lru_cache(maxsize=1)
def _cut_ce_impl():
    import jax
    import jax.numpy as jnp

    def forward(hidden, head, targets, weights, sparse_compaction, cache_bytes):
        rows, width = hidden.shape
        lib = _lib.load()
        scalar = _struct((1,), jnp.float32)
        workspace = int(lib.ct_cutce_fwd_workspace_bytes(_cutce_shape(rows, width, head.shape[1])))
        nll, weight_sum, lse, _, cache = _call(
            "ct_ffi_cutce_fwd",
            [scalar, scalar, _struct((rows,), jnp.float32), _struct((workspace,), jnp.uint8),
             _struct((max(cache_bytes, 16),), jnp.uint8)],              # 16 bytes = "no cache"
            hidden, head, targets, weights, sparse_compaction=bool(sparse_compaction))
        return nll[0], weight_sum[0], lse, cache

    @functools.partial(jax.custom_vjp, nondiff_argnums=(4, 5, 6))
    def cut_ce(hidden, head, targets, weights, lm_head_trainable, sparse_compaction, local_chunk_size):
        nll, weight_sum, _, _ = forward(hidden, head, targets, weights, sparse_compaction, 0)
        return nll, weight_sum

    def cut_ce_fwd(hidden, head, targets, weights, lm_head_trainable, sparse_compaction, local_chunk_size):
        cache_bytes = 0
        if not local_chunk_size:            # a chunked call asks for bounded memory: no logits cache
            size = int(_lib.load().ct_cutce_logits_cache_bytes(_cutce_shape(*hidden.shape, head.shape[1])))
            cache_bytes = size if size <= LOGITS_CACHE_LIMIT_BYTES else 0
        nll, weight_sum, lse, cache = forward(hidden, head, targets, weights, sparse_compaction, cache_bytes)
        return (nll, weight_sum), (hidden, head, targets, weights, lse, cache)

    def cut_ce_bwd(lm_head_trainable, sparse_compaction, local_chunk_size, residual, cotangents):
        hidden, head, targets, weights, lse, cache = residual
        nll_cotangent, _ = cotangents                         # the cotangent of weight_sum is ignored (:608)
        rows, width = hidden.shape
        workspace = backward_workspace_bytes(rows, width, head.shape[1], local_chunk_size)
        # a frozen head gets no gradient buffer: 8 elements stand in for the result XLA insists on
        head_result = _struct(head.shape if lm_head_trainable else (8,), head.dtype)
        dhidden, dhead, _ = _call(
            "ct_ffi_cutce_bwd",
            [_struct(hidden.shape, hidden.dtype), head_result, _struct((workspace,), jnp.uint8)],
            hidden, head, targets, weights, lse, jnp.reshape(nll_cotangent.astype(jnp.float32), (1,)), cache,
            sparse_compaction=bool(sparse_compaction), head_trainable=bool(lm_head_trainable))
        return dhidden, (dhead if lm_head_trainable else None), None, None

    cut_ce.defvjp(cut_ce_fwd, cut_ce_bwd)
    return cut_ce


def pallas_cut_linear_cross_entropy(hidden_states, lm_head_kernel, targets, weights, *, mesh,
                                    sparse_compaction: bool = False, lm_head_trainable: bool = True,
                                    local_chunk_size: int = 0):
    """``(nll_sum, weight_sum)`` of the projection-fused sparse cross-entropy, without logits.

    hidden_states ``[B, S, d]`` and lm_head_kernel ``[d, V]`` in bfloat16, targets int32 ``[B, S]``,
    weights f32 ``[B, S]``; a row is ignored iff its weight is 0. ``local_chunk_size`` > 0 bounds
    the backward's workspace to what one chunk of that many rows needs (``backward_workspace_bytes``).
    """

    import jax.numpy as jnp

    local_chunk_size = _integer(local_chunk_size, "local_chunk_size must be a static non-negative integer")
    if local_chunk_size < 0:
        raise ValueError("local_chunk_size must be non-negative")
    hidden_states, lm_head_kernel = jnp.asarray(hidden_states), jnp.asarray(lm_head_kernel)
    targets, weights = jnp.asarray(targets, dtype=jnp.int32), jnp.asarray(weights, dtype=jnp.float32)
    if hidden_states.ndim != 3:
        raise ValueError("Cut cross-entropy expects hidden_states [batch, sequence, hidden]")
    batch, sequence, hidden = hidden_states.shape
    if lm_head_kernel.ndim != 2 or lm_head_kernel.shape[0] != hidden:
        raise ValueError("lm_head_kernel must have shape [hidden, vocab]")
    if not (targets.shape == weights.shape == (batch, sequence)):
        raise ValueError("targets and weights must match hidden_states.shape[:-1]")
    if batch * sequence == 0:
        raise ValueError("Cut cross-entropy requires at least one token row")
    if hidden == 0 or hidden % _HIDDEN_ALIGN:
        raise ValueError("Cut cross-entropy hidden size must be divisible by 128")
    if lm_head_kernel.shape[1] == 0:
        raise ValueError("Cut cross-entropy requires a non-empty vocabulary")
    if hidden_states.dtype != lm_head_kernel.dtype:
        raise TypeError("hidden_states and lm_head_kernel must use the same compute dtype")
    if not jnp.issubdtype(hidden_states.dtype, jnp.floating):
        raise TypeError("Cut cross-entropy inputs must have a floating dtype")
    if hidden_states.dtype != jnp.bfloat16:
        raise TypeError("this build computes Cut cross-entropy in bfloat16 only")
    _require_gpu("Cut cross-entropy")
    if mesh is None:
        raise ValueError("Cut cross-entropy requires the training Mesh")
    active = _Axes(mesh).beyond_one_device()
    unsupported = [axis for axis in ("fsdp", "ep") if axis in active]
    if unsupported:
        raise ValueError("Cut cross-entropy currently requires fsdp=ep=1; active unsupported axes: "
                         + ", ".join(unsupported))
    if active:
        raise ValueError(f"this build runs on one GPU; mesh axes larger than 1: {active}")
    return _cut_ce_impl()(hidden_states.reshape(-1, hidden), lm_head_kernel, targets.reshape(-1), weights.reshape(-1),
                          bool(lm_head_trainable), bool(sparse_compaction), local_chunk_size)


# ------------------------------------------------------------------------------------------
# preparation steps in front of the hot paths (integer kernels, nothing to differentiate)
# ------------------------------------------------------------------------------------------
def canonicalize_segment_ids(attention_mask, segment_ids=None):
    """One-based ids of contiguous valid runs, zero for padding (int32 ``[batch, sequence]``)."""

    import jax.numpy as jnp

    valid = jnp.asarray(attention_mask, dtype=jnp.bool_)
    if valid.ndim != 2:
        raise ValueError(f"attention_mask must have shape [batch, sequence], got {valid.shape}")
    mask = valid.astype(jnp.int32)
    has_segments = segment_ids is not None
    if has_segments:
        labels = jnp.asarray(segment_ids, dtype=jnp.int32)
        if labels.shape != valid.shape:
            raise ValueError(f"segment_ids must have shape {valid.shape}, got {labels.shape}")
    else:
        labels = mask                                  # placeholder of the right shape, not read
    if valid.size == 0:
        return jnp.zeros(valid.shape, jnp.int32)
    (canonical,) = _call("ct_ffi_canonicalize_segment_ids", [_struct(valid.shape, jnp.int32)], mask, labels,
                         has_segments=has_segments)
    return canonical


def shifted_targets_and_weights(input_ids, attention_mask, segment_ids=None, assistant_mask=None, loss_mask=None,
                                labels=None, *, ignore_index: int = -100):
    """Safe shifted targets (int32) and target-position loss weights (f32), ``[batch, sequence - 1]`` each."""

    import jax.numpy as jnp

    tokens = jnp.asarray(input_ids, dtype=jnp.int32)
    if tokens.ndim != 2:
        raise ValueError(f"input_ids must have shape [batch, sequence], got {tokens.shape}")

    def optional(value, name, convert):
        if value is None:
            return tokens, False                       # placeholder of the right shape, not read
        array = convert(jnp.asarray(value))
        if array.shape != tokens.shape:
            raise ValueError(f"{name} must have shape {tokens.shape}, got {array.shape}")
        return array, True

    label_array, has_labels = optional(labels, "labels", lambda a: a.astype(jnp.int32))
    # validity is "mask == 1" (losses.py:49)
    mask_array, has_mask = optional(attention_mask, "attention_mask", lambda a: (a == 1).astype(jnp.int32))
    segment_array, has_segments = optional(segment_ids, "segment_ids", lambda a: a.astype(jnp.int32))
    assistant_array, has_assistant = optional(assistant_mask, "assistant_mask", lambda a: (a != 0).astype(jnp.int32))
    if loss_mask is None:
        loss_array, has_loss_mask = jnp.zeros(tokens.shape, jnp.float32), False
    else:
        loss_array, has_loss_mask = jnp.asarray(loss_mask, dtype=jnp.float32), True
        if loss_array.shape != tokens.shape:
            raise ValueError(f"loss_mask must have shape {tokens.shape}, got {loss_array.shape}")
    batch, sequence = tokens.shape
    if sequence < 2:
        raise ValueError("input_ids needs at least two positions to form a prediction edge")
    if has_segments and not has_mask:                  # canonical runs need a validity mask: every token valid
        mask_array, has_mask = jnp.ones(tokens.shape, jnp.int32), True
    scratch = max(16, int(_lib.load().ct_shifted_targets_scratch_bytes(batch, sequence)))
    targets, weights, _ = _call(
        "ct_ffi_shifted_targets",
        [_struct((batch, sequence - 1), jnp.int32), _struct((batch, sequence - 1), jnp.float32),
         _struct((scratch,), jnp.uint8)],
        tokens, mask_array, segment_array, assistant_array, loss_array, label_array,
        has_mask=has_mask, has_segments=has_segments, has_assistant=has_assistant, has_loss_mask=has_loss_mask,
        has_labels=has_labels, ignore_index=np.int32(ignore_index))
    return targets, weights


# ------------------------------------------------------------------------------------------
# decoder-layer neighbours of attention
# ------------------------------------------------------------------------------------------
_ROPE_STYLES = {"gpt-j": 0, "gpt-neox": 1}


def _make_position_ids_precanonicalized(attention_mask, segment_ids):
    import jax.numpy as jnp

    valid = jnp.asarray(attention_mask, dtype=jnp.bool_)
    if valid.ndim != 2:
        raise ValueError(f"attention_mask must have shape [batch, sequence], got {valid.shape}")
    segments = jnp.asarray(segment_ids, dtype=jnp.int32)
    if segments.shape != valid.shape:
        raise ValueError(f"segment_ids must have shape {valid.shape}, got {segments.shape}")
    if valid.size == 0:
        return jnp.zeros(valid.shape, jnp.int32)
    (positions,) = _call("ct_ffi_position_ids", [_struct(valid.shape, jnp.int32)], valid.astype(jnp.int32), segments)
    return positions


def make_position_ids(attention_mask, segment_ids=None):
    """Zero-based positions that reset at every packed segment (int32 ``[batch, sequence]``)."""

    import jax.numpy as jnp

    valid = jnp.asarray(attention_mask, dtype=jnp.bool_)
    if valid.ndim != 2:
        raise ValueError(f"attention_mask must have shape [batch, sequence], got {valid.shape}")
    return _make_position_ids_precanonicalized(valid, canonicalize_segment_ids(valid, segment_ids))


def rotary_cos_sin(position_ids, inv_freq, dtype):
    """Per-token cos / sin tables ``[batch, sequence, rotary_dim / 2]``: f32 angles, one cast to bf16."""

    import jax.numpy as jnp

    positions = jnp.asarray(position_ids)
    if positions.ndim != 2:
        raise ValueError(f"position_ids must have shape [batch, sequence], got {positions.shape}")
    frequencies = jnp.asarray(inv_freq, dtype=jnp.float32)
    if frequencies.ndim != 1 or frequencies.shape[0] == 0:
        raise ValueError(f"inv_freq must be a non-empty vector, got {frequencies.shape}")
    if jnp.dtype(dtype) != jnp.bfloat16:
        raise ValueError("the MI355X path computes rotary tables in bfloat16 only")
    table = _struct(positions.shape + (frequencies.shape[0],), jnp.bfloat16)
    cosine, sine = _call("ct_ffi_rotary_cos_sin", [table, table], positions.astype(jnp.int32), frequencies)
    return cosine, sine


@functools.lru_cache(maxsize=1)
def _apply_rotary_impl():
    import jax
    import jax.numpy as jnp

    def rotate(query, key, cosine, sine, style, q_scale, inverse):
        return _call("ct_ffi_apply_rotary", [_struct(query.shape, jnp.bfloat16), _struct(key.shape, jnp.bfloat16)],
                     query, key, cosine, sine, rope_style=np.int32(style), inverse=bool(inverse),
                     q_scale=np.float32(q_scale))

    # the rotation is linear in (query, key): its VJP is the transposed rotation of the cotangents
    @functools.partial(jax.custom_vjp, nondiff_argnums=(4, 5))
    def apply(query, key, cosine, sine, style, q_scale):
        return tuple(rotate(query, key, cosine, sine, style, q_scale, False))

    def apply_fwd(query, key, cosine, sine, style, q_scale):
        return tuple(rotate(query, key, cosine, sine, style, q_scale, False)), (cosine, sine)

    def apply_bwd(style, q_scale, residual, cotangents):
        cosine, sine = residual
        dq, dk = cotangents
        dq_in, dk_in = rotate(dq.astype(jnp.bfloat16), dk.astype(jnp.bfloat16), cosine, sine, style, q_scale, True)
        return dq_in, dk_in, None, None

    apply.defvjp(apply_fwd, apply_bwd)
    return apply


def apply_rotary_cos_sin(query, key, cosine, sine, *, rope_style: str = "gpt-j", q_scale: float = 1.0):
    """Partial RoPE of Q and K ``[batch, sequence, heads, head_dim]`` from precomputed tables.
    ``q_scale`` (not in the reference signature, default off) also applies the attention operator's
    bf16 pre-scale of Q in the same pass; call ``efficient_attention`` with scale 1 then."""

    import jax.numpy as jnp

    if query.ndim != 4 or key.ndim != 4:
        raise ValueError("query and key must have shape [batch, sequence, heads, head_dim]")
    if query.shape[:2] != key.shape[:2] or query.shape[-1] != key.shape[-1]:
        raise ValueError(f"incompatible query/key shapes: {query.shape} and {key.shape}")
    cosine, sine = jnp.asarray(cosine), jnp.asarray(sine)
    if cosine.shape != sine.shape:
        raise ValueError(f"cosine and sine shapes differ: {cosine.shape} and {sine.shape}")
    if cosine.ndim != 3 or cosine.shape[:2] != query.shape[:2]:
        raise ValueError("cosine and sine must have shape "
                         f"[{query.shape[0]}, {query.shape[1]}, rotary_dim / 2], got {cosine.shape}")
    rotary_dim = cosine.shape[-1] * 2
    if rotary_dim <= 0 or rotary_dim > query.shape[-1] or rotary_dim % 2:
        raise ValueError(f"invalid rotary dimension {rotary_dim} for head_dim={query.shape[-1]}")
    if rope_style not in _ROPE_STYLES:
        raise ValueError("rope_style must be 'gpt-j' or 'gpt-neox'")
    if query.dtype != jnp.bfloat16 or key.dtype != jnp.bfloat16:
        raise ValueError("the MI355X path rotates bfloat16 query and key only")
    return _apply_rotary_impl()(query, key, cosine.astype(jnp.bfloat16), sine.astype(jnp.bfloat16),
                                _ROPE_STYLES[rope_style], float(q_scale))


def apply_rotary_embedding(query, key, position_ids, inv_freq, *, rope_style: str = "gpt-j"):
    """Partial RoPE of Q and K from positions (``[sequence]`` or ``[batch, sequence]``) and inverse frequencies."""

    import jax.numpy as jnp

    if query.ndim != 4 or key.ndim != 4:
        raise ValueError("query and key must have shape [batch, sequence, heads, head_dim]")
    if query.shape[:2] != key.shape[:2] or query.shape[-1] != key.shape[-1]:
        raise ValueError(f"incompatible query/key shapes: {query.shape} and {key.shape}")
    positions = jnp.asarray(position_ids)
    if positions.ndim == 1:
        positions = jnp.broadcast_to(positions[None, :], query.shape[:2])
    if positions.shape != query.shape[:2]:
        raise ValueError(f"position_ids must have shape {query.shape[:2]}, got {positions.shape}")
    inv_freq = jnp.asarray(inv_freq, dtype=jnp.float32)
    rotary_dim = inv_freq.shape[0] * 2
    if rotary_dim <= 0 or rotary_dim > query.shape[-1] or rotary_dim % 2:
        raise ValueError(f"invalid rotary dimension {rotary_dim} for head_dim={query.shape[-1]}")
    cosine, sine = rotary_cos_sin(positions, inv_freq, query.dtype)
    return apply_rotary_cos_sin(query, key, cosine, sine, rope_style=rope_style)


@functools.lru_cache(maxsize=1)
def _rms_norm_impl():
    import jax
    import jax.numpy as jnp

    @functools.partial(jax.custom_vjp, nondiff_argnums=(2,))
    def norm(x, scale, eps):
        (y,) = _call("ct_ffi_rms_norm_fwd", [_struct(x.shape, jnp.bfloat16)], x, scale, eps=np.float32(eps))
        return y

    def norm_fwd(x, scale, eps):
        return norm(x, scale, eps), (x, scale)

    def norm_bwd(eps, residual, dy):
        x, scale = residual
        hidden = x.shape[-1]
        workspace = int(_lib.load().ct_rms_norm_bwd_workspace_bytes(hidden))
        dx, dscale, _ = _call(
            "ct_ffi_rms_norm_bwd",
            [_struct(x.shape, jnp.bfloat16), _struct((hidden,), jnp.float32), _struct((max(workspace, 16),), jnp.uint8)],
            x, scale, dy.astype(jnp.bfloat16), eps=np.float32(eps))
        return dx, dscale.astype(scale.dtype)

    norm.defvjp(norm_fwd, norm_bwd)
    return norm


def rms_norm(x, scale, eps: float, compute_dtype):
    """RMS normalisation over the last axis with f32 statistics and a learned scale (bf16 in, bf16 out)."""

    import jax.numpy as jnp

    x, scale = jnp.asarray(x), jnp.asarray(scale)
    if jnp.dtype(compute_dtype) != jnp.bfloat16 or x.dtype != jnp.bfloat16:
        raise ValueError("the MI355X path normalises bfloat16 activations with a bfloat16 compute dtype")
    if scale.ndim != 1 or scale.shape[0] != x.shape[-1]:
        raise ValueError(f"scale must have shape ({x.shape[-1]},), got {scale.shape}")
    if x.size == 0:
        return x
    return _rms_norm_impl()(x, scale.astype(jnp.bfloat16), float(eps))


# ------------------------------------------------------------------------------------------
# sparse cross-entropy on materialised logits (the trainer's non-fused loss backend)
# ------------------------------------------------------------------------------------------
@functools.lru_cache(maxsize=1)
def _sparse_ce_impl():
    import jax
    import jax.numpy as jnp

    def forward(logits, targets, weights):
        rows = _struct((logits.shape[0],), jnp.float32)
        return _call("ct_ffi_sparse_ce_fwd", [rows, rows], logits, targets, weights)

    @jax.custom_vjp
    def loss(logits, targets, weights):
        return forward(logits, targets, weights)[0]

    def loss_fwd(logits, targets, weights):
        per_row, lse = forward(logits, targets, weights)
        return per_row, (logits, targets, weights, lse)

    def loss_bwd(residual, dy):
        logits, targets, weights, lse = residual
        (dlogits,) = _call("ct_ffi_sparse_ce_bwd", [_struct(logits.shape, logits.dtype)], logits, targets, weights,
                           lse, dy.astype(jnp.float32))
        return dlogits, None, None

    loss.defvjp(loss_fwd, loss_bwd)
    return loss


def pallas_fused_sparse_cross_entropy(logits, targets, weights, *, mesh):
    """Per-token weighted CE ``[batch, sequence]`` (f32) of logits ``[batch, sequence, vocab]`` (bf16 or
    f32); rows with target -100 or weight 0 contribute nothing and are not read."""

    import jax.numpy as jnp

    logits = jnp.asarray(logits)
    if logits.ndim != 3 or targets.shape != logits.shape[:-1] or weights.shape != targets.shape:
        raise ValueError("Pallas CE expects logits [batch, sequence, vocab] and matching target/weight rows")
    _require_one_device(mesh, "pallas_fused_sparse_cross_entropy")
    if logits.dtype not in (jnp.bfloat16, jnp.float32):
        raise ValueError("logits must be bfloat16 or float32")
    leading = logits.shape[:-1]
    if logits.size == 0:
        return jnp.zeros(leading, jnp.float32)
    flat = _sparse_ce_impl()(logits.reshape(-1, logits.shape[-1]), jnp.asarray(targets, jnp.int32).reshape(-1),
                             jnp.asarray(weights, jnp.float32).reshape(-1))
    return flat.reshape(leading)


__all__ = ["AttentionKernelProfile", "AttentionMetadata", "HANDLERS", "LOGITS_CACHE_LIMIT_BYTES",
           "apply_rotary_cos_sin", "apply_rotary_embedding", "backward_workspace_bytes", "canonicalize_segment_ids",
           "efficient_attention", "make_position_ids", "pallas_cut_linear_cross_entropy",
           "pallas_fused_sparse_cross_entropy", "prepare_attention_metadata", "register", "resolve_attention_profile",
           "rms_norm", "rotary_cos_sin", "shifted_targets_and_weights"]
