"""Host-side mirror of the reference's Efficient attention operator for MI355X.

Same public names, argument meaning and error behaviour as
``src/causal_trainer/kernels/efficient_attention.py`` (AttentionKernelProfile
:52-60, AttentionMetadata :63-74, resolve_attention_profile :235-279,
prepare_attention_metadata :326-374, efficient_attention :1890-1967), with
torch tensors on a ROCm device instead of jax arrays on TPU, and with the
kernel work done by libct_hotpath.so through its C ABI.

Differences from the reference, all relaxations:
  * GQA: any ``Hkv`` dividing ``Hq`` (the reference kernel needs ``Hkv == 1``;
    the head map ``kv = h // (Hq // Hkv)`` is vanilla_attention's,
    src/causal_trainer/modeling/attention.py:115-118);
  * ``head_dim`` 64 or 128;
  * ``mesh`` may be ``None`` or any mapping / object with ``.shape`` whose axis
    sizes are all 1: this build runs on one GPU.
The profile's tile sizes only set the granularity of the summaries kept in
AttentionMetadata; the HIP kernels use their own 32-row / 64-key tiling and
read per-tile bounds from ``AttentionMetadata.tile_bounds``.
"""

from __future__ import annotations

import math
from typing import NamedTuple

import torch

from . import _lib

from .attention_profile import (AttentionKernelProfile, _Axes, _integer, _positive, _require_single_device,
                                _validate_qkv_shapes, default_attention_scale, resolve_attention_profile,
                                validate_attention_profile)

_SUPPORTED_HEAD_DIMS = (64, 128)


class AttentionMetadata(NamedTuple):
    """Packed metadata reused across layers, optionally with per-query end keys.

    ``attention_end`` holds inclusive global key indices. Hybrid query
    summaries carry the maximum visible end as a third column. ``tile_bounds``
    is this build's addition: the opaque per-tile buffer the HIP kernels read.
    """

    query_segment_ids: torch.Tensor
    kv_segment_ids: torch.Tensor
    q_block_segments: torch.Tensor
    kv_block_segments: torch.Tensor
    attention_end: torch.Tensor | None = None
    tile_bounds: torch.Tensor | None = None


def _as_device_int32(value, name: str) -> torch.Tensor:
    tensor = torch.as_tensor(value)
    if tensor.dtype != torch.int32:
        tensor = tensor.to(torch.int32)
    if not tensor.is_cuda:
        raise RuntimeError(f"{name} must live on a ROCm device")
    return tensor.contiguous()


def _block_summary(segments: torch.Tensor, ends: torch.Tensor | None, block: int) -> torch.Tensor:
    batch, sequence = segments.shape
    width = 3 if ends is not None else 2
    out = torch.empty((batch, sequence // block, width), dtype=torch.int32, device=segments.device)
    lib = _lib.load()
    _lib.check(lib.ct_attn_block_summary(_lib.current_stream(), segments.data_ptr(),
                                         _lib.pointer(ends), batch, sequence, block,
                                         out.data_ptr()))
    return out


def prepare_attention_metadata(canonical_segment_ids, *, mesh, profile,
                               attention_end=None) -> AttentionMetadata:
    """Build per-tile summaries once, immediately before the decoder loop."""

    if not isinstance(profile, AttentionKernelProfile):
        raise TypeError("profile must be an AttentionKernelProfile")
    _require_single_device(mesh)
    segments = _as_device_int32(canonical_segment_ids, "canonical_segment_ids")
    if segments.ndim != 2:
        raise ValueError(f"canonical_segment_ids must be [batch, sequence], got {tuple(segments.shape)}")
    if segments.shape[0] == 0 or segments.shape[1] == 0:
        raise ValueError("canonical_segment_ids must have non-empty batch and sequence dimensions")
    block_q = _positive(profile.block_q, "profile.block_q")
    outer = _positive(profile.block_kv_outer, "profile.block_kv_outer")
    batch, sequence = segments.shape
    if sequence % block_q or sequence % outer:
        raise ValueError(
            f"metadata sequence must be divisible by profile blocks, got shape={tuple(segments.shape)}, "
            f"profile={profile}"
        )
    ends = None
    if attention_end is not None:
        ends = _as_device_int32(attention_end, "attention_end")
        if ends.shape != segments.shape:
            raise ValueError("attention_end must match canonical_segment_ids")

    lib = _lib.load()
    bounds = torch.empty(lib.ct_attn_meta_bytes(batch, sequence) // 4, dtype=torch.int32,
                         device=segments.device)
    with torch.cuda.device(segments.device):
        _lib.check(lib.ct_attn_prepare(_lib.current_stream(), segments.data_ptr(),
                                       _lib.pointer(ends), batch, sequence, bounds.data_ptr()))
        q_summary = _block_summary(segments, ends, block_q)
        kv_summary = _block_summary(segments, None, outer)
    return AttentionMetadata(
        query_segment_ids=segments,
        kv_segment_ids=segments,
        q_block_segments=q_summary,
        kv_block_segments=kv_summary,
        attention_end=ends,
        tile_bounds=bounds,
    )


def tile_bounds_table(metadata: AttentionMetadata) -> torch.Tensor:
    """The ``[B, S/32, 12]`` per-row-block table at the head of ``metadata.tile_bounds``
    (the work-sorted schedules follow it in the same buffer)."""

    batch, sequence = metadata.query_segment_ids.shape
    blocks = sequence // 32
    return metadata.tile_bounds[: batch * blocks * _lib.ATTN_META_WIDTH].view(
        batch, blocks, _lib.ATTN_META_WIDTH)


def _validate_metadata(metadata, query_shape, profile) -> None:
    if not isinstance(metadata, AttentionMetadata):
        raise TypeError("metadata must be AttentionMetadata")
    batch, sequence = query_shape[:2]
    hybrid = metadata.attention_end is not None
    layout = [("query_segment_ids", (batch, sequence)), ("kv_segment_ids", (batch, sequence)),
              ("q_block_segments", (batch, sequence // profile.block_q, 3 if hybrid else 2)),
              ("kv_block_segments", (batch, sequence // profile.block_kv_outer, 2))]
    if hybrid:
        layout.append(("attention_end", (batch, sequence)))
    for name, shape in layout:
        tensor = getattr(metadata, name)
        if tuple(tensor.shape) != shape:
            raise ValueError(f"metadata.{name} must have shape {shape}, got {tuple(tensor.shape)}")
        if tensor.dtype != torch.int32:
            raise TypeError(f"metadata.{name} must have dtype int32, got {tensor.dtype}")
    table = metadata.tile_bounds
    if table is None or table.numel() * 4 != _lib.load().ct_attn_meta_bytes(batch, sequence):
        raise ValueError("metadata.tile_bounds is missing; build it with prepare_attention_metadata")


def _python_scalar(scale) -> float:
    """A static softmax scale as a finite float (the reference rejects traced values, :1950-1957)."""

    complaint = "scale must be a compile-time Python scalar"
    if isinstance(scale, torch.Tensor):
        raise TypeError(complaint)
    try:
        number = float(scale)
    except (TypeError, ValueError):
        raise TypeError(complaint) from None
    if math.isinf(number) or math.isnan(number):
        raise ValueError(f"scale must be finite, got {number}")
    return number


def _attn_forward(query, key, value, metadata, scale):
    batch, sequence, q_heads, head_dim = query.shape
    out = torch.empty_like(query)
    lse = torch.empty((batch, sequence, q_heads), dtype=torch.float32, device=query.device)
    args = _lib.AttnFwdArgs(
        q=query.data_ptr(), k=key.data_ptr(), v=value.data_ptr(),
        segment_ids=metadata.query_segment_ids.data_ptr(),
        attention_end=_lib.pointer(metadata.attention_end),
        tile_meta=metadata.tile_bounds.data_ptr(),
        out=out.data_ptr(), lse=lse.data_ptr(),
        batch=batch, seq=sequence, q_heads=q_heads, kv_heads=key.shape[2], head_dim=head_dim,
        scale=scale,
    )
    with torch.cuda.device(query.device):
        _lib.check(_lib.load().ct_attn_fwd(_lib.current_stream(), args))
    return out, lse


# Left to itself (dq_form=None) the backward offers the library the larger workspace of the
# stored-dS form for rows of up to 4096 positions, if that is at most 4 GiB.
_FROM_DS_UP_TO_SEQ = 4096
_FROM_DS_WORKSPACE_CAP = 4 << 30
_DKV_KERNELS = {None: 0, "narrow": _lib.ATTN_BWD_DKV_NARROW, "wide": _lib.ATTN_BWD_DKV_WIDE}
_DQ_FORMS = {None: 0, "recompute": _lib.ATTN_BWD_DQ_RECOMPUTE, "from_ds": _lib.ATTN_BWD_DQ_FROM_DS}


class BackwardWorkspace:
    """Scratch of the attention backward kept from call to call.

    The dK/dV work list that the backward builds in its scratch buffer depends on the tile metadata,
    the head counts and the form of the backward only. Layers that share one packing can share one
    of these objects (``attention_backward(..., workspace=...)``,
    ``efficient_attention(..., backward_workspace=...)``): the first call builds the list, later
    calls with the same metadata, shape and form tell the library to keep it
    (``CT_ATTN_BWD_WORK_LIST_KEPT``), which saves a launch per call. The calls that share one must
    run on one stream, one after the other."""

    def __init__(self):
        self._buffer = None
        self._built_for = None

    def _acquire(self, nbytes, device, key):
        if self._buffer is None or self._buffer.numel() < nbytes or self._buffer.device != device:
            self._buffer = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self._built_for = None
        return self._buffer, self._built_for == key

    def _built(self, key):
        self._built_for = key


def _attn_backward(query, key, value, metadata, out, lse, dout, scale, with_delta=False, dkv_kernel=None,
                   dq_form=None, workspace_bytes=None, kept=None):
    batch, sequence, q_heads, head_dim = query.shape
    lib = _lib.load()
    dq = torch.empty_like(query)
    dk = torch.empty_like(key)
    dv = torch.empty_like(value)
    delta = torch.empty_like(lse)
    shape = (batch, sequence, query.shape[2], key.shape[2], head_dim)
    if workspace_bytes is None:
        stored = int(lib.ct_attn_bwd_workspace_bytes_from_ds(*shape, int(metadata.attention_end is not None)))
        if dq_form == "from_ds":
            workspace_bytes = stored
            if workspace_bytes == 0:
                raise ValueError("dq_form='from_ds' is not available for this shape (dS blocks of one KV head "
                                 "exceed 64 GiB)")
        elif dq_form is None and sequence <= _FROM_DS_UP_TO_SEQ and 0 < stored <= _FROM_DS_WORKSPACE_CAP:
            # the library then takes the stored-dS form, which is the faster one at such rows
            workspace_bytes = stored
        else:
            workspace_bytes = int(lib.ct_attn_bwd_workspace_bytes(*shape))
    variant = _DKV_KERNELS[dkv_kernel] | _DQ_FORMS[dq_form]
    if kept is None:
        workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=query.device)
    else:
        # (the version counter of the metadata tensor changes when it is written in place)
        built_for = (metadata.tile_bounds.data_ptr(), metadata.tile_bounds._version, shape, variant,
                     workspace_bytes, float(scale))
        workspace, list_kept = kept._acquire(workspace_bytes, query.device, built_for)
        if list_kept:
            variant |= _lib.ATTN_BWD_WORK_LIST_KEPT
    args = _lib.AttnBwdArgs(
        q=query.data_ptr(), k=key.data_ptr(), v=value.data_ptr(),
        segment_ids=metadata.query_segment_ids.data_ptr(),
        attention_end=_lib.pointer(metadata.attention_end),
        tile_meta=metadata.tile_bounds.data_ptr(),
        out=out.data_ptr(), lse=lse.data_ptr(), dout=dout.data_ptr(),
        dq=dq.data_ptr(), dk=dk.data_ptr(), dv=dv.data_ptr(), delta=delta.data_ptr(),
        workspace=workspace.data_ptr(), workspace_bytes=workspace_bytes,
        batch=batch, seq=sequence, q_heads=q_heads, kv_heads=key.shape[2], head_dim=head_dim,
        scale=scale, variant=variant,
    )
    with torch.cuda.device(query.device):
        _lib.check(lib.ct_attn_bwd(_lib.current_stream(), args))
    if kept is not None:
        kept._built(built_for)
    if with_delta:
        return dq, dk, dv, delta.view(batch, q_heads, sequence)
    return dq, dk, dv


class _EfficientAttention(torch.autograd.Function):
    """Custom VJP with the reference's residual (q, k, v, metadata, O, LSE) (:1831-1863)."""

    @staticmethod
    def forward(ctx, query, key, value, metadata, scale, backward_workspace=None):
        out, lse = _attn_forward(query, key, value, metadata, scale)
        ctx.save_for_backward(query, key, value, out, lse)
        ctx.attention_metadata = metadata
        ctx.scale = scale
        ctx.backward_workspace = backward_workspace
        return out

    @staticmethod
    def backward(ctx, output_cotangent):
        query, key, value, out, lse = ctx.saved_tensors
        dout = output_cotangent.to(torch.bfloat16).contiguous()
        dq, dk, dv = _attn_backward(query, key, value, ctx.attention_metadata, out, lse, dout, ctx.scale,
                                    kept=ctx.backward_workspace)
        return dq, dk, dv, None, None, None


def efficient_attention(query, key, value, metadata, *, mesh=None, profile=None, scale=None,
                        causal=True, backward_workspace=None):
    """Segment-isolated causal attention forward with its analytic custom VJP.

    query ``[B, S, Hq, D]``, key / value ``[B, S, Hkv, D]``, all bf16 on a ROCm
    device; returns ``[B, S, Hq, D]`` bf16. Gradients flow to query, key, value.
    ``backward_workspace`` (this build's addition, a :class:`BackwardWorkspace`) lets the layers of
    a model that share ``metadata`` share the scratch buffer of the backward and the work list in it.
    """

    if not isinstance(causal, bool):
        raise TypeError("causal must be a compile-time bool")
    if not causal:
        raise ValueError("the efficient backend implements causal attention only")
    if key.shape != value.shape:
        raise ValueError(f"key and value shapes differ: {tuple(key.shape)} and {tuple(value.shape)}")
    query_shape, key_shape, _, _ = _validate_qkv_shapes(query.shape, key.shape, mesh)
    _require_single_device(mesh)
    if query_shape[-1] not in _SUPPORTED_HEAD_DIMS:
        raise ValueError(
            "the efficient attention kernel requires head_dim in (64, 128); "
            f"got head_dim={query_shape[-1]}"
        )
    if any(t.dtype != torch.bfloat16 for t in (query, key, value)):
        raise TypeError(
            "efficient_attention requires BF16 query/key/value, got "
            f"{query.dtype}, {key.dtype}, {value.dtype}"
        )
    if not (query.is_cuda and key.is_cuda and value.is_cuda):
        raise RuntimeError("efficient_attention is available only on a ROCm GPU")
    has_end = metadata.attention_end is not None if isinstance(metadata, AttentionMetadata) else False
    resolved_profile = (
        resolve_attention_profile(query_shape, key_shape, mesh, has_attention_end=has_end)
        if profile is None else profile
    )
    validate_attention_profile(resolved_profile, query_shape, key_shape, mesh)
    _validate_metadata(metadata, query_shape, resolved_profile)
    resolved_scale = default_attention_scale(query_shape[-1]) if scale is None else _python_scalar(scale)
    return _EfficientAttention.apply(
        query.contiguous(), key.contiguous(), value.contiguous(), metadata, resolved_scale, backward_workspace
    )


def attention_forward_with_lse(query, key, value, metadata, *, scale=None):
    """Forward only, returning ``(O, LSE)``: the residual pair the custom VJP saves."""

    resolved = default_attention_scale(query.shape[-1]) if scale is None else float(scale)
    return _attn_forward(query.contiguous(), key.contiguous(), value.contiguous(), metadata, resolved)


def attention_backward(query, key, value, metadata, out, lse, dout, *, scale=None, with_delta=False,
                       dkv_kernel=None, dq_form=None, workspace_bytes=None, workspace=None):
    """Backward only, from the saved residuals: returns ``(dq, dk, dv)``; with ``with_delta`` also the
    scratch ``-delta = -rowsum(out * dout)`` as the kernels leave it, head-major ``[B, Hq, S]``.

    ``dkv_kernel`` (``"narrow"`` / ``"wide"``) and ``dq_form`` (``"recompute"`` / ``"from_ds"``) pin a
    kernel or a form of the backward for this call (``ct_attn_bwd_args.variant``); ``None`` leaves
    the choice to the library, which is what training code does (the dK/dV kernel goes by sequence
    length; dQ comes from stored dS blocks at rows of up to 4096 positions when their workspace is at
    most 4 GiB, and from a recomputing kernel otherwise). ``workspace_bytes`` overrides the size of the scratch buffer (default: what
    the library asks for the chosen form); ``workspace`` (a :class:`BackwardWorkspace`) keeps the
    buffer, and with it the dK/dV work list, from one call to the next."""

    resolved = default_attention_scale(query.shape[-1]) if scale is None else float(scale)
    return _attn_backward(query, key, value, metadata, out, lse, dout.contiguous(), resolved, with_delta,
                          dkv_kernel, dq_form, workspace_bytes, workspace)


__all__ = [
    "AttentionKernelProfile",
    "AttentionMetadata",
    "BackwardWorkspace",
    "attention_backward",
    "attention_forward_with_lse",
    "default_attention_scale",
    "efficient_attention",
    "prepare_attention_metadata",
    "resolve_attention_profile",
    "tile_bounds_table",
    "validate_attention_profile",
]
