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

import dataclasses
import math
import operator
from collections.abc import Mapping, Sequence
from typing import NamedTuple

import torch

from . import _lib

_TILE_ALIGN = 128
_ROWS_COMMON = 2048
_ROWS_LONG = 1024
_ROWS_HYBRID = 1024
_MAX_QUERY_TOKENS = 512
_MAX_QUERY_COMPUTE_ELEMENTS = 131_072
_SUPPORTED_HEAD_DIMS = (64, 128)


@dataclasses.dataclass(frozen=True)
class AttentionKernelProfile:
    """Static tile choices shared by forward, dQ and dKV (summary granularity here)."""

    block_h: int
    block_q: int
    block_kv_outer: int
    block_kv_compute: int
    compact_statistics: bool = False


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


def _integer(value, complaint: str) -> int:
    """``value`` as a plain int; anything that is not an integer raises ``TypeError(complaint)``."""

    if isinstance(value, bool):
        raise TypeError(complaint)
    try:
        return operator.index(value)
    except TypeError:
        raise TypeError(complaint) from None


def _positive(value, name: str) -> int:
    number = _integer(value, f"{name} must be a static positive integer")
    if number < 1:
        raise ValueError(f"{name} must be positive, got {number}")
    return number


def _dims(shape: Sequence[int], name: str) -> tuple[int, ...]:
    complaint = f"{name} must be a static integer shape"
    try:
        entries = list(shape)
    except TypeError:
        raise TypeError(complaint) from None
    dims = tuple(operator.index(entry) if isinstance(entry, bool) else _integer(entry, complaint)
                 for entry in entries)
    if any(extent < 1 for extent in dims):
        raise ValueError(f"{name} dimensions must be positive, got {dims}")
    return dims


class _Axes:
    """Named axis sizes of a ``mesh`` argument: ``None``, a mapping, or an object whose
    ``.shape`` is one (the reference passes a jax Mesh, :88-104)."""

    def __init__(self, mesh):
        table = {} if mesh is None else getattr(mesh, "shape", mesh)
        if not isinstance(table, Mapping):
            raise TypeError("mesh_shape must be a Mesh or a mapping of named axis sizes")
        self.table = table

    def size(self, axis: str) -> int:
        extent = _integer(self.table.get(axis, 1), f"mesh axis {axis!r} must have a static integer size")
        if extent < 1:
            raise ValueError(f"mesh axis {axis!r} must have a positive size, got {extent}")
        return extent

    def beyond_one_device(self) -> dict[str, int]:
        return {axis: int(extent) for axis, extent in self.table.items() if int(extent) != 1}


def _require_single_device(mesh) -> None:
    active = _Axes(mesh).beyond_one_device()
    if active:
        raise ValueError(f"this build runs on one GPU; mesh axes larger than 1: {active}")


def _validate_qkv_shapes(q_shape, kv_shape, mesh):
    """``(q dims, kv dims, tp, sp)`` after the layout checks of the reference (:107-145)."""

    q, kv = _dims(q_shape, "q_shape"), _dims(kv_shape, "kv_shape")
    if not (len(q) == len(kv) == 4):
        raise ValueError(f"attention shapes must be [batch, sequence, heads, dim], got q={q}, kv={kv}")
    axes = _Axes(mesh)
    tp, sp = axes.size("tp"), axes.size("sp")
    replicas = axes.size("dp") * axes.size("fsdp")
    batch, sequence, heads, width = q
    for broken, text in (
        (kv[:2] != (batch, sequence), f"Q and KV batch/sequence dimensions must match, got q={q}, kv={kv}"),
        (kv[3] != width, f"Q and KV head dimensions must match, got q={width}, kv={kv[3]}"),
        (heads % kv[2] != 0,
         f"query head count must be divisible by the KV head count, got Hq={heads}, Hkv={kv[2]}"),
        (batch % replicas != 0, f"global batch {batch} must be divisible by dp*fsdp={replicas}"),
        (heads % tp != 0, f"Hq={heads} must be divisible by TP={tp}"),
        (sequence % sp != 0, f"sequence={sequence} must be divisible by SP={sp}"),
    ):
        if broken:
            raise ValueError(text)
    return q, kv, tp, sp


_PROFILE_TILES = ("block_h", "block_q", "block_kv_outer", "block_kv_compute")


def validate_attention_profile(profile, q_shape, kv_shape, mesh_shape) -> None:
    """Check divisibility of the profile against the shapes (reference :159-195)."""

    if not isinstance(profile, AttentionKernelProfile):
        raise TypeError(f"profile must be AttentionKernelProfile, got {type(profile).__name__}")
    if type(profile.compact_statistics) is not bool:
        raise TypeError("profile.compact_statistics must be a static bool")
    q, kv, tp, sp = _validate_qkv_shapes(q_shape, kv_shape, mesh_shape)
    heads_h, tile_q, outer, compute = (_positive(getattr(profile, name), name) for name in _PROFILE_TILES)
    sequence, local_heads, local_query = q[1], q[2] // tp, q[1] // sp

    def tiles(length: int, tile: int) -> bool:
        return tile % _TILE_ALIGN == 0 and length % tile == 0

    for broken, text in (
        (heads_h != local_heads, "the efficient kernel requires block_h=local_heads"),
        (not tiles(local_query, tile_q), "block_q must be a 128-aligned divisor of local_query"),
        (not tiles(sequence, outer), "block_kv_outer must be a 128-aligned divisor of sequence"),
        (not tiles(sequence, compute), "block_kv_compute must be a 128-aligned divisor of sequence"),
        (outer % compute != 0, "block_kv_compute must divide block_kv_outer"),
    ):
        if broken:
            raise ValueError(f"{text}; q_shape={q}, kv_shape={kv}, TP={tp}, SP={sp}, local_heads={local_heads}, "
                             f"local_query={local_query}, profile={profile}")


def _pick_tile(length: int, cap: int, complaint: str, nearest_to: float | None = None) -> int:
    """A 128-aligned divisor of ``length`` not above ``cap``: the largest, or the one nearest to
    ``nearest_to`` (ties to the smaller)."""

    options = [tile for tile in range(_TILE_ALIGN, min(length, cap) + 1, _TILE_ALIGN) if length % tile == 0]
    if not options:
        raise ValueError(complaint)
    if nearest_to is None:
        return options[-1]
    return min(options, key=lambda tile: (abs(tile - nearest_to), tile))


# (longest sequence of the tier, query rows per tile summed over heads, outer KV tile, compute KV tile)
_TIERS = ((16_384, _ROWS_COMMON, 512, 256), (262_144, _ROWS_LONG, 1024, 256), (None, _ROWS_LONG, 2048, 512))


def resolve_attention_profile(q_shape, kv_shape, mesh_shape, *, compact_statistics=False,
                              has_attention_end=False) -> AttentionKernelProfile:
    """Resolve the static profile from global shapes (reference tiers, :251-276)."""

    q, _, tp, sp = _validate_qkv_shapes(q_shape, kv_shape, mesh_shape)
    if type(has_attention_end) is not bool:
        raise TypeError("has_attention_end must be a static bool")
    sequence, local_heads, local_query = q[1], q[2] // tp, q[1] // sp
    _, rows, outer_cap, compute_cap = next(tier for tier in _TIERS if tier[0] is None or sequence <= tier[0])
    if has_attention_end:
        rows = min(rows, _ROWS_HYBRID)
    outer = _pick_tile(sequence, outer_cap,
                       f"length has no 128-aligned static divisor: length={sequence}, preferred={outer_cap}")
    compute = _pick_tile(outer, compute_cap,
                         f"length has no 128-aligned static divisor: length={outer}, preferred={compute_cap}")
    tile_q = _pick_tile(local_query, min(_MAX_QUERY_TOKENS, _MAX_QUERY_COMPUTE_ELEMENTS // compute),
                        "SP-local query length has no 128-aligned static divisor: "
                        f"local_query={local_query}, local_heads={local_heads}",
                        nearest_to=rows / local_heads)
    profile = AttentionKernelProfile(block_h=local_heads, block_q=tile_q, block_kv_outer=outer,
                                     block_kv_compute=compute, compact_statistics=compact_statistics)
    validate_attention_profile(profile, q_shape, kv_shape, mesh_shape)
    return profile


def default_attention_scale(head_dim: int) -> float:
    """``head_dim ** -0.5`` (reference :282-286)."""

    return _positive(head_dim, "head_dim") ** -0.5


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


def _attn_backward(query, key, value, metadata, out, lse, dout, scale, with_delta=False):
    batch, sequence, q_heads, head_dim = query.shape
    dq = torch.empty_like(query)
    dk = torch.empty_like(key)
    dv = torch.empty_like(value)
    delta = torch.empty_like(lse)
    workspace_bytes = int(_lib.load().ct_attn_bwd_workspace_bytes(batch, sequence, query.shape[2], key.shape[2], head_dim))
    workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=query.device)
    args = _lib.AttnBwdArgs(
        q=query.data_ptr(), k=key.data_ptr(), v=value.data_ptr(),
        segment_ids=metadata.query_segment_ids.data_ptr(),
        attention_end=_lib.pointer(metadata.attention_end),
        tile_meta=metadata.tile_bounds.data_ptr(),
        out=out.data_ptr(), lse=lse.data_ptr(), dout=dout.data_ptr(),
        dq=dq.data_ptr(), dk=dk.data_ptr(), dv=dv.data_ptr(), delta=delta.data_ptr(),
        workspace=workspace.data_ptr(), workspace_bytes=workspace_bytes,
        batch=batch, seq=sequence, q_heads=q_heads, kv_heads=key.shape[2], head_dim=head_dim,
        scale=scale,
    )
    with torch.cuda.device(query.device):
        _lib.check(_lib.load().ct_attn_bwd(_lib.current_stream(), args))
    if with_delta:
        return dq, dk, dv, delta.view(batch, q_heads, sequence)
    return dq, dk, dv


class _EfficientAttention(torch.autograd.Function):
    """Custom VJP with the reference's residual (q, k, v, metadata, O, LSE) (:1831-1863)."""

    @staticmethod
    def forward(ctx, query, key, value, metadata, scale):
        out, lse = _attn_forward(query, key, value, metadata, scale)
        ctx.save_for_backward(query, key, value, out, lse)
        ctx.attention_metadata = metadata
        ctx.scale = scale
        return out

    @staticmethod
    def backward(ctx, output_cotangent):
        query, key, value, out, lse = ctx.saved_tensors
        dout = output_cotangent.to(torch.bfloat16).contiguous()
        dq, dk, dv = _attn_backward(query, key, value, ctx.attention_metadata, out, lse, dout, ctx.scale)
        return dq, dk, dv, None, None


def efficient_attention(query, key, value, metadata, *, mesh=None, profile=None, scale=None,
                        causal=True):
    """Segment-isolated causal attention forward with its analytic custom VJP.

    query ``[B, S, Hq, D]``, key / value ``[B, S, Hkv, D]``, all bf16 on a ROCm
    device; returns ``[B, S, Hq, D]`` bf16. Gradients flow to query, key, value.
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
        query.contiguous(), key.contiguous(), value.contiguous(), metadata, resolved_scale
    )


def attention_forward_with_lse(query, key, value, metadata, *, scale=None):
    """Forward only, returning ``(O, LSE)``: the residual pair the custom VJP saves."""

    resolved = default_attention_scale(query.shape[-1]) if scale is None else float(scale)
    return _attn_forward(query.contiguous(), key.contiguous(), value.contiguous(), metadata, resolved)


def attention_backward(query, key, value, metadata, out, lse, dout, *, scale=None, with_delta=False):
    """Backward only, from the saved residuals: returns ``(dq, dk, dv)``; with ``with_delta`` also the
    scratch ``delta = rowsum(out * dout)`` as the kernels leave it, head-major ``[B, Hq, S]``."""

    resolved = default_attention_scale(query.shape[-1]) if scale is None else float(scale)
    return _attn_backward(query, key, value, metadata, out, lse, dout.contiguous(), resolved, with_delta)


__all__ = [
    "AttentionKernelProfile",
    "AttentionMetadata",
    "attention_backward",
    "attention_forward_with_lse",
    "default_attention_scale",
    "efficient_attention",
    "prepare_attention_metadata",
    "resolve_attention_profile",
    "tile_bounds_table",
    "validate_attention_profile",
]
