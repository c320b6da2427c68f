"""Framework-neutral part of the attention operator mirror: the static tile profile, its
resolution from global shapes and the shape / mesh validation of the reference
(src/causal_trainer/kernels/efficient_attention.py: AttentionKernelProfile :52-60, mesh and
shape checks :88-145, validate_attention_profile :159-195, resolve_attention_profile :235-279,
default_attention_scale :282-286). Pure Python on ints: imported by the torch operator
(efficient_attention.py) and by the JAX binding (jax_ffi.py), neither of which it imports.
"""

from __future__ import annotations

import dataclasses
import operator
from collections.abc import Mapping, Sequence

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
