"""CPU restatement of the decoder-layer neighbours of attention. TEST INFRASTRUCTURE ONLY.

Imported by ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline leg; the
product package never imports it.

Restates, operation by operation and with the reference's dtype steps:

* ``make_position_ids`` / ``_make_position_ids_precanonicalized``
  (src/causal_trainer/modeling/rotary.py:63-110),
* ``inverse_frequencies`` (:53-60), ``rotary_cos_sin`` (:132-157),
* ``apply_rotary_cos_sin`` with ``_rotate_adjacent_pairs`` / ``_rotate_half_pairs``
  (:113-129, :160-204), ``apply_rotary_embedding`` (:207-234),
* ``rms_norm`` (src/causal_trainer/modeling/architecture.py:155-162).

Pinned by the known answers of the reference's tests/modeling/test_rotary.py (adjacent and half
pairings against closed-form cos/sin, untouched tail channels, reset and jump positions, the
canonical-run examples), by closed forms (rotation preserves pair norms, inverse rotation
undoes it, unit-scale RMSNorm of a constant row is +-1), by a float64 brute force, and for the
RMSNorm gradients by torch autograd of the same chain against an analytic float64 formula.
Parity unpinned: none of the functions here.
"""

from __future__ import annotations

import numpy as np
import torch

from .attention_ref import canonicalize_segment_ids


def make_position_ids_precanonicalized(attention_mask, segment_ids) -> np.ndarray:
    """rotary.py:82-110: index minus the running maximum of run-start indices."""

    valid = np.asarray(attention_mask).astype(bool)
    if valid.ndim != 2:
        raise ValueError(f"attention_mask must have shape [batch, sequence], got {valid.shape}")
    segments = np.asarray(segment_ids, dtype=np.int32)
    if segments.shape != valid.shape:
        raise ValueError(f"segment_ids must have shape {valid.shape}, got {segments.shape}")
    batch, sequence = valid.shape
    indices = np.broadcast_to(np.arange(sequence, dtype=np.int32), (batch, sequence))
    previous = np.concatenate((np.zeros((batch, 1), np.int32), segments[:, :-1]), axis=1)
    starts = valid & ((segments != previous) | (previous == 0))
    start_indices = np.where(starts, indices, 0)
    segment_starts = np.maximum.accumulate(start_indices, axis=1)
    return np.where(valid, indices - segment_starts, 0).astype(np.int32)


def make_position_ids(attention_mask, segment_ids=None) -> np.ndarray:
    """rotary.py:63-79."""

    valid = np.asarray(attention_mask).astype(bool)
    return make_position_ids_precanonicalized(valid, canonicalize_segment_ids(valid, segment_ids))


def inverse_frequencies(rotary_dim: int, rope_theta: float) -> np.ndarray:
    """rotary.py:53-60: 1 / (base ** (index / dim)) in float32."""

    channels = np.arange(0, rotary_dim, 2, dtype=np.float32)
    base = np.float32(rope_theta)
    return (np.float32(1.0) / np.power(base, channels / np.float32(rotary_dim))).astype(np.float32)


def rotary_cos_sin(position_ids, inv_freq, dtype=torch.bfloat16):
    """rotary.py:132-157: float32 angles and transcendentals, one cast to ``dtype``."""

    positions = np.asarray(position_ids).astype(np.float32)
    if positions.ndim != 2:
        raise ValueError(f"position_ids must have shape [batch, sequence], got {positions.shape}")
    frequencies = np.asarray(inv_freq, dtype=np.float32)
    if frequencies.ndim != 1 or frequencies.shape[0] == 0:
        raise ValueError(f"inv_freq must be a non-empty vector, got {frequencies.shape}")
    angles = positions[..., None] * frequencies[None, None, :]
    cosine = torch.from_numpy(np.cos(angles).astype(np.float32)).to(dtype)
    sine = torch.from_numpy(np.sin(angles).astype(np.float32)).to(dtype)
    return cosine, sine


def _rotate(x: torch.Tensor, cosine: torch.Tensor, sine: torch.Tensor, rope_style: str) -> torch.Tensor:
    # every product and sum is rounded to x's dtype, as jnp evaluates them one by one
    if rope_style == "gpt-j":
        even, odd = x[..., ::2], x[..., 1::2]
        out_even = even * cosine - odd * sine
        out_odd = odd * cosine + even * sine
        return torch.stack((out_even, out_odd), dim=-1).reshape(x.shape)
    first, second = torch.chunk(x, 2, dim=-1)
    out_first = first * cosine - second * sine
    out_second = second * cosine + first * sine
    return torch.cat((out_first, out_second), dim=-1)


def apply_rotary_cos_sin(query, key, cosine, sine, *, rope_style: str = "gpt-j"):
    """rotary.py:160-204 for torch tensors ``[B, S, H, D]`` (any float dtype)."""

    if query.ndim != 4 or key.ndim != 4:
        raise ValueError("query and key must have shape [batch, sequence, heads, head_dim]")
    if query.shape[:2] != key.shape[:2] or query.shape[-1] != key.shape[-1]:
        raise ValueError(f"incompatible query/key shapes: {tuple(query.shape)} and {tuple(key.shape)}")
    if cosine.shape != sine.shape:
        raise ValueError(f"cosine and sine shapes differ: {tuple(cosine.shape)} and {tuple(sine.shape)}")
    if cosine.ndim != 3 or cosine.shape[:2] != query.shape[:2]:
        raise ValueError("cosine and sine must have shape "
                         f"[{query.shape[0]}, {query.shape[1]}, rotary_dim / 2], got {tuple(cosine.shape)}")
    rotary_dim = cosine.shape[-1] * 2
    if rotary_dim <= 0 or rotary_dim > query.shape[-1] or rotary_dim % 2:
        raise ValueError(f"invalid rotary dimension {rotary_dim} for head_dim={query.shape[-1]}")
    if rope_style not in {"gpt-j", "gpt-neox"}:
        raise ValueError("rope_style must be 'gpt-j' or 'gpt-neox'")
    cos4 = cosine[:, :, None, :].to(query.dtype)
    sin4 = sine[:, :, None, :].to(query.dtype)

    def rotate(x):
        rotated = _rotate(x[..., :rotary_dim], cos4, sin4, rope_style)
        if rotary_dim == x.shape[-1]:
            return rotated
        return torch.cat((rotated, x[..., rotary_dim:]), dim=-1)

    return rotate(query), rotate(key)


def apply_rotary_embedding(query, key, position_ids, inv_freq, *, rope_style: str = "gpt-j"):
    """rotary.py:207-234: tables in the query's dtype, then the rotation."""

    cosine, sine = rotary_cos_sin(position_ids, inv_freq, query.dtype)
    return apply_rotary_cos_sin(query, key, cosine, sine, rope_style=rope_style)


def apply_rotary_f64(x, cosine, sine, *, rope_style: str = "gpt-j", inverse: bool = False):
    """Exact rotation of the leading 2*pairs channels in float64 (tables taken as given)."""

    x = x.double()
    c = cosine[:, :, None, :].double()
    s = sine[:, :, None, :].double() * (-1.0 if inverse else 1.0)
    rotary_dim = 2 * cosine.shape[-1]
    return torch.cat((_rotate(x[..., :rotary_dim], c, s, rope_style), x[..., rotary_dim:]), dim=-1)


def rms_norm(x: torch.Tensor, scale: torch.Tensor, eps: float, compute_dtype=torch.bfloat16) -> torch.Tensor:
    """architecture.py:155-162: float32 statistics, product in the compute dtype."""

    original_dtype = x.dtype
    work = x.float()
    normalized = work * torch.rsqrt(torch.mean(torch.square(work), dim=-1, keepdim=True) + eps)
    output = normalized.to(compute_dtype) * scale.to(compute_dtype)
    return output.to(original_dtype)


def rms_norm_vjp(x, scale, eps: float, dy, compute_dtype=torch.bfloat16):
    """Autograd of :func:`rms_norm` (dx in x's dtype, dscale in float32)."""

    xg = x.detach().clone().requires_grad_(True)
    sg = scale.detach().float().clone().requires_grad_(True)
    y = rms_norm(xg, sg, eps, compute_dtype)
    dx, dscale = torch.autograd.grad(y, (xg, sg), dy)
    return dx, dscale


def rms_norm_f64(x, scale, eps: float, dy=None):
    """Closed form in float64: y, and with dy also (dx, dscale)."""

    x64, w64 = x.double(), scale.double()
    r = 1.0 / torch.sqrt(torch.mean(x64 * x64, dim=-1, keepdim=True) + eps)
    xhat = x64 * r
    y = xhat * w64
    if dy is None:
        return y
    g = dy.double() * w64
    dx = r * (g - xhat * torch.mean(g * xhat, dim=-1, keepdim=True))
    dscale = (dy.double() * xhat).reshape(-1, x.shape[-1]).sum(dim=0)
    return y, dx, dscale
