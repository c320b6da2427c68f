"""Device-side mirrors of the decoder-layer operations on either side of attention.

``make_position_ids`` / ``rotary_cos_sin`` / ``apply_rotary_cos_sin`` /
``apply_rotary_embedding`` (src/causal_trainer/modeling/rotary.py:63-234) and ``rms_norm``
(src/causal_trainer/modeling/architecture.py:155-162) keep the reference's names, argument
meaning and validation errors; tensors are torch tensors on a ROCm device, bf16 where the
reference's compute dtype is bf16, and the work is done by libct_hotpath.so. ``rms_norm`` and
``apply_rotary_cos_sin`` are differentiable (their backward passes are library kernels too).
"""

from __future__ import annotations

import torch

from . import _lib
from .prep import _int32, canonicalize_segment_ids

_STYLES = {"gpt-j": 0, "gpt-neox": 1}


def _make_position_ids_precanonicalized(attention_mask, segment_ids) -> torch.Tensor:
    mask = torch.as_tensor(attention_mask)
    if mask.ndim != 2:
        raise ValueError(f"attention_mask must have shape [batch, sequence], got {tuple(mask.shape)}")
    valid = _int32(mask != 0, "attention_mask")
    segments = torch.as_tensor(segment_ids)
    if tuple(segments.shape) != tuple(valid.shape):
        raise ValueError(f"segment_ids must have shape {tuple(valid.shape)}, got {tuple(segments.shape)}")
    segments = _int32(segments, "segment_ids")
    batch, sequence = valid.shape
    out = torch.empty_like(valid)
    if batch == 0 or sequence == 0:
        return out
    with torch.cuda.device(valid.device):
        _lib.check(_lib.load().ct_position_ids(_lib.current_stream(), valid.data_ptr(), segments.data_ptr(),
                                               batch, sequence, out.data_ptr()))
    return out


def make_position_ids(attention_mask, segment_ids=None) -> torch.Tensor:
    """Zero-based positions that reset at every packed segment (int32 ``[batch, sequence]``)."""

    mask = torch.as_tensor(attention_mask)
    if mask.ndim != 2:
        raise ValueError(f"attention_mask must have shape [batch, sequence], got {tuple(mask.shape)}")
    return _make_position_ids_precanonicalized(mask, canonicalize_segment_ids(mask, segment_ids))


def rotary_cos_sin(position_ids, inv_freq, dtype=torch.bfloat16):
    """Per-token cos / sin tables ``[batch, sequence, rotary_dim / 2]`` (f32 angles, one cast)."""

    positions = torch.as_tensor(position_ids)
    if positions.ndim != 2:
        raise ValueError(f"position_ids must have shape [batch, sequence], got {tuple(positions.shape)}")
    frequencies = torch.as_tensor(inv_freq)
    if frequencies.ndim != 1 or frequencies.shape[0] == 0:
        raise ValueError(f"inv_freq must be a non-empty vector, got {tuple(frequencies.shape)}")
    if dtype != torch.bfloat16:
        raise ValueError("the MI355X path computes rotary tables in bfloat16 only")
    positions = _int32(positions, "position_ids")
    frequencies = frequencies.to(device=positions.device, dtype=torch.float32).contiguous()
    batch, sequence = positions.shape
    pairs = frequencies.shape[0]
    cosine = torch.empty((batch, sequence, pairs), dtype=torch.bfloat16, device=positions.device)
    sine = torch.empty_like(cosine)
    if batch * sequence:
        with torch.cuda.device(positions.device):
            _lib.check(_lib.load().ct_rotary_cos_sin(
                _lib.current_stream(), positions.data_ptr(), frequencies.data_ptr(), batch * sequence, pairs,
                cosine.data_ptr(), sine.data_ptr()))
    return cosine, sine


def _rotate(query, key, cosine, sine, style: int, inverse: bool, q_scale: float):
    batch, sequence, q_heads, head_dim = query.shape
    q_out, k_out = torch.empty_like(query), torch.empty_like(key)
    args = _lib.RotaryArgs(
        q_in=query.data_ptr(), k_in=key.data_ptr(), q_out=q_out.data_ptr(), k_out=k_out.data_ptr(),
        cosine=cosine.data_ptr(), sine=sine.data_ptr(), tokens=batch * sequence,
        q_heads=q_heads, kv_heads=key.shape[2], head_dim=head_dim, rotary_pairs=cosine.shape[-1],
        rope_style=style, inverse=1 if inverse else 0, q_scale=float(q_scale))
    with torch.cuda.device(query.device):
        _lib.check(_lib.load().ct_apply_rotary(_lib.current_stream(), args))
    return q_out, k_out


class _ApplyRotary(torch.autograd.Function):
    @staticmethod
    def forward(ctx, query, key, cosine, sine, style, q_scale):
        ctx.save_for_backward(cosine, sine)
        ctx.style, ctx.q_scale = style, q_scale
        return _rotate(query, key, cosine, sine, style, False, q_scale)

    @staticmethod
    def backward(ctx, dq, dk):
        cosine, sine = ctx.saved_tensors
        dq_in, dk_in = _rotate(dq.contiguous(), dk.contiguous(), cosine, sine, ctx.style, True, ctx.q_scale)
        return dq_in, dk_in, None, None, None, None


def apply_rotary_cos_sin(query, key, cosine, sine, *, rope_style: str = "gpt-j", q_scale: float = 1.0):
    """Partial RoPE of Q and K ``[batch, sequence, heads, head_dim]`` from precomputed tables.

    ``q_scale`` (not in the reference signature, default off) also applies the attention
    operator's bf16 pre-scale of Q in the same pass; call the attention operator with scale 1 then.
    """

    if query.ndim != 4 or key.ndim != 4:
        raise ValueError("query and key must have shape [batch, sequence, heads, head_dim]")
    if query.shape[:2] != key.shape[:2] or query.shape[-1] != key.shape[-1]:
        raise ValueError(f"incompatible query/key shapes: {tuple(query.shape)} and {tuple(key.shape)}")
    cosine, sine = torch.as_tensor(cosine), torch.as_tensor(sine)
    if cosine.shape != sine.shape:
        raise ValueError(f"cosine and sine shapes differ: {tuple(cosine.shape)} and {tuple(sine.shape)}")
    if cosine.ndim != 3 or cosine.shape[:2] != query.shape[:2]:
        raise ValueError("cosine and sine must have shape "
                         f"[{query.shape[0]}, {query.shape[1]}, rotary_dim / 2], got {tuple(cosine.shape)}")
    rotary_dim = cosine.shape[-1] * 2
    if rotary_dim <= 0 or rotary_dim > query.shape[-1] or rotary_dim % 2:
        raise ValueError(f"invalid rotary dimension {rotary_dim} for head_dim={query.shape[-1]}")
    if rope_style not in _STYLES:
        raise ValueError("rope_style must be 'gpt-j' or 'gpt-neox'")
    if not query.is_cuda:
        raise RuntimeError("query must live on a ROCm GPU")
    if query.dtype != torch.bfloat16 or key.dtype != torch.bfloat16:
        raise ValueError("the MI355X path rotates bfloat16 query and key only")
    cosine = cosine.to(torch.bfloat16).contiguous()
    sine = sine.to(torch.bfloat16).contiguous()
    return _ApplyRotary.apply(query.contiguous(), key.contiguous(), cosine, sine, _STYLES[rope_style],
                              float(q_scale))


def apply_rotary_embedding(query, key, position_ids, inv_freq, *, rope_style: str = "gpt-j"):
    """Partial RoPE of Q and K from positions and inverse frequencies."""

    cosine, sine = rotary_cos_sin(position_ids, inv_freq, query.dtype)
    return apply_rotary_cos_sin(query, key, cosine, sine, rope_style=rope_style)


class _RmsNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, scale, eps):
        hidden = x.shape[-1]
        x2 = x.reshape(-1, hidden)
        y = torch.empty_like(x2)
        with torch.cuda.device(x.device):
            _lib.check(_lib.load().ct_rms_norm_fwd(_lib.current_stream(), x2.data_ptr(), scale.data_ptr(), eps,
                                                   x2.shape[0], hidden, y.data_ptr(), None))
        ctx.save_for_backward(x2, scale)
        ctx.eps, ctx.shape = eps, x.shape
        return y.reshape(x.shape)

    @staticmethod
    def backward(ctx, dy):
        x2, scale = ctx.saved_tensors
        hidden = x2.shape[-1]
        lib = _lib.load()
        dy2 = dy.contiguous().reshape(-1, hidden)
        dx = torch.empty_like(x2)
        dscale = torch.empty(hidden, dtype=torch.float32, device=x2.device)
        workspace = torch.empty(lib.ct_rms_norm_bwd_workspace_bytes(hidden), dtype=torch.uint8, device=x2.device)
        with torch.cuda.device(x2.device):
            _lib.check(lib.ct_rms_norm_bwd(_lib.current_stream(), x2.data_ptr(), scale.data_ptr(), dy2.data_ptr(),
                                           ctx.eps, x2.shape[0], hidden, dx.data_ptr(), dscale.data_ptr(),
                                           workspace.data_ptr(), workspace.numel()))
        return dx.reshape(ctx.shape), dscale.to(scale.dtype), None


def rms_norm(x, scale, eps: float, compute_dtype=torch.bfloat16) -> torch.Tensor:
    """RMS normalisation over the last axis with f32 statistics and a learned scale."""

    if compute_dtype != torch.bfloat16 or x.dtype != torch.bfloat16:
        raise ValueError("the MI355X path normalises bfloat16 activations with a bfloat16 compute dtype")
    if not x.is_cuda:
        raise RuntimeError("x must live on a ROCm GPU")
    if scale.ndim != 1 or scale.shape[0] != x.shape[-1]:
        raise ValueError(f"scale must have shape ({x.shape[-1]},), got {tuple(scale.shape)}")
    if x.numel() == 0:
        return torch.empty_like(x)
    return _RmsNorm.apply(x.contiguous(), scale.to(device=x.device, dtype=torch.bfloat16).contiguous(), float(eps))


__all__ = ["make_position_ids", "rotary_cos_sin", "apply_rotary_cos_sin", "apply_rotary_embedding", "rms_norm"]
