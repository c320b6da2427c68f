"""CPU oracle for the attention hot path. TEST INFRASTRUCTURE ONLY.

This file restates, in NumPy / torch-CPU, what the reference computes on the
attention path. It is imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, and by nothing else: the product never calls it.

The reference is a JAX program that cannot be imported in this environment
(jax / jaxlib absent), so parity is anchored on this restatement, which is
pinned by tests/test_oracle_attention.py against
  * every known answer the reference's own tests hold for this path
    (canonical ids, tile summaries, skip predicate, attention_end semantics,
    bidirectional dependency, isolation, default scale),
  * a brute-force float64 triple loop on tiny inputs,
  * torch.nn.functional.scaled_dot_product_attention for the single-segment
    causal special case, and autograd vs the analytic backward.
Citations are relative to the reference root; "src/" = src/causal_trainer/.

Functions and what they follow:
  canonicalize_segment_ids   src/modeling/rotary.py:13-50
  allowed_mask               src/modeling/attention.py:67-97
  segment_block_summary      src/kernels/efficient_attention.py:313-323
  block_summaries            src/kernels/efficient_attention.py:352-365
  summary_should_run         src/kernels/efficient_attention.py:377-412
  vanilla_attention          src/modeling/attention.py:100-148 (dtype steps exact)
  vanilla_attention_vjp      autograd of the above, as jax.vjp would give
  efficient_lse              src/kernels/efficient_attention.py:586-591, :746-760, :906-907
  efficient_backward         src/kernels/efficient_attention.py:1015-1048, :1170-1173,
                             :1294-1343, :1735-1738, :1774
  attention_f64              float64 evaluation of the same mathematics, for error budgets
  segment_sampled_rows       the same analytic forward/backward (:586-591, :746-760, :1015-1048,
                             :1294-1343, :1735-1738) restricted to sampled rows of one long
                             segment, evaluated in query chunks so that segments of tens of
                             thousands of positions fit in memory; pinned against
                             efficient_forward / efficient_backward on short segments
  attention_end_from_blocks  src/data/maskgit.py:106, :116
"""

from __future__ import annotations

import numpy as np
import torch

INT32_MAX = np.iinfo(np.int32).max


# --------------------------------------------------------------------------
# integer side: ids, mask, summaries
# --------------------------------------------------------------------------
def canonicalize_segment_ids(attention_mask, segment_ids=None) -> np.ndarray:
    valid = np.asarray(attention_mask).astype(bool)
    if valid.ndim != 2:
        raise ValueError(f"attention_mask must have shape [batch, sequence], got {valid.shape}")
    if segment_ids is None:
        labels = np.zeros(valid.shape, dtype=np.int32)
    else:
        labels = np.asarray(segment_ids).astype(np.int32)
        if labels.shape != valid.shape:
            raise ValueError(f"segment_ids must have shape {valid.shape}, got {labels.shape}")
    previous_valid = np.concatenate((np.zeros((valid.shape[0], 1), bool), valid[:, :-1]), axis=1)
    previous_labels = np.concatenate((labels[:, :1], labels[:, :-1]), axis=1)
    starts = valid & (~previous_valid | (labels != previous_labels))
    runs = np.cumsum(starts, axis=1, dtype=np.int32)
    return np.where(valid, runs, 0).astype(np.int32)


def allowed_mask(attention_mask, segment_ids, attention_end=None) -> np.ndarray:
    """bool [B, S, S]: allowed[b, q, k]."""

    valid = np.asarray(attention_mask).astype(bool)
    segments = np.asarray(segment_ids).astype(np.int32)
    if segments.shape != valid.shape:
        raise ValueError(f"segment_ids must have shape {valid.shape}, got {segments.shape}")
    sequence = valid.shape[1]
    row = np.arange(sequence)[:, None]
    column = np.arange(sequence)[None, :]
    if attention_end is None:
        causal = np.broadcast_to((column <= row)[None], (valid.shape[0], sequence, sequence))
    else:
        ends = np.asarray(attention_end).astype(np.int32)
        if ends.shape != valid.shape:
            raise ValueError("attention_end must match attention_mask")
        causal = column[None, :, :] <= ends[:, :, None]
    same_segment = segments[:, :, None] == segments[:, None, :]
    non_padding = segments[:, :, None] != 0
    valid_pairs = valid[:, :, None] & valid[:, None, :]
    return causal & same_segment & non_padding & valid_pairs


def allowed_from_canonical(segment_ids, attention_end=None) -> np.ndarray:
    """allowed_mask for canonical ids, where validity is ``id != 0``."""

    segments = np.asarray(segment_ids)
    return allowed_mask(segments != 0, segments, attention_end)


def segment_block_summary(segment_ids, block_size: int) -> np.ndarray:
    segments = np.asarray(segment_ids).astype(np.int32)
    batch, sequence = segments.shape
    blocks = segments.reshape(batch, sequence // block_size, block_size)
    nonzero = blocks != 0
    maximum = np.max(np.where(nonzero, blocks, 0), axis=-1)
    minimum = np.min(np.where(nonzero, blocks, INT32_MAX), axis=-1)
    minimum = np.where(maximum == 0, 0, minimum)
    return np.stack((minimum, maximum), axis=-1).astype(np.int32)


def block_summaries(segment_ids, block_q: int, block_kv: int, attention_end=None):
    """(q_summary [B, S/bq, 2 or 3], kv_summary [B, S/bkv, 2])."""

    segments = np.asarray(segment_ids).astype(np.int32)
    q_summary = segment_block_summary(segments, block_q)
    kv_summary = segment_block_summary(segments, block_kv)
    if attention_end is not None:
        ends = np.where(segments != 0, np.asarray(attention_end).astype(np.int32), 0)
        maximum = ends.reshape(segments.shape[0], -1, block_q).max(axis=-1)
        q_summary = np.concatenate((q_summary, maximum[..., None]), axis=-1)
    return q_summary, kv_summary


def summary_should_run(q_summary, kv_summary, batch, q_block, kv_block, *, block_q, block_kv,
                       q_offset: int = 0) -> bool:
    hybrid = q_summary.shape[-1] == 3
    q_min, q_max = int(q_summary[batch, q_block, 0]), int(q_summary[batch, q_block, 1])
    kv_min, kv_max = int(kv_summary[batch, kv_block, 0]), int(kv_summary[batch, kv_block, 1])
    overlap = q_min != 0 and kv_min != 0 and max(q_min, kv_min) <= min(q_max, kv_max)
    q_global_end = q_offset + (q_block + 1) * block_q - 1
    if hybrid:
        q_global_end = int(q_summary[batch, q_block, 2])
    return bool(overlap and kv_block * block_kv <= q_global_end)


def attention_end_from_blocks(sequence: int, blocks) -> np.ndarray:
    """``end[q] = q`` except inside a bidirectional block [start, stop): ``stop - 1``."""

    end = np.arange(sequence, dtype=np.int32)
    for start, stop in blocks:
        end[start:stop] = stop - 1
    return end


def count_allowed_pairs(segment_ids, attention_end=None) -> int:
    return int(allowed_from_canonical(segment_ids, attention_end).sum())


# --------------------------------------------------------------------------
# floating-point side
# --------------------------------------------------------------------------
def _bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16)


def _expand_kv(x: torch.Tensor, groups: int) -> torch.Tensor:
    # [B, S, Hkv, D] -> [B, S, Hq, D], query head h reads kv head h // groups
    return x.repeat_interleave(groups, dim=2)


def _bf16_dot(a: torch.Tensor, b: torch.Tensor, equation: str) -> torch.Tensor:
    """A bf16 x bf16 contraction whose result dtype is bf16: products are exact in f32,
    accumulation is f32, one rounding to bf16 at the end."""

    return _bf16(torch.einsum(equation, a.float(), b.float()))


class _Bf16Dot(torch.autograd.Function):
    """einsum on bf16 operands with bf16 result and bf16 cotangents (jnp.einsum on bf16)."""

    @staticmethod
    def forward(ctx, a, b, equation):
        ctx.save_for_backward(a, b)
        ctx.equation = equation
        return _bf16_dot(a, b, equation)

    @staticmethod
    def backward(ctx, grad):
        a, b = ctx.saved_tensors
        lhs, out = ctx.equation.split("->")
        ia, ib = lhs.split(",")
        grad = _bf16(grad)
        da = _bf16_dot(grad, b, f"{out},{ib}->{ia}")
        db = _bf16_dot(grad, a, f"{out},{ia}->{ib}")
        return da, db, None


def vanilla_attention(query, key, value, allowed, *, scale: float) -> torch.Tensor:
    """bf16 [B, S, Hq, D] -> bf16 [B, S, Hq, D]; differentiable (torch autograd).

    ``allowed``: bool [B, S, S] (or [B, 1, S, S]).
    """

    if query.dtype != torch.bfloat16 or key.dtype != torch.bfloat16 or value.dtype != torch.bfloat16:
        raise TypeError("vanilla_attention restates the bf16 path")
    batch, q_len, q_heads, _ = query.shape
    kv_heads = key.shape[2]
    groups = q_heads // kv_heads
    allowed = torch.as_tensor(np.asarray(allowed)) if not torch.is_tensor(allowed) else allowed
    if allowed.ndim == 4:
        allowed = allowed[:, 0]
    allowed = allowed.bool()[:, None, :, :]  # [B, 1, Sq, Sk]

    scaled = query * torch.tensor(scale, dtype=torch.bfloat16)      # bf16 multiply
    keys = _expand_kv(key, groups)
    values = _expand_kv(value, groups)
    scores = _Bf16Dot.apply(scaled, keys, "bqhd,bkhd->bhqk").float()  # rounded to bf16, then f32
    minimum = torch.finfo(torch.float32).min
    probabilities = torch.softmax(torch.where(allowed, scores, minimum), dim=-1)
    probabilities = torch.where(allowed.any(dim=-1, keepdim=True), probabilities, 0.0)
    probabilities = _bf16(probabilities)
    return _Bf16Dot.apply(probabilities, values, "bhqk,bkhd->bqhd")


def vanilla_attention_vjp(query, key, value, allowed, dout, *, scale: float):
    """(out, dq, dk, dv) of vanilla_attention for cotangent ``dout`` (bf16)."""

    q = query.detach().clone().requires_grad_(True)
    k = key.detach().clone().requires_grad_(True)
    v = value.detach().clone().requires_grad_(True)
    out = vanilla_attention(q, k, v, allowed, scale=scale)
    out.backward(dout.to(out.dtype))
    return out.detach(), q.grad, k.grad, v.grad


def _scaled_query_f32(query: torch.Tensor, scale: float) -> torch.Tensor:
    return (query * torch.tensor(scale, dtype=torch.bfloat16)).float()


def efficient_scores(query, key, *, scale: float) -> torch.Tensor:
    """f32 scores [B, Hq, S, S] from bf16(q * bf16(scale)) and bf16 k, f32 accumulation."""

    groups = query.shape[2] // key.shape[2]
    return torch.einsum("bqhd,bkhd->bhqk", _scaled_query_f32(query, scale),
                        _expand_kv(key, groups).float())


def efficient_lse(query, key, allowed, *, scale: float) -> torch.Tensor:
    """f32 [B, S, Hq]: natural-log logsumexp of the scaled scores over allowed keys, 0 where none."""

    allowed_t = torch.as_tensor(np.asarray(allowed)).bool()[:, None, :, :]
    scores = efficient_scores(query, key, scale=scale)
    masked = torch.where(allowed_t, scores, float("-inf"))
    row_max = masked.amax(dim=-1)
    has = torch.isfinite(row_max)
    safe_max = torch.where(has, row_max, 0.0)
    total = torch.exp(masked - safe_max[..., None]).sum(dim=-1)
    lse = torch.where(has, torch.log(torch.where(has, total, 1.0)) + safe_max, 0.0)
    return lse.permute(0, 2, 1).contiguous()


def efficient_forward(query, key, value, allowed, *, scale: float):
    """(O bf16, LSE f32) the way the reference kernel computes them (f32 P, f32 PV)."""

    groups = query.shape[2] // key.shape[2]
    allowed_t = torch.as_tensor(np.asarray(allowed)).bool()[:, None, :, :]
    scores = efficient_scores(query, key, scale=scale)
    lse = efficient_lse(query, key, allowed, scale=scale)
    prob = torch.where(allowed_t, torch.exp(scores - lse.permute(0, 2, 1)[..., None]), 0.0)
    out = torch.einsum("bhqk,bkhd->bqhd", prob, _expand_kv(value, groups).float())
    return _bf16(out), lse


def efficient_backward(query, key, value, allowed, out, lse, dout, *, scale: float):
    """(dq, dk, dv) bf16 following the reference kernel's analytic backward."""

    batch, seq, q_heads, dim = query.shape
    kv_heads = key.shape[2]
    groups = q_heads // kv_heads
    allowed_t = torch.as_tensor(np.asarray(allowed)).bool()[:, None, :, :]
    qs = _scaled_query_f32(query, scale)
    kf = _expand_kv(key, groups).float()
    vf = _expand_kv(value, groups).float()
    do = dout.float()
    delta = (out.float() * do).sum(dim=-1)                                   # [B, S, Hq]
    scores = torch.einsum("bqhd,bkhd->bhqk", qs, kf)
    prob = torch.where(allowed_t, torch.exp(scores - lse.permute(0, 2, 1)[..., None]), 0.0)
    dprob = torch.einsum("bqhd,bkhd->bhqk", do, vf)
    dscore = prob * (dprob - delta.permute(0, 2, 1)[..., None])
    scale_f32 = float(torch.tensor(scale, dtype=torch.bfloat16).float())
    dq = torch.einsum("bhqk,bkhd->bqhd", dscore, kf) * scale_f32
    dk_full = torch.einsum("bhqk,bqhd->bkhd", dscore, qs)
    dv_full = torch.einsum("bhqk,bqhd->bkhd", prob, do)
    dk = dk_full.reshape(batch, seq, kv_heads, groups, dim).sum(dim=3)
    dv = dv_full.reshape(batch, seq, kv_heads, groups, dim).sum(dim=3)
    return _bf16(dq), _bf16(dk), _bf16(dv)


def attention_f64(query, key, value, allowed, *, scale: float, dout=None):
    """float64 attention from the bf16 inputs: (O, LSE) or (O, LSE, dq, dk, dv).

    The scale is the bf16-rounded one but the product q*scale is NOT rounded:
    this is the mathematical function the kernels approximate.
    """

    groups = query.shape[2] // key.shape[2]
    batch, seq, q_heads, dim = query.shape
    kv_heads = key.shape[2]
    allowed_t = torch.as_tensor(np.asarray(allowed)).bool()[:, None, :, :]
    scale64 = float(torch.tensor(scale, dtype=torch.bfloat16).double())
    q = query.double()
    k = _expand_kv(key, groups).double()
    v = _expand_kv(value, groups).double()
    scores = torch.einsum("bqhd,bkhd->bhqk", q, k) * scale64
    masked = torch.where(allowed_t, scores, float("-inf"))
    row_max = masked.amax(dim=-1, keepdim=True)
    has = torch.isfinite(row_max)
    safe_max = torch.where(has, row_max, 0.0)
    expd = torch.exp(masked - safe_max)
    total = expd.sum(dim=-1, keepdim=True)
    prob = torch.where(has, expd / torch.where(has, total, 1.0), 0.0)
    lse = torch.where(has, torch.log(torch.where(has, total, 1.0)) + safe_max, 0.0)[..., 0]
    out = torch.einsum("bhqk,bkhd->bqhd", prob, v)
    lse = lse.permute(0, 2, 1).contiguous()
    if dout is None:
        return out, lse
    do = dout.double()
    delta = (out * do).sum(dim=-1)
    dprob = torch.einsum("bqhd,bkhd->bhqk", do, v)
    dscore = prob * (dprob - delta.permute(0, 2, 1)[..., None])
    dq = torch.einsum("bhqk,bkhd->bqhd", dscore, k) * scale64
    dk = (torch.einsum("bhqk,bqhd->bkhd", dscore, q) * scale64)
    dv = torch.einsum("bhqk,bqhd->bkhd", prob, do)
    dk = dk.reshape(batch, seq, kv_heads, groups, dim).sum(dim=3)
    dv = dv.reshape(batch, seq, kv_heads, groups, dim).sum(dim=3)
    return out, lse, dq, dk, dv


def segment_sampled_rows(query, key, value, dout, ends, *, scale: float, query_rows, key_rows,
                         chunk: int = 2048):
    """Sampled rows of one segment of length L that shares one KV head.

    ``query`` / ``dout``: bf16 [L, G, D] (the G query heads of the KV head); ``key`` / ``value``:
    bf16 [L, D]; ``ends``: int [L], last visible key of each query (``arange(L)`` for plain
    causal), positions relative to the segment. Every position belongs to the segment.

    Returns (out [Rq, G, D] f32, lse [Rq, G] f32, dq [Rq, G, D] f32, dk [Rk, D] f32,
    dv [Rk, D] f32) for the query positions ``query_rows`` and key positions ``key_rows``,
    following the reference kernel's analytic backward: delta from the bf16-rounded output,
    f32 scores from bf16(q * bf16(scale)), natural-log LSE. dK / dV need every query of the
    segment, so the whole forward is evaluated, chunk by chunk.
    """

    length, groups, dim = query.shape
    qs = _scaled_query_f32(query, scale)                      # [L, G, D]
    kf, vf, do = key.float(), value.float(), dout.float()
    ends_t = torch.as_tensor(np.asarray(ends)).long()
    query_rows = torch.as_tensor(np.asarray(query_rows)).long()
    key_rows = torch.as_tensor(np.asarray(key_rows)).long()
    scale_f32 = float(torch.tensor(scale, dtype=torch.bfloat16).float())
    out_rows = torch.zeros((len(query_rows), groups, dim))
    lse_rows = torch.zeros((len(query_rows), groups))
    dq_rows = torch.zeros((len(query_rows), groups, dim))
    dk_rows = torch.zeros((len(key_rows), dim))
    dv_rows = torch.zeros((len(key_rows), dim))
    k_sel, v_sel = kf[key_rows], vf[key_rows]
    for start in range(0, length, chunk):
        stop = min(length, start + chunk)
        reach = int(ends_t[start:stop].max()) + 1             # keys any query of the chunk can see
        visible = torch.arange(reach)[None, :] <= ends_t[start:stop, None]          # [c, reach]
        in_chunk = (query_rows >= start) & (query_rows < stop)
        local = query_rows[in_chunk] - start
        sel_visible = key_rows[None, :] <= ends_t[start:stop, None]                  # [c, Rk]
        for head in range(groups):
            scores = qs[start:stop, head] @ kf[:reach].T                             # [c, reach]
            masked = torch.where(visible, scores, float("-inf"))
            row_max = masked.amax(dim=-1, keepdim=True)
            total = torch.exp(masked - row_max).sum(dim=-1, keepdim=True)
            lse = torch.log(total) + row_max                                          # [c, 1]
            prob = torch.exp(masked - lse)                                            # 0 where masked
            out = prob @ vf[:reach]                                                   # [c, D]
            delta = (_bf16(out).float() * do[start:stop, head]).sum(dim=-1, keepdim=True)
            if len(local):
                p_rows = prob[local]
                dprob = do[start:stop, head][local] @ vf[:reach].T
                dscore = p_rows * (dprob - delta[local])
                out_rows[in_chunk, head] = out[local]
                lse_rows[in_chunk, head] = lse[local, 0]
                dq_rows[in_chunk, head] = (dscore @ kf[:reach]) * scale_f32
            # sampled key columns, every query of the chunk
            p_cols = torch.where(sel_visible, torch.exp(qs[start:stop, head] @ k_sel.T - lse), 0.0)
            ds_cols = p_cols * (do[start:stop, head] @ v_sel.T - delta)
            dv_rows += p_cols.T @ do[start:stop, head]
            dk_rows += ds_cols.T @ qs[start:stop, head]
    return out_rows, lse_rows, dq_rows, dk_rows, dv_rows


def relative_l2(actual, expected) -> float:
    a = torch.as_tensor(actual).double().flatten()
    e = torch.as_tensor(expected).double().flatten()
    denom = float(torch.linalg.norm(e))
    return float(torch.linalg.norm(a - e)) / (denom if denom > 0 else 1.0)
