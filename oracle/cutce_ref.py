"""CPU oracle for the cut cross-entropy hot path. TEST INFRASTRUCTURE ONLY.

Imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
bench.py, and by nothing else: the product never calls it.

The reference (JAX) cannot be imported in this environment, so parity is
anchored on this restatement, pinned by tests/test_oracle_cutce.py against
  * the reference's closed forms (zero hidden => nll = sum(w) * log V),
  * the known answers of its shifted-target tests,
  * torch.nn.functional.cross_entropy / log_softmax and autograd,
  * the per-row identity sum_v dlogits = 0.
Citations are relative to the reference root; "src/" = src/causal_trainer/.

Functions and what they follow:
  shifted_targets_and_weights   src/training/losses.py:21-85
  mean_loss                     src/training/losses.py:234-237
  compact_active_rows           src/kernels/cut_cross_entropy.py:673-694
  cut_forward                   src/kernels/cut_cross_entropy.py:85-156, :474-521
  cut_backward                  src/kernels/cut_cross_entropy.py:225-278, :349-403, :597-667
  chunked_cut_forward / chunked_cut_backward
                                src/kernels/cut_cross_entropy.py:697-825 on a one-device mesh
  xla_sparse_cross_entropy(+vjp)  src/kernels/fused_cross_entropy.py:64-109
  cut_f64                       float64 evaluation of the same mathematics
"""

from __future__ import annotations

import numpy as np
import torch

from .attention_ref import canonicalize_segment_ids


def shifted_targets_and_weights(input_ids, attention_mask, segment_ids=None, assistant_mask=None,
                                loss_mask=None, labels=None, *, ignore_index: int = -100):
    tokens = np.asarray(input_ids).astype(np.int32)
    if tokens.ndim != 2:
        raise ValueError(f"input_ids must have shape [batch, sequence], got {tokens.shape}")
    labels = tokens if labels is None else np.asarray(labels).astype(np.int32)
    valid_tokens = (np.ones(tokens.shape, bool) if attention_mask is None
                    else np.asarray(attention_mask) == 1)
    targets = labels[:, 1:]
    valid = valid_tokens[:, :-1] & valid_tokens[:, 1:] & (targets != ignore_index)
    if segment_ids is not None:
        segments = canonicalize_segment_ids(valid_tokens, np.asarray(segment_ids))
        valid &= (segments[:, :-1] == segments[:, 1:]) & (segments[:, 1:] != 0)
    weights = valid.astype(np.float32)
    if assistant_mask is not None:
        weights = weights * (np.asarray(assistant_mask) != 0)[:, 1:].astype(np.float32)
    if loss_mask is not None:
        weights = weights * np.asarray(loss_mask, dtype=np.float32)[:, 1:]
    safe_targets = np.where(weights > 0.0, targets, 0).astype(np.int32)
    return safe_targets, weights.astype(np.float32)


def mean_loss(nll_sum, weight_sum):
    return nll_sum / max(float(weight_sum), 1.0)


def compact_active_rows(hidden, targets, weights):
    """Stable fixed-shape gather: active rows first; returns the reference's 5-tuple."""

    weights = torch.as_tensor(weights)
    rows = weights.shape[0]
    active = weights != 0
    nonzero = torch.nonzero(active).flatten()
    indices = torch.zeros(rows, dtype=torch.long)
    indices[: nonzero.numel()] = nonzero
    slot_valid = torch.arange(rows) < nonzero.numel()
    compact_hidden = hidden[indices]
    compact_targets = torch.where(slot_valid, torch.as_tensor(targets)[indices], 0)
    compact_weights = torch.where(slot_valid, weights[indices], 0.0)
    return compact_hidden, compact_targets, compact_weights, indices, slot_valid


def _logits_f32(hidden, head):
    # bf16 x bf16 products are exact in f32; accumulation in f32.
    return hidden.float() @ head.float()


def cut_forward(hidden, head, targets, weights):
    """(nll_sum f32, weight_sum f32, lse f32 [N]) for hidden [N, d], head [d, V]."""

    targets = torch.as_tensor(targets).long()
    weights = torch.as_tensor(weights).float()
    logits = _logits_f32(hidden, head)
    valid = weights != 0
    vocab = logits.shape[1]
    lse = torch.where(valid, torch.logsumexp(logits, dim=-1), 0.0)
    in_range = (targets >= 0) & (targets < vocab)
    gathered = logits.gather(1, targets.clamp(0, vocab - 1)[:, None])[:, 0]
    target_logit = torch.where(in_range, gathered, 0.0)
    losses = torch.where(valid, weights * (lse - target_logit), 0.0)
    return losses.sum(dtype=torch.float32), weights.sum(dtype=torch.float32), lse


def cut_backward(hidden, head, targets, weights, lse, dy: float, *, head_trainable: bool = True):
    """(dhidden bf16 [N, d], dhead bf16 [d, V] or None). G is rounded to bf16 before both products."""

    targets = torch.as_tensor(targets).long()
    weights = torch.as_tensor(weights).float()
    logits = _logits_f32(hidden, head)
    valid = (weights != 0)[:, None]
    vocab = logits.shape[1]
    prob = torch.where(valid, torch.exp(logits - lse[:, None]), 0.0)
    onehot = torch.zeros_like(prob)
    in_range = (targets >= 0) & (targets < vocab) & (weights != 0)
    rows = torch.nonzero(in_range).flatten()
    onehot[rows, targets[rows]] = 1.0
    g = ((weights * float(dy))[:, None] * (prob - onehot)).to(torch.bfloat16)
    dhidden = (g.float() @ head.float().T).to(hidden.dtype)
    dhead = (hidden.float().T @ g.float()).to(head.dtype) if head_trainable else None
    return dhidden, dhead


def _row_chunks(rows: int, chunk_size: int):
    """Row ranges of the zero-padded chunk grid (cut_cross_entropy.py:697-708)."""

    if chunk_size <= 0:
        raise ValueError("chunk_size must be positive")
    return [(start, min(start + chunk_size, rows)) for start in range(0, rows, chunk_size)]


def chunked_cut_forward(hidden, head, targets, weights, chunk_size: int, *, sparse_compaction: bool = False):
    """The row-chunk loop of the reference without a vocabulary axis (:723-741).

    Every chunk is padded to chunk_size with zero-weight rows, optionally compacted on its own,
    and adds its (nll, weight) to f32 running totals in chunk order. Returns the totals and
    the per-row lse (padding rows dropped, in original row order).
    """

    targets = torch.as_tensor(targets)
    weights = torch.as_tensor(weights).float()
    rows = hidden.shape[0]
    nll_total = torch.zeros((), dtype=torch.float32)
    weight_total = torch.zeros((), dtype=torch.float32)
    lse_rows = torch.zeros(rows, dtype=torch.float32)
    for start, stop in _row_chunks(rows, chunk_size):
        pad = chunk_size - (stop - start)
        h = torch.cat([hidden[start:stop], hidden.new_zeros(pad, hidden.shape[1])])
        t = torch.cat([targets[start:stop], targets.new_zeros(pad)])
        w = torch.cat([weights[start:stop], weights.new_zeros(pad)])
        if sparse_compaction:
            h, t, w, indices, slot_valid = compact_active_rows(h, t, w)
        nll, weight, lse = cut_forward(h, head, t, w)
        nll_total = nll_total + nll
        weight_total = weight_total + weight
        if sparse_compaction:
            full = torch.zeros(chunk_size, dtype=torch.float32)
            full[indices[slot_valid]] = lse[slot_valid]
            lse = full
        lse_rows[start:stop] = lse[: stop - start]
    return nll_total, weight_total, lse_rows


def chunked_cut_backward(hidden, head, targets, weights, lse, dy: float, chunk_size: int, *,
                         head_trainable: bool = True):
    """Backward of the chunk loop (:767-822): dHidden per chunk from f32 products rounded once;
    dHead added up in f32 over the chunks and rounded once at the end."""

    targets = torch.as_tensor(targets).long()
    weights = torch.as_tensor(weights).float()
    rows = hidden.shape[0]
    dhidden = torch.zeros_like(hidden)
    dhead_acc = torch.zeros(head.shape, dtype=torch.float32) if head_trainable else None
    vocab = head.shape[1]
    for start, stop in _row_chunks(rows, chunk_size):
        h, t, w = hidden[start:stop], targets[start:stop], weights[start:stop]
        logits = _logits_f32(h, head)
        valid = (w != 0)[:, None]
        prob = torch.where(valid, torch.exp(logits - lse[start:stop, None]), 0.0)
        onehot = torch.zeros_like(prob)
        hit = torch.nonzero((t >= 0) & (t < vocab) & (w != 0)).flatten()
        onehot[hit, t[hit]] = 1.0
        g = ((w * float(dy))[:, None] * (prob - onehot)).to(torch.bfloat16)
        dhidden[start:stop] = (g.float() @ head.float().T).to(hidden.dtype)
        if head_trainable:
            dhead_acc += h.float().T @ g.float()
    return dhidden, (dhead_acc.to(head.dtype) if head_trainable else None)


def xla_sparse_cross_entropy(logits, targets, weights):
    """Per-row weighted CE on materialised logits, differentiable via torch autograd."""

    compute = logits.float()
    log_normalizer = torch.logsumexp(compute, dim=-1)
    target_logits = compute.gather(-1, torch.as_tensor(targets).long()[..., None])[..., 0]
    return ((log_normalizer - target_logits) * torch.as_tensor(weights).float()).float()


def xla_sparse_cross_entropy_vjp(logits, targets, weights, cotangent):
    """Analytic logits cotangent: (softmax - onehot) * w * dy, cast to the logits dtype."""

    compute = logits.float()
    log_normalizer = torch.logsumexp(compute, dim=-1)
    prob = torch.exp(compute - log_normalizer[..., None])
    onehot = torch.nn.functional.one_hot(torch.as_tensor(targets).long(), logits.shape[-1]).float()
    factor = (torch.as_tensor(weights).float() * torch.as_tensor(cotangent).float())[..., None]
    return ((prob - onehot) * factor).to(logits.dtype)


def pallas_sparse_cross_entropy(logits, targets, weights, *, ignore_index: int = -100):
    """(loss, lse) per row as the streaming kernel defines them (src/causal_trainer/kernels/
    cross_entropy.py:99-190, :400-420): rows with target == ignore_index or weight == 0 give 0 for
    both; on the other rows a target outside the vocabulary contributes a target logit of 0."""

    compute = logits.float()
    targets = torch.as_tensor(targets).long()
    weights = torch.as_tensor(weights).float()
    valid = (targets != ignore_index) & (weights != 0)
    lse = torch.logsumexp(compute, dim=-1)
    inside = (targets >= 0) & (targets < logits.shape[-1])
    picked = compute.gather(-1, targets.clamp(0, logits.shape[-1] - 1)[..., None])[..., 0]
    target_logit = torch.where(inside, picked, torch.zeros_like(picked))
    zero = torch.zeros_like(lse)
    return torch.where(valid, weights * (lse - target_logit), zero), torch.where(valid, lse, zero)


def pallas_sparse_cross_entropy_vjp(logits, targets, weights, cotangent, *, ignore_index: int = -100):
    """Logits cotangent of the streaming kernel (cross_entropy.py:254-323), in the logits dtype."""

    compute = logits.float()
    targets = torch.as_tensor(targets).long()
    weights = torch.as_tensor(weights).float()
    valid = (targets != ignore_index) & (weights != 0)
    lse = torch.logsumexp(compute, dim=-1)
    prob = torch.exp(compute - lse[..., None])
    columns = torch.arange(logits.shape[-1])
    comparable = torch.where((targets >= 0) & (targets < logits.shape[-1]), targets, torch.full_like(targets, -1))
    onehot = (columns == comparable[..., None]).float()
    factor = torch.where(valid, weights * torch.as_tensor(cotangent).float(), torch.zeros_like(weights))
    return (factor[..., None] * torch.where(valid[..., None], prob - onehot, torch.zeros_like(prob))).to(logits.dtype)


def full_logits_loss_and_grads(hidden, head, targets, weights, dy: float):
    """The reference's pure path: materialise f32 logits, sparse CE, autograd to hidden / head."""

    h = hidden.detach().clone().requires_grad_(True)
    w = head.detach().clone().requires_grad_(True)
    logits = (h.float() @ w.float())
    safe_targets = torch.as_tensor(targets).long().clamp(0, head.shape[1] - 1)
    losses = xla_sparse_cross_entropy(logits, safe_targets, weights)
    nll = losses.sum()
    (nll * dy).backward()
    return nll.detach(), h.grad, w.grad


def cut_f64(hidden, head, targets, weights, dy: float):
    """float64 (nll_sum, weight_sum, lse, dhidden, dhead) from the bf16 inputs, no intermediate rounding."""

    targets = torch.as_tensor(targets).long()
    weights64 = torch.as_tensor(weights).double()
    logits = hidden.double() @ head.double()
    valid = weights64 != 0
    vocab = logits.shape[1]
    lse = torch.where(valid, torch.logsumexp(logits, dim=-1), 0.0)
    in_range = (targets >= 0) & (targets < vocab)
    gathered = logits.gather(1, targets.clamp(0, vocab - 1)[:, None])[:, 0]
    target_logit = torch.where(in_range, gathered, 0.0)
    nll = torch.where(valid, weights64 * (lse - target_logit), 0.0).sum()
    prob = torch.where(valid[:, None], torch.exp(logits - lse[:, None]), 0.0)
    onehot = torch.zeros_like(prob)
    rows = torch.nonzero(in_range & valid).flatten()
    onehot[rows, targets[rows]] = 1.0
    g = (weights64 * dy)[:, None] * (prob - onehot)
    return nll, weights64.sum(), lse, g @ head.double().T, hidden.double().T @ g
