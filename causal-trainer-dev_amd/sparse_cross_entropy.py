"""Sparse cross-entropy on materialised logits, the trainer's non-fused loss backend.

Mirrors ``pallas_fused_sparse_cross_entropy`` (src/causal_trainer/kernels/cross_entropy.py:600-643;
per-token f32 losses, custom VJP with the analytic logits gradient, rows with target -100 or
weight 0 contribute nothing and are not read) on one MI355X: same name, argument meaning and
shape errors; ``mesh`` is accepted for signature compatibility and must describe one device.
"""

from __future__ import annotations

import torch

from . import _lib

_IGNORE_INDEX = -100
_DTYPES = {torch.bfloat16: 0, torch.float32: 1}


def _args(logits2, targets1, weights1):
    return _lib.SparseCeArgs(logits=logits2.data_ptr(), targets=targets1.data_ptr(), weights=weights1.data_ptr(),
                             rows=logits2.shape[0], vocab=logits2.shape[1], logits_dtype=_DTYPES[logits2.dtype],
                             ignore_index=_IGNORE_INDEX)


class _SparseCE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits2, targets1, weights1):
        rows = logits2.shape[0]
        loss = torch.empty(rows, dtype=torch.float32, device=logits2.device)
        lse = torch.empty_like(loss)
        with torch.cuda.device(logits2.device):
            _lib.check(_lib.load().ct_sparse_ce_fwd(_lib.current_stream(), _args(logits2, targets1, weights1),
                                                    loss.data_ptr(), lse.data_ptr()))
        ctx.save_for_backward(logits2, lse, targets1, weights1)
        return loss

    @staticmethod
    def backward(ctx, dy):
        logits2, lse, targets1, weights1 = ctx.saved_tensors
        dlogits = torch.empty_like(logits2)
        dy = dy.to(torch.float32).contiguous()
        with torch.cuda.device(logits2.device):
            _lib.check(_lib.load().ct_sparse_ce_bwd(_lib.current_stream(), _args(logits2, targets1, weights1),
                                                    lse.data_ptr(), dy.data_ptr(), dlogits.data_ptr()))
        return dlogits, None, None


def pallas_fused_sparse_cross_entropy(logits, targets, weights, *, mesh=None) -> torch.Tensor:
    """Per-token weighted CE ``[batch, sequence]`` (f32) of logits ``[batch, sequence, vocab]``."""

    if logits.ndim != 3 or tuple(targets.shape) != tuple(logits.shape[:-1]) or tuple(weights.shape) != tuple(targets.shape):
        raise ValueError("Pallas CE expects logits [batch, sequence, vocab] and matching target/weight rows")
    if mesh is not None and getattr(mesh, "size", 1) != 1:
        raise ValueError("this build runs on one device: pass mesh=None or a one-device mesh")
    if not logits.is_cuda:
        raise RuntimeError("logits must live on a ROCm GPU")
    if logits.dtype not in _DTYPES:
        raise ValueError("logits must be bfloat16 or float32")
    leading = logits.shape[:-1]
    if logits.numel() == 0:
        return torch.zeros(leading, dtype=torch.float32, device=logits.device)
    flat_logits = logits.reshape(-1, logits.shape[-1]).contiguous()
    flat_targets = targets.reshape(-1).to(device=logits.device, dtype=torch.int32).contiguous()
    flat_weights = weights.reshape(-1).to(device=logits.device, dtype=torch.float32).contiguous()
    return _SparseCE.apply(flat_logits, flat_targets, flat_weights).reshape(leading)


__all__ = ["pallas_fused_sparse_cross_entropy"]
