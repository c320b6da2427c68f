"""Device-side mirrors of the two preparation functions directly in front of the hot paths.

``canonicalize_segment_ids`` (src/causal_trainer/modeling/rotary.py:13-50) and
``shifted_targets_and_weights`` (``_shifted_targets_and_weights``,
src/causal_trainer/training/losses.py:21-85) keep the reference's argument meaning and
validation errors; tensors are torch tensors on a ROCm device and the work is done by
libct_hotpath.so. They define which tokens attention may connect and which rows the loss
ignores, so they are integer kernels that match the reference bit for bit.
"""

from __future__ import annotations

import torch

from . import _lib


def _int32(tensor, name: str, shape=None) -> torch.Tensor:
    tensor = torch.as_tensor(tensor)
    if not tensor.is_cuda:
        raise RuntimeError(f"{name} must live on a ROCm GPU")
    if shape is not None and tuple(tensor.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(tensor.shape)}")
    return tensor.to(torch.int32).contiguous()


def canonicalize_segment_ids(attention_mask, segment_ids=None) -> torch.Tensor:
    """One-based ids of contiguous valid runs, zero for padding (int32 ``[batch, sequence]``)."""

    mask = torch.as_tensor(attention_mask)
    if mask.ndim != 2:
        raise ValueError(f"attention_mask must have shape [batch, sequence], got {tuple(mask.shape)}")
    valid = _int32(mask != 0, "attention_mask")
    labels = None
    if segment_ids is not None:
        labels = torch.as_tensor(segment_ids)
        if tuple(labels.shape) != tuple(valid.shape):
            raise ValueError(f"segment_ids must have shape {tuple(valid.shape)}, got {tuple(labels.shape)}")
        labels = _int32(labels, "segment_ids")
    batch, sequence = valid.shape
    out = torch.empty_like(valid)
    if batch == 0 or sequence == 0:
        return out
    with torch.cuda.device(valid.device):
        _lib.check(_lib.load().ct_canonicalize_segment_ids(
            _lib.current_stream(), valid.data_ptr(), _lib.pointer(labels), batch, sequence, out.data_ptr()))
    return out


def shifted_targets_and_weights(input_ids, attention_mask, segment_ids=None, assistant_mask=None,
                                loss_mask=None, labels=None, *, ignore_index: int = -100):
    """Safe shifted targets (int32) and target-position loss weights (f32), both ``[batch, sequence - 1]``."""

    tokens = torch.as_tensor(input_ids)
    if tokens.ndim != 2:
        raise ValueError(f"input_ids must have shape [batch, sequence], got {tuple(tokens.shape)}")
    tokens = _int32(tokens, "input_ids")
    shape = tokens.shape
    label_t = None if labels is None else _int32(labels, "labels", shape)
    # validity is "mask == 1": other values, True included as 1, follow the reference's comparison
    mask_t = None if attention_mask is None else _int32(attention_mask, "attention_mask", shape)
    segment_t = None if segment_ids is None else _int32(segment_ids, "segment_ids", shape)
    assistant_t = None
    if assistant_mask is not None:
        assistant = torch.as_tensor(assistant_mask)
        if tuple(assistant.shape) != tuple(shape):
            raise ValueError(f"assistant_mask must have shape {tuple(shape)}, got {tuple(assistant.shape)}")
        assistant_t = _int32(assistant != 0, "assistant_mask")
    loss_t = None
    if loss_mask is not None:
        loss_t = torch.as_tensor(loss_mask)
        if tuple(loss_t.shape) != tuple(shape):
            raise ValueError(f"loss_mask must have shape {tuple(shape)}, got {tuple(loss_t.shape)}")
        loss_t = loss_t.to(torch.float32).contiguous()
    batch, sequence = shape
    if sequence < 2:
        raise ValueError("input_ids needs at least two positions to form a prediction edge")
    lib = _lib.load()
    targets = torch.empty((batch, sequence - 1), dtype=torch.int32, device=tokens.device)
    weights = torch.empty((batch, sequence - 1), dtype=torch.float32, device=tokens.device)
    scratch = None
    if segment_t is not None:
        if mask_t is None:          # every token valid
            mask_t = torch.ones_like(tokens)
        scratch = torch.empty(lib.ct_shifted_targets_scratch_bytes(batch, sequence), dtype=torch.uint8,
                              device=tokens.device)
    args = _lib.ShiftedTargetsArgs(
        input_ids=tokens.data_ptr(), attention_mask=_lib.pointer(mask_t),
        segment_ids=_lib.pointer(segment_t), assistant_mask=_lib.pointer(assistant_t),
        loss_mask=_lib.pointer(loss_t), labels=_lib.pointer(label_t),
        targets=targets.data_ptr(), weights=weights.data_ptr(),
        scratch=_lib.pointer(scratch), scratch_bytes=0 if scratch is None else scratch.numel(),
        batch=batch, seq=sequence, ignore_index=int(ignore_index),
    )
    with torch.cuda.device(tokens.device):
        _lib.check(lib.ct_shifted_targets_and_weights(_lib.current_stream(), args))
    return targets, weights


__all__ = ["canonicalize_segment_ids", "shifted_targets_and_weights"]
