"""Seeded synthetic inputs of the benchmark shapes, and their FLOP / byte accounting.

Inputs are drawn on the host with ``numpy.random.default_rng(seed)`` and cast
to bf16 with round-to-nearest-even. Segment layouts follow the five named
configurations: packed documents with a tail of padding (segment id 0), and,
for the MaskGIT configuration, image blocks that are bidirectional inside the
block (expressed as ``attention_end``: the inclusive last visible key of each
query, src/causal_trainer/data/maskgit.py:106, :116 in the reference).
"""

from __future__ import annotations

import dataclasses
import math

import numpy as np
import torch


@dataclasses.dataclass(frozen=True)
class AttentionConfig:
    name: str
    batch: int
    seq: int
    q_heads: int
    kv_heads: int
    head_dim: int
    layout: str          # "uniform", "loguniform", "maskgit"
    min_len: int
    max_len: int
    seed: int

    @property
    def scale(self) -> float:
        return self.head_dim ** -0.5


ATTENTION_CONFIGS = {
    # B=2, S=1024, Hq=Hkv=8, D=64; documents of length U[32, 512]
    "packed_small": AttentionConfig("packed_small", 2, 1024, 8, 8, 64, "uniform", 32, 512, 101),
    # Llama-3-8B shape: B=4, S=4096, Hq=32, Hkv=8, D=128; lengths log-uniform [64, 4096]
    "llama3_8b": AttentionConfig("llama3_8b", 4, 4096, 32, 8, 128, "loguniform", 64, 4096, 202),
    # MaskGIT mixed mask: B=2, S=8192, Hq=Hkv=16, D=128
    "maskgit": AttentionConfig("maskgit", 2, 8192, 16, 16, 128, "maskgit", 0, 0, 404),
    # 70B-layer shape, long context: B=1, S=32768, Hq=64, Hkv=8, D=128; log-uniform [512, 32768]
    "long_70b": AttentionConfig("long_70b", 1, 32768, 64, 8, 128, "loguniform", 512, 32768, 505),
}


def packed_segment_ids(rng, batch: int, seq: int, layout: str, min_len: int, max_len: int):
    """int32 [batch, seq] canonical ids: documents packed from position 0, tail padding = 0."""

    ids = np.zeros((batch, seq), dtype=np.int32)
    for row in range(batch):
        position, segment = 0, 1
        while position < seq:
            if layout == "uniform":
                length = int(rng.integers(min_len, max_len + 1))
            else:
                length = int(round(math.exp(rng.uniform(math.log(min_len), math.log(max_len)))))
            length = max(1, length)
            if position + length > seq:
                # The document does not fit: leave the tail as padding, unless the row
                # would otherwise be empty.
                if position == 0:
                    length = seq
                else:
                    break
            ids[row, position:position + length] = segment
            position += length
            segment += 1
    return ids


def maskgit_layout(rng, batch: int, seq: int):
    """(segment ids, attention_end): causal text plus 1-3 image blocks of 32 x (32 + 1) tokens."""

    image = 32 * 33
    ids = np.zeros((batch, seq), dtype=np.int32)
    end = np.broadcast_to(np.arange(seq, dtype=np.int32), (batch, seq)).copy()
    for row in range(batch):
        position, segment = 0, 1
        while position < seq:
            n_images = int(rng.integers(1, 4))
            pieces = []
            for _ in range(n_images):
                pieces.append(("text", int(rng.integers(16, 257))))
                pieces.append(("image", image))
            pieces.append(("text", int(rng.integers(16, 129))))
            length = sum(size for _, size in pieces)
            if position + length > seq:
                break
            cursor = position
            for kind, size in pieces:
                if kind == "image":
                    end[row, cursor:cursor + size] = cursor + size - 1
                cursor += size
            ids[row, position:position + length] = segment
            position += length
            segment += 1
    return ids, end


def to_bf16(array: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)


def make_attention_inputs(config: AttentionConfig, device="cpu"):
    """dict with q, k, v, dout (bf16), segment_ids, attention_end (int32 or None)."""

    rng = np.random.default_rng(config.seed)
    if config.layout == "maskgit":
        segment_ids, attention_end = maskgit_layout(rng, config.batch, config.seq)
    else:
        segment_ids = packed_segment_ids(rng, config.batch, config.seq, config.layout,
                                         config.min_len, config.max_len)
        attention_end = None
    q_shape = (config.batch, config.seq, config.q_heads, config.head_dim)
    kv_shape = (config.batch, config.seq, config.kv_heads, config.head_dim)

    def normal(shape):
        return to_bf16(rng.standard_normal(shape, dtype=np.float32)).to(device)

    return {
        "q": normal(q_shape),
        "k": normal(kv_shape),
        "v": normal(kv_shape),
        "dout": normal(q_shape),
        "segment_ids": torch.from_numpy(segment_ids).to(device),
        "attention_end": None if attention_end is None else torch.from_numpy(attention_end).to(device),
        "scale": config.scale,
    }


def count_allowed_pairs(segment_ids, attention_end=None) -> int:
    """Exact number of allowed (query, key) pairs, O(B * S log S) on the host.

    allowed(q, k) = k <= end[q] and seg[q] == seg[k] != 0. For each query this is the
    number of positions <= end[q] carrying the query's id, read from per-id sorted
    position lists, so ids need not be contiguous runs.
    """

    segments = np.asarray(torch.as_tensor(segment_ids).cpu()).astype(np.int64)
    batch, seq = segments.shape
    ends = (np.broadcast_to(np.arange(seq), (batch, seq)) if attention_end is None
            else np.asarray(torch.as_tensor(attention_end).cpu()).astype(np.int64))
    total = 0
    for row in range(batch):
        ids = segments[row]
        order = np.argsort(ids, kind="stable")
        sorted_ids = ids[order]
        for value in np.unique(ids):
            if value == 0:
                continue
            lo, hi = np.searchsorted(sorted_ids, value, "left"), np.searchsorted(sorted_ids, value, "right")
            positions = order[lo:hi]            # ascending (stable sort)
            total += int(np.searchsorted(positions, ends[row, positions], "right").sum())
    return total


def attention_flops(config: AttentionConfig, pairs: int) -> dict:
    """Mask-aware algorithmic FLOPs: forward 4*D*Hq*pairs, backward 10*D*Hq*pairs."""

    unit = config.head_dim * config.q_heads * pairs
    return {"fwd": 4 * unit, "bwd": 10 * unit, "total": 14 * unit}


def attention_delta_bytes(config: AttentionConfig) -> int:
    """Bytes of the delta pass: read O and dO (bf16), write delta (f32)."""

    rows = config.batch * config.seq * config.q_heads
    return 2 * rows * config.head_dim * 2 + 4 * rows


@dataclasses.dataclass(frozen=True)
class CutCEConfig:
    name: str
    rows: int
    hidden: int
    vocab: int
    ignore_fraction: float
    seed: int


CUTCE_CONFIGS = {
    # N=16384, d=4096, V=128256, 30% ignored
    "llama3_8b_head": CutCEConfig("llama3_8b_head", 16384, 4096, 128256, 0.30, 303),
}


def make_cutce_inputs(config: CutCEConfig, device="cpu"):
    """hidden [N, d] ~ N(0,1), head [d, V] ~ N(0, 0.02^2) (bf16), targets, weights.

    Labels are uniform in [0, V) with ``ignore_fraction`` of them set to -100; the
    caller-side rule of the reference (src/causal_trainer/training/losses.py:57, :84)
    turns those into weight 0 / target 0.
    """

    rng = np.random.default_rng(config.seed)
    labels = rng.integers(0, config.vocab, size=config.rows, dtype=np.int64).astype(np.int32)
    ignored = rng.random(config.rows) < config.ignore_fraction
    labels[ignored] = -100
    weights = (labels != -100).astype(np.float32)
    targets = np.where(weights > 0, labels, 0).astype(np.int32)
    generator = torch.Generator(device="cpu").manual_seed(config.seed)
    hidden = torch.randn((config.rows, config.hidden), generator=generator).to(torch.bfloat16)
    head = (torch.randn((config.hidden, config.vocab), generator=generator) * 0.02).to(torch.bfloat16)
    return {
        "hidden": hidden.to(device),
        "head": head.to(device),
        "targets": torch.from_numpy(targets).to(device),
        "weights": torch.from_numpy(weights).to(device),
        "labels": torch.from_numpy(labels).to(device),
    }


def cutce_flops(config: CutCEConfig, active_rows: int) -> dict:
    """Algorithmic FLOPs: forward 2*N_act*d*V, backward 4*N_act*d*V."""

    unit = 2 * active_rows * config.hidden * config.vocab
    dense = 2 * config.rows * config.hidden * config.vocab
    return {"fwd": unit, "bwd": 2 * unit, "total": 3 * unit, "dense_total": 3 * dense}
