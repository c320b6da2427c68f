"""Fixed-length sequence packing: the host-side format both hot paths consume.

Mirror of the reference's packing utilities (src/causal_trainer/data/packing.py:105-252, :260-301,
:356-383): same names, argument meaning, output fields and error messages. A packed row is a
dict of equally long per-token lists; ``segment_ids`` (1, 2, ... per contiguous run of valid tokens,
0 on padding) are what the attention operator isolates on and what the shifted loss uses to drop
cross-example targets, so they are always regenerated here and never taken from the input.

This is host code in the reference as well (plain Python over token lists, run once per dataset
batch); columns are handled as NumPy arrays here and converted back to lists at the boundary.
"""

from __future__ import annotations

from collections.abc import Iterable, Mapping, Sequence
from typing import Any

import numpy as np

Scalar = int | float
PackedExample = dict[str, list[Scalar]]

_WEIGHTS = "loss_weights"
_STRICT = ("attention_mask", "position_ids", "segment_ids", "loss_weights", "labels")
_BINARY = ("attention_mask", "assistant_masks", "assistant_mask", "assistant_tokens_mask")


def _column(value: Any, name: str) -> np.ndarray:
    """One per-token field as a 1-D array: float64 for loss weights, int64 otherwise."""

    if hasattr(value, "tolist"):
        value = value.tolist()
    if isinstance(value, tuple):
        value = list(value)
    if not isinstance(value, list) or (value and isinstance(value[0], (list, tuple))):
        raise ValueError(f"Per-token field {name!r} must be a one-dimensional sequence.")
    if name == _WEIGHTS:
        try:
            out = np.array([float(item) for item in value], dtype=np.float64)
        except (TypeError, ValueError) as exc:
            raise ValueError(f"Per-token field {name!r} must contain numbers.") from exc
        if not np.isfinite(out).all():
            raise ValueError(f"Per-token field {name!r} must contain only finite numbers.")
        return out
    try:
        return np.array([int(item) for item in value], dtype=np.int64)
    except (TypeError, ValueError) as exc:
        raise ValueError(f"Per-token field {name!r} must contain integers.") from exc


def _normalized(example: Mapping[str, Any], max_length: int) -> dict[str, np.ndarray]:
    """Validated columns of one example, truncated to max_length (packing.py:49-88)."""

    if "input_ids" not in example:
        raise ValueError("Every example must contain input_ids.")
    tokens = _column(example["input_ids"], "input_ids")
    if min(len(tokens), max_length) <= 0:
        raise ValueError("Cannot pack an empty input_ids sequence.")
    out = {"input_ids": tokens[:max_length]}
    for name, value in example.items():
        if name == "input_ids" or isinstance(value, (str, bytes, Mapping)):
            continue
        try:
            column = _column(value, name)
        except ValueError:
            # fields that are not per-token data are dropped, the known ones must parse
            if name in _STRICT or name.endswith(("_mask", "_masks")):
                raise
            continue
        if len(column) != len(tokens):
            raise ValueError(f"Per-token field {name!r} has length {len(column)}, expected {len(tokens)}.")
        out[name] = column[:max_length]
    out.setdefault("attention_mask", np.ones(len(out["input_ids"]), dtype=np.int64))
    for name in _BINARY:
        if name in out and not np.isin(out[name], (0, 1)).all():
            raise ValueError(f"{name} must contain only binary 0/1 values.")
    if "position_ids" in out and (out["position_ids"] < 0).any():
        raise ValueError("position_ids must be non-negative.")
    if _WEIGHTS in out and (out[_WEIGHTS] < 0.0).any():
        raise ValueError("loss_weights must be non-negative.")
    return out


def _run_metadata(valid: np.ndarray, first_segment: int = 0) -> tuple[np.ndarray, np.ndarray, int]:
    """(position_ids, segment_ids, last id used) of the contiguous runs of valid tokens.

    Every run gets the next segment id after first_segment and positions from 0; invalid
    tokens get 0 / 0 (packing.py:156-184).
    """

    valid = np.asarray(valid) == 1
    starts = valid & ~np.concatenate(([False], valid[:-1]))
    run = np.cumsum(starts)
    segments = np.where(valid, first_segment + run, 0)
    index = np.arange(len(valid))
    run_start = np.maximum.accumulate(np.where(starts, index, 0))
    positions = np.where(valid, index - run_start, 0)
    return positions.astype(np.int64), segments.astype(np.int64), first_segment + int(run[-1] if len(run) else 0)


def _fill(name: str, pad_token_id: int) -> Scalar:
    return int(pad_token_id) if name == "input_ids" else (0.0 if name == _WEIGHTS else 0)


def _padded(columns: Mapping[str, np.ndarray], max_length: int, pad_token_id: int, padding_side: str) -> PackedExample:
    length = len(columns["input_ids"])
    if length > max_length:
        raise ValueError(f"Packed sequence length {length} exceeds max_length {max_length}.")
    out: PackedExample = {}
    for name, column in columns.items():
        if len(column) != length:
            raise ValueError(f"Packed field {name!r} is not aligned with input_ids.")
        fill = [_fill(name, pad_token_id)] * (max_length - length)
        body = column.tolist()
        out[name] = fill + body if padding_side == "left" else body + fill
    return out


def pad_example(example: Mapping[str, Sequence[Scalar]], *, max_length: int, pad_token_id: int,
                padding_side: str = "left") -> PackedExample:
    """Pad an already aligned example to a fixed sequence length (packing.py:187-217)."""

    if max_length <= 0:
        raise ValueError("max_length must be positive.")
    if padding_side not in {"left", "right"}:
        raise ValueError("padding_side must be either 'left' or 'right'.")
    if "input_ids" not in example:
        raise ValueError("example must contain input_ids.")
    return _padded({name: _column(value, name) for name, value in example.items()}, max_length, pad_token_id,
                   padding_side)


def best_fit_decreasing(examples: Sequence[Mapping[str, Any]], *, max_length: int) -> list[list[Mapping[str, Any]]]:
    """Deterministic best-fit decreasing (packing.py:105-145): longest first (ties in input order),
    each into the open row it fills most tightly (ties to the oldest row), else a new row."""

    if max_length <= 0:
        raise ValueError("max_length must be positive.")
    lengths = np.array([len(example["input_ids"]) for example in examples], dtype=np.int64)
    rows: list[list[Mapping[str, Any]]] = []
    free = np.empty(0, dtype=np.int64)
    for index in np.argsort(-lengths, kind="stable"):
        length = int(lengths[index])
        if length > max_length:
            raise ValueError(f"Sequence length {length} exceeds packing max_length {max_length}.")
        slack = np.where(free >= length, free - length, max_length + 1)
        if len(slack) and slack.min() <= max_length:
            chosen = int(slack.argmin())
            rows[chosen].append(examples[index])
            free[chosen] -= length
        else:
            rows.append([examples[index]])
            free = np.append(free, max_length - length)
    return rows


def _packed_row(members: Sequence[Mapping[str, np.ndarray]], fields: Sequence[str], max_length: int,
                pad_token_id: int, padding_side: str) -> PackedExample:
    columns = {name: np.concatenate([member[name] for member in members]) for name in fields}
    positions, segments, last = [], [], 0
    for member in members:
        member_positions, member_segments, last = _run_metadata(member["attention_mask"], last)
        positions.append(member_positions)
        segments.append(member_segments)
    # explicit position ids survive (terminal anchors use a non-contiguous range); segment ids never do
    if "position_ids" not in columns:
        columns["position_ids"] = np.concatenate(positions)
    columns["segment_ids"] = np.concatenate(segments)
    return _padded(columns, max_length, pad_token_id, padding_side)


def pack_examples(examples: Iterable[Mapping[str, Any]], *, max_length: int, pad_token_id: int,
                  packing_batch_size: int = 1000, padding_side: str = "left") -> list[PackedExample]:
    """Pack examples in independent best-fit-decreasing batches and pad every row (packing.py:260-301).

    No token is inserted between examples; isolation rests on ``segment_ids`` alone.
    """

    if max_length <= 0:
        raise ValueError("max_length must be positive.")
    if packing_batch_size <= 0:
        raise ValueError("packing_batch_size must be positive.")
    if padding_side not in {"left", "right"}:
        raise ValueError("padding_side must be either 'left' or 'right'.")
    out: list[PackedExample] = []
    batch: list[dict[str, np.ndarray]] = []

    def flush() -> None:
        names = set(batch[0])
        for index, member in enumerate(batch[1:], start=1):
            if set(member) != names:
                raise ValueError(
                    "All examples in a packing batch must have the same per-token fields; "
                    f"example {index} is missing {sorted(names - set(member))} and adds {sorted(set(member) - names)}."
                )
        fields = [name for name in batch[0] if name != "segment_ids"]
        for members in best_fit_decreasing(batch, max_length=max_length):
            out.append(_packed_row(members, fields, max_length, pad_token_id, padding_side))
        batch.clear()

    for example in examples:
        batch.append(_normalized(example, max_length))
        if len(batch) == packing_batch_size:
            flush()
    if batch:
        flush()
    return out


def pad_examples(examples: Iterable[Mapping[str, Any]], *, max_length: int, pad_token_id: int,
                 padding_side: str = "left") -> list[PackedExample]:
    """Truncate and pad examples without combining independent samples (packing.py:356-383)."""

    if max_length <= 0:
        raise ValueError("max_length must be positive.")
    if padding_side not in {"left", "right"}:
        raise ValueError("padding_side must be either 'left' or 'right'.")
    out = []
    for example in examples:
        columns = _normalized(example, max_length)
        positions, segments, _ = _run_metadata(columns["attention_mask"])
        columns.setdefault("position_ids", positions)
        columns["segment_ids"] = segments
        out.append(_padded(columns, max_length, pad_token_id, padding_side))
    return out


MODEL_FIELDS = ("input_ids", "attention_mask", "position_ids", "segment_ids")


def collate(rows: Sequence[Mapping[str, Sequence[Scalar]]], *, assistant_only_loss: bool = False) -> dict[str, np.ndarray]:
    """Stack packed rows into the [batch, sequence] arrays the operators take.

    The batch layout of the reference (src/causal_trainer/data/batching.py:54-101): the four
    model fields as int32 plus f32 ``loss_weights`` - the rows' own weights when they carry
    them (all rows or none), else the assistant masks when only assistant tokens are trained
    on, else the attention mask.
    """

    if not rows:
        raise ValueError("cannot collate an empty list of rows")
    for index, row in enumerate(rows):
        missing = [name for name in MODEL_FIELDS if name not in row]
        if missing:
            raise ValueError(f"dataset record {index} is missing model fields: {missing}")
    batch = {name: np.asarray([row[name] for row in rows], dtype=np.int32) for name in MODEL_FIELDS}
    weighted = [index for index, row in enumerate(rows) if _WEIGHTS in row]
    if weighted and len(weighted) != len(rows):
        raise ValueError("a batch cannot mix weighted and unweighted training records")
    if assistant_only_loss:
        absent = [index for index, row in enumerate(rows) if "assistant_masks" not in row]
        if absent:
            raise ValueError(f"assistant-masked loss dataset is missing assistant_masks for records {absent}")
    source = _WEIGHTS if weighted else ("assistant_masks" if assistant_only_loss else "attention_mask")
    for index, row in enumerate(rows):
        if len(row[source]) != len(row["input_ids"]):
            raise ValueError(f"dataset record {index} has {source} that are not aligned with input_ids")
    batch[_WEIGHTS] = np.asarray([row[source] for row in rows], dtype=np.float32)
    if not np.isfinite(batch[_WEIGHTS]).all() or (batch[_WEIGHTS] < 0).any():
        raise ValueError("loss_weights must be finite and non-negative")
    return batch


__all__ = ["MODEL_FIELDS", "PackedExample", "Scalar", "best_fit_decreasing", "collate", "pack_examples", "pad_example",
           "pad_examples"]
