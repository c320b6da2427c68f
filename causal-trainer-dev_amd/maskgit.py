"""MaskGIT batch transform: ``attention_end`` and same-position prediction targets for image blocks.

Host-side stage between packing and the two GPU operators (the reference's counterpart is
src/causal_trainer/data/maskgit.py:20-135; class name, constructor, call signature, output
fields and error texts are kept so that a trainer can swap the import). Written from the
behaviour the reference's tests and the reference-derived vectors pin down, as three stages:

1. ``find_blocks``: one pass over a whole batch that fills a ``BlockTable`` (flat arrays) with
   every image grid that sits inside a complete assistant message: batch row, first position,
   one past the last position, the positions of its codes, and whether any code is supervised.
2. ``plan``: the only stage that touches the random stream. For every supervised block, in table
   order: one uniform decides whether the block is selected, and for a selected block a second
   uniform gives the masked share ``cos(pi/2 * u)`` and one ``choice`` without replacement names
   the codes. The generator is ``default_rng(SeedSequence([seed, step]))``, so a batch is masked
   as a function of (seed, optimizer step) only: resume-safe and identical to the reference's.
3. ``apply``: array updates only. Outside selected blocks everything stays next-token
   prediction: target = following token, weight = the following token's loss weight when both
   tokens are valid and in the same run. A selected block becomes bidirectional
   (``attention_end`` = its last position for every position in it), loses every next-token edge
   into, inside and out of it (newlines and the closing delimiter come from the template), and
   each masked code is replaced by ``[MASK]`` and predicts its own original code with its own
   loss weight.

Outputs: ``input_ids`` (masked copy), ``attention_end`` int32 [B, S] (the operand of the attention
operator's hybrid mask), ``prediction_targets`` int32 [B, S] and ``prediction_weights`` f32 [B, S]
(the operands of the cut cross-entropy operator). The input batch is not modified.

The tokenizer is duck-typed: ``get_vocab()``, ``__call__(text)["input_ids"]``, ``decode(ids)`` and
optionally ``pad_token_id``.
"""

from __future__ import annotations

import dataclasses
import math
import re
from collections.abc import Iterator, Mapping

import numpy as np

IMAGE_CODE = re.compile(r"<\|image_[0-9]+\|>")
MASK, OPEN, CLOSE = "[MASK]", "<|im_start|>", "<|im_end|>"
ROLE_PROBE = 32       # tokens after the opening delimiter that are decoded to read the role
ROW_BREAK_LIMIT = 8   # a longer stretch between two codes is never a row break
ROW_BREAKS = ("\n", "\r\n")
ASSISTANT = tuple("assistant" + eol for eol in ROW_BREAKS)


@dataclasses.dataclass
class BlockTable:
    """Image blocks of a batch, in (row, position) order. Block i covers positions
    ``first[i] .. stop[i] - 1`` of row ``row[i]``; its codes sit at
    ``codes[code_begin[i]:code_begin[i + 1]]``."""

    row: np.ndarray
    first: np.ndarray
    stop: np.ndarray
    code_begin: np.ndarray
    codes: np.ndarray
    supervised: np.ndarray

    def __len__(self) -> int:
        return len(self.row)

    def codes_of(self, index: int) -> np.ndarray:
        return self.codes[self.code_begin[index]:self.code_begin[index + 1]]


@dataclasses.dataclass
class MaskPlan:
    """What the random stream decided: selected block indices and the masked positions."""

    selected: np.ndarray      # indices into the BlockTable
    masked_row: np.ndarray    # batch row of every masked code
    masked_col: np.ndarray    # its position


def _vocabulary_ids(tokenizer):
    vocabulary = tokenizer.get_vocab()
    ids = []
    for token in (MASK, OPEN, CLOSE):
        index = vocabulary.get(token)
        if index is None or tokenizer(token)["input_ids"] != [index]:
            raise ValueError(f"MaskGIT requires {token!r} to encode as one token")
        ids.append(index)
    codes = sorted(index for token, index in vocabulary.items() if IMAGE_CODE.fullmatch(token))
    if not codes:
        raise ValueError("MaskGIT requires <|image_i|> tokens in the tokenizer vocabulary")
    table_size = 1 + max(max(vocabulary.values()), getattr(tokenizer, "pad_token_id", None) or 0)
    lookup = np.zeros(table_size, dtype=np.bool_)
    lookup[codes] = True
    return ids, lookup


class MaskGITBatchTransform:
    """Select each complete, supervised assistant image block with probability p and mask a
    cosine-scheduled share of its codes."""

    def __init__(self, tokenizer, *, probability: float, seed: int) -> None:
        if not (math.isfinite(probability) and 0.0 <= probability <= 1.0):
            raise ValueError("maskgit_probability must be between 0 and 1")
        (self.mask_id, self.start_id, self.end_id), self.is_image = _vocabulary_ids(tokenizer)
        self.tokenizer, self.probability, self.seed = tokenizer, probability, seed

    # ---------------------------------------------------------------- stage 1: block table
    def _row_grids(self, tokens: np.ndarray, valid: np.ndarray, segments: np.ndarray):
        """(first, stop, code positions) of the grids of one row, left to right.

        The row is scanned once through its events: where a run of equal (valid, segment) ends,
        where messages open and close, and where codes sit. A message counts when its closing
        delimiter comes before the next opening delimiter and before the end of its run, and
        when the text right after the opening delimiter names the assistant.
        """

        code_at = self.is_image[tokens]
        if not code_at.any():
            return []
        length = len(tokens)
        run_id = np.concatenate(([0], np.cumsum((segments[1:] != segments[:-1]) | (valid[1:] != valid[:-1]))))
        opens = np.flatnonzero((tokens == self.start_id) & valid)
        if not len(opens):
            return []
        closes = np.flatnonzero(tokens == self.end_id)
        # for every opening delimiter: the first closing delimiter after it, if it comes before
        # the next opening delimiter of the same run and inside the same run
        nearest = np.searchsorted(closes, opens)
        has_close = nearest < len(closes)
        close_at = np.where(has_close, closes[np.minimum(nearest, len(closes) - 1)] if len(closes) else 0, length)
        next_open = np.append(opens[1:], length)
        same_run_next = np.append(run_id[opens[1:]] == run_id[opens[:-1]], False)
        limit = np.where(same_run_next, next_open, length)
        complete = has_close & (close_at < limit) & (run_id[np.minimum(close_at, length - 1)] == run_id[opens])
        grids = []
        for start, end in zip(opens[complete].tolist(), close_at[complete].tolist()):
            role = self.tokenizer.decode(tokens[start + 1:min(end, start + 1 + ROLE_PROBE)].tolist())
            if not role.startswith(ASSISTANT):
                continue
            grids.extend(self._split_into_grids(tokens, start + 1 + np.flatnonzero(code_at[start + 1:end])))
        return grids

    def _split_into_grids(self, tokens: np.ndarray, positions: np.ndarray):
        """Cut the code positions of one message body into grids. Adjacent codes share a grid row;
        a gap that decodes to a bare line break separates two rows of one grid; any other gap
        separates two grids. Rows of a grid must be equally wide."""

        if not len(positions):
            return []
        gaps = np.flatnonzero(np.diff(positions) > 1)
        # classify every gap: 1 = row break, 2 = grid break
        kind = np.empty(len(gaps), dtype=np.int8)
        for slot, gap in enumerate(gaps.tolist()):
            filler = tokens[positions[gap] + 1:positions[gap + 1]]
            is_break = len(filler) <= ROW_BREAK_LIMIT and self.tokenizer.decode(filler.tolist()) in ROW_BREAKS
            kind[slot] = 1 if is_break else 2
        grid_edges = np.concatenate(([0], gaps[kind == 2] + 1, [len(positions)]))
        row_edges = np.concatenate(([0], gaps + 1, [len(positions)]))      # every gap ends a row
        grids = []
        for lo, hi in zip(grid_edges[:-1].tolist(), grid_edges[1:].tolist()):
            inside = row_edges[(row_edges >= lo) & (row_edges <= hi)]
            if len(set(np.diff(inside).tolist())) > 1:
                raise ValueError("assistant image grid has unequal row widths")
            grids.append((int(positions[lo]), int(positions[hi - 1]) + 1, positions[lo:hi]))
        return grids

    def _blocks(self, tokens, valid, segments):
        """Grids of one row as (first, one past last, code positions)."""

        return self._row_grids(np.asarray(tokens), np.asarray(valid) != 0, np.asarray(segments))

    def find_blocks(self, tokens: np.ndarray, valid: np.ndarray, segments: np.ndarray,
                    weights: np.ndarray) -> BlockTable:
        rows, firsts, stops, pieces, supervised = [], [], [], [], []
        for row in range(tokens.shape[0]):
            for first, stop, codes in self._row_grids(tokens[row], valid[row], segments[row]):
                rows.append(row)
                firsts.append(first)
                stops.append(stop)
                pieces.append(codes)
                supervised.append(bool((weights[row, codes] > 0).any()))
        sizes = [len(piece) for piece in pieces]
        return BlockTable(
            row=np.asarray(rows, dtype=np.int64), first=np.asarray(firsts, dtype=np.int64),
            stop=np.asarray(stops, dtype=np.int64),
            code_begin=np.concatenate(([0], np.cumsum(sizes))).astype(np.int64),
            codes=np.concatenate(pieces).astype(np.int64) if pieces else np.zeros(0, np.int64),
            supervised=np.asarray(supervised, dtype=np.bool_))

    # ---------------------------------------------------------------- stage 2: the random plan
    def plan(self, table: BlockTable, *, step: int) -> MaskPlan:
        stream = np.random.default_rng(np.random.SeedSequence([self.seed, step]))
        selected, masked_row, masked_col = [], [], []
        for index in np.flatnonzero(table.supervised).tolist():   # unsupervised blocks draw nothing
            if stream.random() >= self.probability:
                continue
            codes = table.codes_of(index)
            share = math.cos(0.5 * math.pi * stream.random())
            count = max(1, math.ceil(len(codes) * share))
            picked = stream.choice(codes, size=count, replace=False)
            selected.append(index)
            masked_col.append(picked)
            masked_row.append(np.full(count, table.row[index]))
        join = (lambda parts: np.concatenate(parts).astype(np.int64)) if selected else (lambda parts: np.zeros(0, np.int64))
        return MaskPlan(np.asarray(selected, dtype=np.int64), join(masked_row), join(masked_col))

    # ---------------------------------------------------------------- stage 3: array updates
    def apply(self, original: np.ndarray, valid: np.ndarray, segments: np.ndarray, weights: np.ndarray,
              table: BlockTable, plan: MaskPlan):
        rows, length = original.shape
        # next-token supervision everywhere first
        targets = np.concatenate((original[:, 1:], np.zeros((rows, 1), original.dtype)), axis=1)
        linked = valid[:, :-1] & valid[:, 1:] & (segments[:, :-1] == segments[:, 1:])
        prediction_weights = np.zeros(weights.shape, dtype=weights.dtype)
        prediction_weights[:, :-1] = np.where(linked, weights[:, 1:], 0)
        attention_end = np.broadcast_to(np.arange(length, dtype=np.int32), (rows, length)).copy()
        tokens = original.copy()

        # selected blocks: coverage by a difference array over the flattened batch, so that every
        # block is handled by the same few array operations
        block_row, first, stop = table.row[plan.selected], table.first[plan.selected], table.stop[plan.selected]
        if len(block_row):
            flat = np.zeros(rows * length + 1, dtype=np.int32)
            np.add.at(flat, block_row * length + first, 1)
            np.add.at(flat, block_row * length + stop, -1)
            inside = np.cumsum(flat[:-1]).reshape(rows, length) > 0
            last = np.zeros(rows * length + 1, dtype=np.int64)
            np.add.at(last, block_row * length + first, stop - 1)
            np.add.at(last, block_row * length + stop, -(stop - 1))
            attention_end = np.where(inside, np.cumsum(last[:-1]).reshape(rows, length), attention_end).astype(np.int32)
            # the edge into the block belongs to the position in front of it
            cut = inside.copy()
            before = first - 1
            cut[block_row[before >= 0], before[before >= 0]] = True
            prediction_weights[cut] = 0
            tokens[plan.masked_row, plan.masked_col] = self.mask_id
            targets[plan.masked_row, plan.masked_col] = original[plan.masked_row, plan.masked_col]
            prediction_weights[plan.masked_row, plan.masked_col] = weights[plan.masked_row, plan.masked_col]
        return tokens, attention_end, targets, prediction_weights

    def __call__(self, batch: Mapping[str, np.ndarray], *, step: int) -> dict[str, np.ndarray]:
        if self.probability == 0.0:
            return dict(batch)
        original = np.asarray(batch["input_ids"], dtype=np.int32)
        valid = np.asarray(batch["attention_mask"]) != 0
        segments = np.asarray(batch["segment_ids"])
        weights = np.asarray(batch["loss_weights"], dtype=np.float32)
        table = self.find_blocks(original, valid, segments, weights)
        tokens, attention_end, targets, prediction_weights = self.apply(
            original, valid, segments, weights, table, self.plan(table, step=step))
        result = dict(batch)
        result.update(input_ids=tokens, attention_end=attention_end, prediction_targets=targets,
                      prediction_weights=prediction_weights)
        return result

    def batches(self, stream, *, start_step: int) -> Iterator:
        """Transform a stream of batches; batch i of the stream is masked as optimizer step
        ``start_step + i`` (so a resumed run repeats the masks of the interrupted one). Items are
        mappings, or objects with ``.data`` and ``.with_data(mapping)``."""

        step = start_step
        for item in stream:
            yield self(item, step=step) if isinstance(item, Mapping) else item.with_data(self(item.data, step=step))
            step += 1


__all__ = ["BlockTable", "MaskGITBatchTransform", "MaskPlan"]
