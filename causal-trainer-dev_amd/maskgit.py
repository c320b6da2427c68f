"""MaskGIT batch transform: produces ``attention_end`` and the aligned prediction targets.

Mirror of the reference's host-side transform (src/causal_trainer/data/maskgit.py:20-135): same
class name, constructor and call signature, output fields and random stream. It runs on host
batches after packing and adds three O(B*S) arrays:

  attention_end       int32 [B, S]  last key each query may see; ``arange(S)`` (plain causal) except
                                    inside a selected image block, where every position sees the whole
                                    block - the operand the attention operator's hybrid mask takes
  prediction_targets  int32 [B, S]  next-token targets, except at masked image codes, whose target
                                    is their own original code (same-position prediction)
  prediction_weights  f32   [B, S]  loss weight per position for the cut cross-entropy operator

``input_ids`` is returned with the chosen codes replaced by ``[MASK]``. Every random choice is a
function of (seed, optimizer step) through ``numpy.random.default_rng(SeedSequence([seed, step]))``
and the draws happen in the reference's order (per block: one uniform for selection, one for the
masking ratio, one ``choice`` without replacement), so a batch is masked identically in both.

The tokenizer is duck-typed: ``get_vocab()``, ``__call__(text)["input_ids"]``, ``decode(ids)`` and
optionally ``pad_token_id``.
"""

from __future__ import annotations

import math
import re
from collections.abc import Iterator, Mapping

import numpy as np

_IMAGE_TOKEN = re.compile(r"<\|image_[0-9]+\|>")
_SPECIAL = ("[MASK]", "<|im_start|>", "<|im_end|>")
_HEADER_TOKENS = 32  # tokens of a message header decoded to find its role
_GAP_TOKENS = 8      # longest gap between codes that can still be a row break


class MaskGITBatchTransform:
    """Select each complete, supervised assistant image block with probability p and mask a
    cosine-scheduled share of its codes."""

    def __init__(self, tokenizer, *, probability: float, seed: int) -> None:
        if not math.isfinite(probability) or not 0.0 <= probability <= 1.0:
            raise ValueError("maskgit_probability must be between 0 and 1")
        self.probability = probability
        self.seed = seed
        self.tokenizer = tokenizer
        vocabulary = tokenizer.get_vocab()
        for token in _SPECIAL:
            if token not in vocabulary or tokenizer(token)["input_ids"] != [vocabulary[token]]:
                raise ValueError(f"MaskGIT requires {token!r} to encode as one token")
        self.mask_id, self.start_id, self.end_id = (vocabulary[token] for token in _SPECIAL)
        codes = [index for token, index in vocabulary.items() if _IMAGE_TOKEN.fullmatch(token)]
        if not codes:
            raise ValueError("MaskGIT requires <|image_i|> tokens in the tokenizer vocabulary")
        size = max(max(vocabulary.values()), getattr(tokenizer, "pad_token_id", None) or 0) + 1
        self.is_image = np.zeros(size, dtype=np.bool_)
        self.is_image[codes] = True

    # ------------------------------------------------------------------ block discovery
    def _messages(self, tokens, lo, hi):
        """(start, end) of every message in [lo, hi) that has its closing delimiter before the
        next opening one."""

        window = tokens[lo:hi]
        opens = lo + np.flatnonzero(window == self.start_id)
        closes = lo + np.flatnonzero(window == self.end_id)
        following = np.append(opens[1:], hi)
        slot = np.searchsorted(closes, opens)
        for start, limit, at in zip(opens, following, slot):
            if at < len(closes) and closes[at] < limit:
                yield int(start), int(closes[at])

    def _grids(self, tokens, start, end):
        """Image grids inside the message body (start, end): runs of codes joined by single
        newlines; any other text between codes starts a new grid."""

        where = start + 1 + np.flatnonzero(self.is_image[tokens[start + 1:end]])
        if not len(where):
            return
        grid_cuts, row_cuts = [0], []
        for gap in np.flatnonzero(np.diff(where) > 1):
            between = tokens[where[gap] + 1:where[gap + 1]]
            text = self.tokenizer.decode(between.tolist()) if len(between) <= _GAP_TOKENS else None
            (row_cuts if text in ("\n", "\r\n") else grid_cuts).append(int(gap) + 1)
        grid_cuts.append(len(where))
        for first, last in zip(grid_cuts[:-1], grid_cuts[1:]):
            edges = np.array([first, *[cut for cut in row_cuts if first < cut < last], last])
            widths = np.diff(edges)
            if (widths != widths[0]).any():
                raise ValueError("assistant image grid has unequal row widths")
            yield where[first:last]

    def _blocks(self, tokens, valid, segments):
        """Yield (first, one past last, code positions) of the image grids inside complete
        assistant messages of one row (maskgit.py:48-91)."""

        tokens = np.asarray(tokens)
        valid = np.asarray(valid) != 0
        segments = np.asarray(segments)
        if not self.is_image[tokens].any():
            return
        change = (segments[1:] != segments[:-1]) | (valid[1:] != valid[:-1])
        bounds = np.flatnonzero(np.concatenate(([True], change, [True])))
        for lo, hi in zip(bounds[:-1], bounds[1:]):
            if not valid[lo]:
                continue
            for start, end in self._messages(tokens, lo, hi):
                header = self.tokenizer.decode(tokens[start + 1:min(end, start + 1 + _HEADER_TOKENS)].tolist())
                if not header.startswith(("assistant\n", "assistant\r\n")):
                    continue
                for codes in self._grids(tokens, start, end):
                    yield int(codes[0]), int(codes[-1]) + 1, codes

    # ------------------------------------------------------------------ the transform
    def __call__(self, batch: Mapping[str, np.ndarray], *, step: int) -> dict[str, np.ndarray]:
        if self.probability == 0.0:
            return dict(batch)
        original = np.asarray(batch["input_ids"], dtype=np.int32)
        valid = np.asarray(batch["attention_mask"]) != 0
        segments = np.asarray(batch["segment_ids"])
        weights = np.asarray(batch["loss_weights"], dtype=np.float32)
        rows, length = original.shape

        # ordinary autoregressive supervision: position i predicts token i + 1 of the same run
        tokens = original.copy()
        targets = np.zeros_like(original)
        targets[:, :-1] = original[:, 1:]
        same_run = valid[:, :-1] & valid[:, 1:] & (segments[:, :-1] == segments[:, 1:])
        prediction_weights = np.zeros_like(weights)
        prediction_weights[:, :-1] = weights[:, 1:] * same_run
        attention_end = np.tile(np.arange(length, dtype=np.int32), (rows, 1))

        rng = np.random.default_rng(np.random.SeedSequence([self.seed, step]))
        for row in range(rows):
            for first, stop, codes in self._blocks(original[row], valid[row], segments[row]):
                # blocks without supervision (disabled turns, dummy rows) stay as they are and
                # draw nothing; the selection draw comes before the ratio draw
                if not (weights[row, codes] > 0).any() or rng.random() >= self.probability:
                    continue
                share = math.cos(math.pi * 0.5 * rng.random())
                chosen = rng.choice(codes, size=max(1, math.ceil(len(codes) * share)), replace=False)
                tokens[row, chosen] = self.mask_id
                attention_end[row, first:stop] = stop - 1
                # no next-token edge into, inside or out of the block (newlines and the closing
                # delimiter come from the template); masked codes predict themselves
                prediction_weights[row, max(0, first - 1):stop] = 0.0
                targets[row, chosen] = original[row, chosen]
                prediction_weights[row, chosen] = weights[row, chosen]
        return {**batch, "input_ids": tokens, "attention_end": attention_end,
                "prediction_targets": targets, "prediction_weights": prediction_weights}

    def batches(self, batches, *, start_step: int) -> Iterator:
        """Transform a stream of batches, numbering them from start_step (resume-safe)."""

        for step, batch in enumerate(batches, start=start_step):
            if isinstance(batch, Mapping):
                yield self(batch, step=step)
            else:
                yield batch.with_data(self(batch.data, step=step))


__all__ = ["MaskGITBatchTransform"]
