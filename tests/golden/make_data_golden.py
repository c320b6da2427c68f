"""Writes tests/golden/data_formats_ref.json: reference-derived vectors for packing and MaskGIT.

Nothing else pins two things about these host-side formats: which row best-fit-decreasing puts
every example in for arbitrary lengths, and which codes a (seed, step) pair masks (the order of the
draws from the NumPy generator). For those, this script imports the reference's two pure-NumPy
modules (src/causal_trainer/data/packing.py, maskgit.py, batching.py's _collate; no JAX involved)
from /root/reference, runs them on seeded inputs and stores inputs and outputs as JSON. It needs
the reference tree and is therefore run in the build container only; the tests read the JSON.

Run from the repository root:  python -m tests.golden.make_data_golden
"""

from __future__ import annotations

import json
import sys
from pathlib import Path

import numpy as np

from .chatml_tokenizer import ByteChatTokenizer, image_grid, record

GOLDEN = Path(__file__).resolve().parent / "data_formats_ref.json"
REFERENCE_SRC = Path("/root/reference/src")


def packing_inputs():
    """Seeded packing batches: ragged lengths, optional masks / weights / explicit positions, holes."""

    rng = np.random.default_rng(2024)
    cases = []
    for case in range(6):
        max_length = int(rng.choice([16, 32, 48]))
        count = int(rng.integers(3, 14))
        with_assistant, with_weights, with_positions = (bool(rng.integers(2)) for _ in range(3))
        examples = []
        for _ in range(count):
            length = int(rng.integers(1, max_length + 6))  # some get truncated
            example = {"input_ids": rng.integers(1, 1000, size=length).tolist()}
            mask = (rng.random(length) > 0.12).astype(int)
            if case % 2:
                example["attention_mask"] = mask.tolist()
            else:
                mask = np.ones(length, dtype=int)
            if with_assistant:
                example["assistant_masks"] = (rng.random(length) > 0.5).astype(int).tolist()
            if with_weights:
                example["loss_weights"] = rng.choice([0.0, 0.25, 0.5, 1.0], size=length).tolist()
            if with_positions:
                example["position_ids"] = np.sort(rng.integers(0, 64, size=length)).tolist()
            examples.append(example)
        cases.append({"max_length": max_length, "pad_token_id": 0 if case % 3 else 99,
                      "packing_batch_size": int(rng.choice([4, 1000])),
                      "padding_side": "left" if case % 2 == 0 else "right", "examples": examples})
    return cases


def maskgit_inputs(tokenizer):
    """Conversations with one or several image grids, plain answers, CRLF rows, a disabled turn."""

    two_grids = image_grid() + "\n\nnext:\n" + image_grid(2, 2, first=8)
    wide = image_grid(8, 4)
    records = [
        record(tokenizer), record(tokenizer, "plain answer"), record(tokenizer, two_grids),
        record(tokenizer, wide), record(tokenizer, image_grid().replace("\n", "\r\n")),
        record(tokenizer, "<|image_0|><|image_16383|>"), record(tokenizer, role="user"),
        record(tokenizer, "look: " + image_grid(4, 3, first=3) + " done"),
    ]
    disabled = record(tokenizer, wide)
    disabled["assistant_masks"] = [0] * len(disabled["input_ids"])
    records.append(disabled)
    return records


def main() -> None:
    if not REFERENCE_SRC.is_dir():
        raise SystemExit("the reference tree is needed to regenerate these vectors")
    sys.path.insert(0, str(REFERENCE_SRC))
    from causal_trainer.data import maskgit as ref_maskgit
    from causal_trainer.data import packing as ref_packing
    from causal_trainer.data.batching import _collate

    out = {"packing": [], "maskgit": []}
    for case in packing_inputs():
        kwargs = {key: case[key] for key in ("max_length", "pad_token_id", "packing_batch_size", "padding_side")}
        packed = ref_packing.pack_examples(case["examples"], **kwargs)
        padded = ref_packing.pad_examples(case["examples"], max_length=case["max_length"],
                                          pad_token_id=case["pad_token_id"], padding_side=case["padding_side"])
        out["packing"].append({**case, "packed": packed, "padded": padded})

    tokenizer = ByteChatTokenizer()
    records = maskgit_inputs(tokenizer)
    for packing, length in ((True, 256), (False, 128)):
        fn = ref_packing.pack_examples if packing else ref_packing.pad_examples
        rows = fn(records, max_length=length, pad_token_id=tokenizer.pad_token_id)
        batch = _collate(rows, np.arange(len(rows)), True)
        blocks = None
        for probability, seed, steps in ((1.0, 3, (0, 1, 7)), (0.5, 34, (0, 5, 37, 1000)), (0.25, 2, (11,))):
            transform = ref_maskgit.MaskGITBatchTransform(tokenizer, probability=probability, seed=seed)
            if blocks is None:
                blocks = [[[start, end, codes.tolist()] for start, end, codes in transform._blocks(
                    batch["input_ids"][row], batch["attention_mask"][row], batch["segment_ids"][row])]
                    for row in range(len(rows))]
            for step in steps:
                mixed = transform(batch, step=step)
                out["maskgit"].append({
                    "packing": packing, "length": length, "probability": probability, "seed": seed, "step": step,
                    "batch": {key: value.tolist() for key, value in batch.items()},
                    "blocks": blocks,
                    "mixed": {key: mixed[key].tolist() for key in ("input_ids", "attention_end", "prediction_targets",
                                                                    "prediction_weights")},
                })
    # the batch repeats per entry; store it once per packing mode
    seen = {}
    for entry in out["maskgit"]:
        key = str(entry["packing"])
        if key in seen:
            assert entry["batch"] == seen[key]
            entry["batch"] = None
        else:
            seen[key] = entry["batch"]
    GOLDEN.write_text(json.dumps(out, separators=(",", ":")))
    print(f"wrote {GOLDEN} ({GOLDEN.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
