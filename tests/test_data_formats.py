"""Packing and the MaskGIT batch transform: the host-side formats that feed both hot paths (CPU).

Known answers restated from the reference's tests/data/test_packing.py and
tests/training/test_maskgit.py (each test names the one it repeats), and reference-derived vectors
(tests/golden/data_formats_ref.json, written by tests/golden/make_data_golden.py) for what those
leave open: best-fit placement of arbitrary lengths and the exact random stream of the masking.
"""

import json
from pathlib import Path

import numpy as np
import pytest

from oracle import attention_ref, cutce_ref
from tests.golden.chatml_tokenizer import ByteChatTokenizer, image_grid, record

GOLDEN = json.loads((Path(__file__).parent / "golden" / "data_formats_ref.json").read_text())


@pytest.fixture(scope="module")
def fmt():
    import causal_trainer_dev_amd as ct

    return ct


@pytest.fixture(scope="module")
def tokenizer():
    return ByteChatTokenizer()


def row(token, length, assistant_masks=None):
    result = {"input_ids": [token] * length, "attention_mask": [1] * length}
    if assistant_masks is not None:
        result["assistant_masks"] = assistant_masks
    return result


def batch_of(fmt, tokenizer, records, *, packing=True, length=256):
    fn = fmt.pack_examples if packing else fmt.pad_examples
    return fmt.collate(fn(records, max_length=length, pad_token_id=tokenizer.pad_token_id), assistant_only_loss=True)


# ----------------------------------------------------------------------------- packing
def test_bfd_packs_without_separator_and_resets_segment_positions(fmt):
    packed = fmt.pack_examples([row(1, 6), row(2, 4), row(3, 4), row(4, 2)], max_length=8, pad_token_id=99)
    assert len(packed) == 2
    assert packed[0]["input_ids"] == [1] * 6 + [4] * 2
    assert packed[0]["position_ids"] == [0, 1, 2, 3, 4, 5, 0, 1]
    assert packed[0]["segment_ids"] == [1] * 6 + [2] * 2
    assert packed[1]["input_ids"] == [2] * 4 + [3] * 4
    assert 99 not in packed[0]["input_ids"]


def test_bfd_is_scoped_to_each_packing_batch(fmt):
    packed = fmt.pack_examples([row(1, 6), row(2, 6), row(3, 2), row(4, 2)], max_length=8, pad_token_id=0,
                               packing_batch_size=2)
    assert len(packed) == 3


def test_left_padding_is_fixed_length_and_all_masks_stay_aligned(fmt):
    result = fmt.pack_examples([row(5, 3, [0, 1, 1]), row(6, 2, [0, 1])], max_length=8, pad_token_id=99)[0]
    assert result["input_ids"] == [99, 99, 99, 5, 5, 5, 6, 6]
    assert result["attention_mask"] == [0, 0, 0, 1, 1, 1, 1, 1]
    assert result["assistant_masks"] == [0, 0, 0, 0, 1, 1, 0, 1]
    assert result["position_ids"] == [0, 0, 0, 0, 1, 2, 0, 1]
    assert result["segment_ids"] == [0, 0, 0, 1, 1, 1, 2, 2]
    assert all(len(value) == 8 for value in result.values())


def test_metadata_resets_for_every_contiguous_valid_run(fmt):
    packed = fmt.pack_examples([{"input_ids": [10, 11, 12, 13], "attention_mask": [1, 1, 0, 1]},
                                {"input_ids": [20, 21, 22], "attention_mask": [0, 1, 1]}],
                               max_length=7, pad_token_id=99)[0]
    assert packed["attention_mask"] == [1, 1, 0, 1, 0, 1, 1]
    assert packed["position_ids"] == [0, 1, 0, 0, 0, 0, 1]
    assert packed["segment_ids"] == [1, 1, 0, 2, 0, 3, 3]


def test_truncation_keeps_all_per_token_fields_synchronized(fmt):
    packed = fmt.pack_examples([{"input_ids": [1, 2, 3, 4, 5, 6], "attention_mask": [1] * 6,
                                 "assistant_masks": [0, 0, 1, 1, 0, 1]}], max_length=4, pad_token_id=0)[0]
    assert packed["input_ids"] == [1, 2, 3, 4]
    assert packed["assistant_masks"] == [0, 0, 1, 1]
    assert packed["position_ids"] == [0, 1, 2, 3]


def test_endprompt_packing_preserves_anchored_positions_and_float_weights(fmt):
    packed = fmt.pack_examples(
        [{"input_ids": [10, 11, 90], "attention_mask": [1, 1, 1], "position_ids": [0, 1, 15],
          "loss_weights": [1.0, 1.0, 0.1]},
         {"input_ids": [20, 91], "attention_mask": [1, 1], "position_ids": [0, 31], "loss_weights": [1.0, 0.25]}],
        max_length=6, pad_token_id=0)[0]
    assert packed["input_ids"] == [0, 10, 11, 90, 20, 91]
    assert packed["position_ids"] == [0, 0, 1, 15, 0, 31]
    assert packed["segment_ids"] == [0, 1, 1, 1, 2, 2]
    assert packed["loss_weights"] == [0.0, 1.0, 1.0, 0.1, 1.0, 0.25]


def test_endprompt_assistant_masks_and_combined_weights_survive_packing(fmt):
    packed = fmt.pack_examples(
        [{"input_ids": [10, 11, 90], "attention_mask": [1, 1, 1], "assistant_masks": [0, 1, 0],
          "position_ids": [0, 1, 15], "loss_weights": [0.0, 1.0, 0.1]},
         {"input_ids": [20, 21, 91], "attention_mask": [1, 1, 1], "assistant_masks": [0, 1, 0],
          "position_ids": [0, 1, 31], "loss_weights": [0.0, 0.5, 0.25]}],
        max_length=6, pad_token_id=0)[0]
    assert packed["segment_ids"] == [1, 1, 1, 2, 2, 2]
    assert packed["assistant_masks"] == [0, 1, 0, 0, 1, 0]
    assert packed["loss_weights"] == [0.0, 1.0, 0.1, 0.0, 0.5, 0.25]


def test_endprompt_nonpacking_padding_also_preserves_anchor_positions(fmt):
    padded = fmt.pad_examples([{"input_ids": [10, 90], "attention_mask": [1, 1], "position_ids": [0, 63],
                                "loss_weights": [1.0, 0.1]}], max_length=4, pad_token_id=0)[0]
    assert padded["position_ids"] == [0, 0, 0, 63]
    assert padded["segment_ids"] == [0, 0, 1, 1]
    assert padded["loss_weights"] == [0.0, 0.0, 1.0, 0.1]


def test_inconsistent_optional_masks_fail_instead_of_silently_dropping_them(fmt):
    with pytest.raises(ValueError, match="same per-token fields"):
        fmt.pack_examples([row(1, 2, [0, 1]), row(2, 2)], max_length=4, pad_token_id=0)


def test_pad_examples_does_not_combine_samples(fmt):
    padded = fmt.pad_examples([row(7, 2), row(8, 3)], max_length=4, pad_token_id=99)
    assert [item["input_ids"] for item in padded] == [[99, 99, 7, 7], [99, 8, 8, 8]]
    assert padded[0]["segment_ids"] == [0, 0, 1, 1]


def test_pad_examples_metadata_respects_internal_padding(fmt):
    padded = fmt.pad_examples([{"input_ids": [1, 2, 3, 4], "attention_mask": [0, 1, 1, 0]}], max_length=6,
                              pad_token_id=99)[0]
    assert padded["attention_mask"] == [0, 0, 0, 1, 1, 0]
    assert padded["position_ids"] == [0, 0, 0, 0, 1, 0]
    assert padded["segment_ids"] == [0, 0, 0, 1, 1, 0]


def test_misaligned_mask_and_bad_values_are_rejected(fmt):
    with pytest.raises(ValueError, match="expected 3"):
        fmt.pack_examples([{"input_ids": [1, 2, 3], "assistant_masks": [0, 1]}], max_length=4, pad_token_id=0)
    with pytest.raises(ValueError, match="binary"):
        fmt.pack_examples([{"input_ids": [1, 2], "attention_mask": [1, 2]}], max_length=4, pad_token_id=0)
    with pytest.raises(ValueError, match="non-negative"):
        fmt.pack_examples([{"input_ids": [1, 2], "loss_weights": [1.0, -1.0]}], max_length=4, pad_token_id=0)
    with pytest.raises(ValueError, match="finite"):
        fmt.pack_examples([{"input_ids": [1, 2], "loss_weights": [1.0, float("nan")]}], max_length=4, pad_token_id=0)
    with pytest.raises(ValueError, match="empty input_ids"):
        fmt.pack_examples([{"input_ids": []}], max_length=4, pad_token_id=0)
    with pytest.raises(ValueError, match="max_length must be positive"):
        fmt.pack_examples([row(1, 2)], max_length=0, pad_token_id=0)
    with pytest.raises(ValueError, match="padding_side"):
        fmt.pad_example(row(1, 2), max_length=4, pad_token_id=0, padding_side="middle")


@pytest.mark.parametrize("case", range(len(GOLDEN["packing"])))
def test_packing_matches_the_reference_vectors(fmt, case):
    """Where best-fit-decreasing puts examples of arbitrary lengths is what the reference's own tests
    leave open: the vectors under tests/golden were written by the reference's packing module."""

    entry = GOLDEN["packing"][case]
    kwargs = {key: entry[key] for key in ("max_length", "pad_token_id", "packing_batch_size", "padding_side")}
    packed = fmt.pack_examples(entry["examples"], **kwargs)
    assert packed == entry["packed"]
    assert [list(item) for item in packed] == [list(item) for item in entry["packed"]]  # field order too
    padded = fmt.pad_examples(entry["examples"], max_length=entry["max_length"], pad_token_id=entry["pad_token_id"],
                              padding_side=entry["padding_side"])
    assert padded == entry["padded"]
    assert [list(item) for item in padded] == [list(item) for item in entry["padded"]]


def test_packed_segments_feed_the_operators(fmt):
    # what packing emits is what the operators' metadata takes: the ids are already canonical, and
    # the shifted loss drops exactly the targets that cross an example boundary or touch padding
    rng = np.random.default_rng(3)
    examples = [{"input_ids": rng.integers(1, 50, size=int(n)).tolist()} for n in rng.integers(2, 30, size=9)]
    rows = fmt.pack_examples(examples, max_length=32, pad_token_id=0)
    batch = fmt.collate(rows)
    valid = batch["attention_mask"] == 1
    assert np.array_equal(attention_ref.canonicalize_segment_ids(valid, batch["segment_ids"]), batch["segment_ids"])
    assert np.array_equal(batch["loss_weights"], batch["attention_mask"].astype(np.float32))
    targets, weights = cutce_ref.shifted_targets_and_weights(batch["input_ids"], batch["attention_mask"],
                                                             batch["segment_ids"])
    same = (batch["segment_ids"][:, :-1] == batch["segment_ids"][:, 1:]) & (batch["segment_ids"][:, 1:] != 0)
    assert np.array_equal(weights > 0, same)
    assert sum(len(e["input_ids"]) for e in examples) == int(valid.sum())


# ----------------------------------------------------------------------------- MaskGIT
def test_probability_zero_is_identity_and_bad_options_are_rejected(fmt, tokenizer):
    batch = batch_of(fmt, tokenizer, [record(tokenizer)])
    result = fmt.MaskGITBatchTransform(tokenizer, probability=0, seed=3)(batch, step=9)
    assert result.keys() == batch.keys()
    for key in batch:
        np.testing.assert_array_equal(batch[key], result[key])
    for value in (float("nan"), float("inf"), -0.1, 1.1):
        with pytest.raises(ValueError, match="maskgit_probability"):
            fmt.MaskGITBatchTransform(tokenizer, probability=value, seed=0)


def test_vq_code_numbers_use_tokenizer_ids_including_16383(fmt, tokenizer):
    vocabulary = tokenizer.get_vocab()
    low, high = vocabulary["<|image_0|>"], vocabulary["<|image_16383|>"]
    assert low != 0 and high != 16383
    batch = batch_of(fmt, tokenizer, [record(tokenizer, "<|image_0|><|image_16383|>")])
    transform = fmt.MaskGITBatchTransform(tokenizer, probability=1, seed=3)
    assert transform.is_image[low] and transform.is_image[high]
    mixed = transform(batch, step=0)
    masked = mixed["input_ids"] == transform.mask_id
    assert masked.any()
    np.testing.assert_array_equal(mixed["prediction_targets"][masked], batch["input_ids"][masked])
    assert set(mixed["prediction_targets"][masked]) <= {low, high}


@pytest.mark.parametrize("packing", [False, True])
def test_actual_shape_newlines_and_mixed_text_are_preserved(fmt, tokenizer, packing):
    batch = batch_of(fmt, tokenizer, [record(tokenizer), record(tokenizer, "plain answer")], packing=packing)
    saved = {key: value.copy() for key, value in batch.items()}
    transform = fmt.MaskGITBatchTransform(tokenizer, probability=1, seed=1)
    mixed = transform(batch, step=0)
    blocks = [(r, *block) for r in range(len(batch["input_ids"])) for block in transform._blocks(
        batch["input_ids"][r], batch["attention_mask"][r], batch["segment_ids"][r])]
    assert len(blocks) == 1
    r, start, end, images = blocks[0]
    assert len(images) == 6  # the prompt claims 999 x 999: it must not determine the shape
    masked = np.flatnonzero(mixed["input_ids"][r] == transform.mask_id)
    assert set(masked) <= set(images) and len(masked) > 0
    np.testing.assert_array_equal(mixed["prediction_targets"][r, masked], batch["input_ids"][r, masked])
    assert np.all(mixed["prediction_weights"][r, masked] == 1)
    newline_positions = np.setdiff1d(np.arange(start, end), images)
    assert len(newline_positions) > 0
    np.testing.assert_array_equal(mixed["input_ids"][r, newline_positions], batch["input_ids"][r, newline_positions])
    assert np.all(mixed["prediction_weights"][r, newline_positions] == 0)
    assert mixed["prediction_weights"][r, start - 1] == 0
    assert np.all(mixed["attention_end"][r, start:end] == end - 1)
    # the mask the attention operator builds from these arrays
    allowed = attention_ref.allowed_mask(mixed["attention_mask"], mixed["segment_ids"], mixed["attention_end"])
    assert allowed[r, start, end - 1]
    assert not allowed[r, start - 1, start]
    assert not allowed[r, start, end]
    for b, mask in enumerate(allowed):
        segments = mixed["segment_ids"][b]
        assert not mask[segments[:, None] != segments[None, :]].any()
    for key in batch:
        np.testing.assert_array_equal(batch[key], saved[key])


def test_per_block_selection_reproducibility_resume_and_multiple_grids(fmt, tokenizer):
    batch = batch_of(fmt, tokenizer, [record(tokenizer, image_grid() + "\n\nnext:\n" + image_grid(2, 2))])
    transform = fmt.MaskGITBatchTransform(tokenizer, probability=0.5, seed=34)
    blocks = list(transform._blocks(batch["input_ids"][0], batch["attention_mask"][0], batch["segment_ids"][0]))
    assert [len(block[2]) for block in blocks] == [6, 4]
    selected = []
    for step in range(100):
        mixed = transform(batch, step=step)
        repeated = transform(batch, step=step)
        for key in mixed:
            np.testing.assert_array_equal(mixed[key], repeated[key])
        selected.append(tuple(mixed["attention_end"][0, start] == end - 1 for start, end, _ in blocks))
    assert set(selected) == {(False, False), (False, True), (True, False), (True, True)}
    assert 65 < np.sum(selected) < 135
    resumed = next(transform.batches([batch], start_step=37))
    np.testing.assert_array_equal(resumed["input_ids"], transform(batch, step=37)["input_ids"])


def test_unselected_blocks_keep_original_ar_targets_and_attention(fmt, tokenizer):
    batch = batch_of(fmt, tokenizer, [record(tokenizer), record(tokenizer, "ordinary text")])
    mixed = fmt.MaskGITBatchTransform(tokenizer, probability=.001, seed=2)(batch, step=0)
    np.testing.assert_array_equal(mixed["input_ids"], batch["input_ids"])
    targets, weights = cutce_ref.shifted_targets_and_weights(batch["input_ids"], batch["attention_mask"],
                                                             batch["segment_ids"], loss_mask=batch["loss_weights"])
    np.testing.assert_array_equal(mixed["prediction_weights"][:, :-1], weights)
    supervised = weights > 0
    np.testing.assert_array_equal(mixed["prediction_targets"][:, :-1][supervised], targets[supervised])
    np.testing.assert_array_equal(
        attention_ref.allowed_mask(batch["attention_mask"], batch["segment_ids"], mixed["attention_end"]),
        attention_ref.allowed_mask(batch["attention_mask"], batch["segment_ids"]))


def test_crlf_and_disabled_turn_preserve_context(fmt, tokenizer):
    first = record(tokenizer, image_grid().replace("\n", "\r\n"))
    disabled = record(tokenizer)
    disabled["assistant_masks"] = [0] * len(disabled["input_ids"])
    batch = batch_of(fmt, tokenizer, [first, disabled])
    transform = fmt.MaskGITBatchTransform(tokenizer, probability=1, seed=9)
    mixed = transform(batch, step=0)
    masked = mixed["input_ids"] == transform.mask_id
    assert masked.any()
    assert not masked[batch["loss_weights"] == 0].any()
    images = transform.is_image[batch["input_ids"]]
    np.testing.assert_array_equal(mixed["input_ids"][~images], batch["input_ids"][~images])


def test_disabled_input_images_and_truncation_are_not_corrupted(fmt, tokenizer):
    transform = fmt.MaskGITBatchTransform(tokenizer, probability=1, seed=0)
    for entry in (record(tokenizer, role="user"), record(tokenizer)):
        batch = batch_of(fmt, tokenizer, [entry])
        batch["loss_weights"][:] = 0
        mixed = transform(batch, step=0)
        np.testing.assert_array_equal(mixed["input_ids"], batch["input_ids"])
        assert not mixed["prediction_weights"].any()
    truncated = {key: value[:-2] for key, value in record(tokenizer).items()}
    batch = batch_of(fmt, tokenizer, [truncated])
    np.testing.assert_array_equal(transform(batch, step=0)["input_ids"], batch["input_ids"])


def test_non_rectangular_grid_is_rejected(fmt, tokenizer):
    batch = batch_of(fmt, tokenizer, [record(tokenizer, image_grid() + "<|image_9|>")])
    with pytest.raises(ValueError, match="unequal row widths"):
        fmt.MaskGITBatchTransform(tokenizer, probability=1, seed=0)(batch, step=0)


def test_tokenizer_requirements_are_checked(fmt, tokenizer):
    class NoImages(ByteChatTokenizer):
        def get_vocab(self):
            return {token: index for token, index in super().get_vocab().items() if not token.startswith("<|image_")}

    with pytest.raises(ValueError, match="image_i"):
        fmt.MaskGITBatchTransform(NoImages(), probability=1, seed=0)

    class NoMask(ByteChatTokenizer):
        def get_vocab(self):
            return {token: index for token, index in super().get_vocab().items() if token != "[MASK]"}

    with pytest.raises(ValueError, match="MASK"):
        fmt.MaskGITBatchTransform(NoMask(), probability=1, seed=0)


def _golden_batch(entry):
    source = next(e for e in GOLDEN["maskgit"] if e["packing"] == entry["packing"] and e["batch"] is not None)
    dtypes = {"loss_weights": np.float32}
    return {key: np.asarray(value, dtype=dtypes.get(key, np.int32)) for key, value in source["batch"].items()}


@pytest.mark.parametrize("index", range(len(GOLDEN["maskgit"])))
def test_maskgit_matches_the_reference_vectors(fmt, tokenizer, index):
    entry = GOLDEN["maskgit"][index]
    batch = _golden_batch(entry)
    transform = fmt.MaskGITBatchTransform(tokenizer, probability=entry["probability"], seed=entry["seed"])
    blocks = [[[start, end, codes.tolist()] for start, end, codes in transform._blocks(
        batch["input_ids"][r], batch["attention_mask"][r], batch["segment_ids"][r])] for r in range(len(batch["input_ids"]))]
    assert blocks == entry["blocks"]
    mixed = transform(batch, step=entry["step"])
    for key, dtype in (("input_ids", np.int32), ("attention_end", np.int32), ("prediction_targets", np.int32),
                       ("prediction_weights", np.float32)):
        assert mixed[key].dtype == dtype
        np.testing.assert_array_equal(mixed[key], np.asarray(entry["mixed"][key], dtype=dtype), err_msg=key)


def test_golden_batches_come_from_this_packing(fmt, tokenizer):
    # the batches in the vectors were packed and collated by the reference from the same records
    from tests.golden.make_data_golden import maskgit_inputs

    records = maskgit_inputs(tokenizer)
    for packing, length in ((True, 256), (False, 128)):
        entry = next(e for e in GOLDEN["maskgit"] if e["packing"] == packing and e["batch"] is not None)
        batch = batch_of(fmt, tokenizer, records, packing=packing, length=length)
        assert list(batch) == list(entry["batch"])
        for key, value in batch.items():
            np.testing.assert_array_equal(value, np.asarray(entry["batch"][key]), err_msg=key)
