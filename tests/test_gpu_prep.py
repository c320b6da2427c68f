"""GPU parity of the preparation kernels (through the C ABI) against the oracle: bit-exact.

Known answers are the reference's own (tests/modeling/test_attention.py:61-74,
tests/training/test_losses.py:27-28, :40-109); the rest is seeded random input compared with
oracle/attention_ref.py and oracle/cutce_ref.py, including ragged lengths, holes of padding,
reused and zero labels, and the maximum sequence length.
"""

import numpy as np
import pytest
import torch

from oracle import attention_ref, cutce_ref

pytestmark = pytest.mark.gpu


def _canon(ct, gpu, mask, labels=None):
    out = ct.canonicalize_segment_ids(torch.from_numpy(np.asarray(mask)).to(gpu),
                                      None if labels is None else torch.from_numpy(np.asarray(labels)).to(gpu))
    return out.cpu().numpy()


def test_canonical_ids_known_answer(ct, gpu):
    valid = np.array([[0, 1, 1, 1, 1, 1, 1]], dtype=np.int32)
    labels = np.array([[0, 0, 0, 8, 8, 0, 0]], dtype=np.int32)
    assert _canon(ct, gpu, valid, labels).tolist() == [[0, 1, 1, 2, 2, 3, 3]]
    assert _canon(ct, gpu, valid).tolist() == [[0, 1, 1, 1, 1, 1, 1]]


@pytest.mark.parametrize("batch,seq", [(1, 1), (3, 7), (2, 64), (5, 1000), (2, 1025), (4, 4096), (1, 262144)])
def test_canonical_ids_match_oracle(ct, gpu, batch, seq):
    rng = np.random.default_rng(batch * 100003 + seq)
    for density in (0.0, 0.5, 0.97, 1.0):
        mask = (rng.random((batch, seq)) < density).astype(np.int32) * rng.integers(1, 4, (batch, seq)).astype(np.int32)
        # labels in long constant runs, with reuse and zeros
        run = np.maximum(1, seq // 37)
        labels = np.repeat(rng.integers(0, 5, (batch, seq // run + 1)), run, axis=1)[:, :seq].astype(np.int32)
        expected = attention_ref.canonicalize_segment_ids(mask, labels)
        np.testing.assert_array_equal(_canon(ct, gpu, mask, labels), expected)
        np.testing.assert_array_equal(_canon(ct, gpu, mask), attention_ref.canonicalize_segment_ids(mask))


def _shifted(ct, gpu, ids, mask, segments=None, assistant=None, loss=None, labels=None, ignore_index=-100):
    def dev(x, dtype=None):
        if x is None:
            return None
        t = torch.from_numpy(np.asarray(x))
        return (t if dtype is None else t.to(dtype)).to(gpu)
    targets, weights = ct.shifted_targets_and_weights(dev(ids), dev(mask), dev(segments), dev(assistant),
                                                      dev(loss, torch.float32), dev(labels),
                                                      ignore_index=ignore_index)
    return targets.cpu().numpy(), weights.cpu().numpy()


def test_shifted_known_answers(ct, gpu):
    # src tests/training/test_losses.py:40-46
    ids = np.array([[0, 10, 11, 20, 21]], np.int32)
    mask = np.array([[0, 1, 1, 1, 1]], np.int32)
    segments = np.array([[0, 1, 1, 2, 2]], np.int32)
    targets, weights = _shifted(ct, gpu, ids, mask, segments)
    assert targets.tolist() == [[0, 11, 0, 21]]
    assert (weights > 0).tolist() == [[False, True, False, True]]
    # zero and reused labels are canonicalised (:49-59)
    segments = np.array([[0, 0, 0, 7, 7]], np.int32)
    targets, weights = _shifted(ct, gpu, ids, mask, segments)
    assert (weights > 0).tolist() == [[False, True, False, True]]
    # assistant mask at the target position (:62-77)
    assistant = np.array([[0, 0, 1, 0, 1]], np.int32)
    _, weights = _shifted(ct, gpu, ids, mask, np.array([[0, 1, 1, 1, 1]], np.int32), assistant)
    assert weights.tolist() == [[0.0, 1.0, 0.0, 1.0]]


@pytest.mark.parametrize("batch,seq", [(1, 2), (3, 9), (2, 513), (4, 4096), (2, 16385)])
def test_shifted_matches_oracle(ct, gpu, batch, seq):
    rng = np.random.default_rng(batch * 7919 + seq)
    for case in range(4):
        ids = rng.integers(0, 1000, (batch, seq)).astype(np.int32)
        mask = (rng.random((batch, seq)) < 0.9).astype(np.int32)
        if case == 3:
            mask = mask * rng.integers(1, 3, (batch, seq)).astype(np.int32)   # 2 is not "valid" for the loss
        run = max(1, seq // 11)
        segments = np.repeat(rng.integers(0, 4, (batch, seq // run + 1)), run, axis=1)[:, :seq].astype(np.int32)
        assistant = (rng.random((batch, seq)) < 0.6).astype(np.int32) if case >= 1 else None
        loss = rng.choice(np.array([0.0, 0.25, 0.5, 1.0, 2.0], np.float32), (batch, seq)) if case >= 2 else None
        labels = np.where(rng.random((batch, seq)) < 0.1, -100, ids).astype(np.int32) if case >= 1 else None
        for use_segments in (False, True):
            for use_mask in (True, False):
                seg = segments if use_segments else None
                m = mask if use_mask else None
                got_t, got_w = _shifted(ct, gpu, ids, m, seg, assistant, loss, labels)
                exp_t, exp_w = cutce_ref.shifted_targets_and_weights(ids, m, seg, assistant, loss, labels)
                np.testing.assert_array_equal(got_t, exp_t)
                np.testing.assert_array_equal(got_w, exp_w)           # f32 products, bit for bit


def test_prepared_targets_feed_the_loss_unchanged(ct, gpu):
    # the ignored-token set of the loss kernel is exactly the zero-weight set computed here
    rng = np.random.default_rng(5)
    batch, seq, width, vocab = 2, 129, 128, 300
    ids = rng.integers(0, vocab, (batch, seq)).astype(np.int32)
    mask = (rng.random((batch, seq)) < 0.85).astype(np.int32)
    segments = np.repeat(rng.integers(1, 4, (batch, 5)), 26, axis=1)[:, :seq].astype(np.int32)
    targets, weights = ct.shifted_targets_and_weights(torch.from_numpy(ids).to(gpu), torch.from_numpy(mask).to(gpu),
                                                      torch.from_numpy(segments).to(gpu))
    hidden = torch.from_numpy(rng.normal(size=(batch * (seq - 1), width)).astype(np.float32)).to(torch.bfloat16).to(gpu)
    head = torch.from_numpy(rng.normal(scale=0.05, size=(width, vocab)).astype(np.float32)).to(torch.bfloat16).to(gpu)
    nll, weight_sum, lse = ct.cutce_forward(hidden, head, targets.reshape(-1), weights.reshape(-1),
                                            sparse_compaction=True)
    flat = weights.reshape(-1).cpu()
    assert float(weight_sum) == float(flat.sum())
    assert ((lse.cpu() == 0) == (flat == 0)).all()
