"""Pins for oracle/cutce_ref.py: reference known answers, closed forms and library routines."""

import math

import numpy as np
import pytest
import torch

from oracle import cutce_ref as ref
from oracle.attention_ref import relative_l2


def _bf16(array):
    return torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)


# ---- shifted targets / weights: tests/training/test_losses.py ------------------------------
def test_shifted_mask_excludes_padding_and_packed_boundaries():
    # :38-46
    targets, weights = ref.shifted_targets_and_weights(
        [[0, 10, 11, 20, 21]], [[0, 1, 1, 1, 1]], [[0, 1, 1, 2, 2]])
    assert targets.tolist() == [[0, 11, 0, 21]]
    assert (weights > 0).tolist() == [[False, True, False, True]]


def test_shifted_mask_canonicalizes_zero_and_reused_labels():
    # :49-59
    targets, weights = ref.shifted_targets_and_weights(
        [[10, 11, 20, 21, 30, 31]], np.ones((1, 6), np.int32), [[0, 0, 7, 7, 0, 0]])
    assert targets.tolist() == [[11, 0, 21, 0, 31]]
    assert (weights > 0).tolist() == [[True, False, True, False, True]]


def test_assistant_mask_applies_at_target_position():
    # :62-77
    _, weights = ref.shifted_targets_and_weights([[1, 2, 3, 4]], np.ones((1, 4)), assistant_mask=[[0, 0, 1, 1]])
    assert (weights > 0).tolist() == [[False, True, True]]
    _, weights = ref.shifted_targets_and_weights([[10, 11, 12]], [[0, 1, 1]], assistant_mask=[[0, 1, 0]])
    assert (weights > 0).tolist() == [[False, False]]


def test_sequence_parallel_known_answer():
    # :12-36: ids 1..6 + padding, segments [1,1,2,2,2,2,0,0], fractional weights
    ids = np.array([[1, 2, 3, 4, 5, 6, 0, 0]], np.int32)
    segments = np.array([[1, 1, 2, 2, 2, 2, 0, 0]], np.int32)
    loss_mask = np.array([[0, 1, .5, .25, .5, 1, 0, 0]], np.float32)
    targets, weights = ref.shifted_targets_and_weights(ids, ids != 0, segments, loss_mask=loss_mask)
    np.testing.assert_array_equal(targets[:, :6], [[2, 0, 4, 5, 6, 0]])
    np.testing.assert_array_equal(weights, [[1, 0, .25, .5, 1, 0, 0]])
    assert float(weights.sum()) == 2.75


# ---- closed forms -------------------------------------------------------------------------
@pytest.mark.parametrize("weights,vocab,expected", [
    ([1.0, 1.0], 32, 2 * math.log(32)),              # :125
    ([1.0, 1.0], 5, 2 * math.log(5)),                # :133
    ([1.0, 0.25, 0.5], 5, 1.75 * math.log(5)),       # :149
    ([0.5, 0.0, 0.25], 5, 0.75 * math.log(5)),       # :167
    ([1.0, 0.35], 100, 1.35 * math.log(100)),        # :202-203
])
def test_zero_hidden_gives_weighted_log_vocab(weights, vocab, expected):
    rows = len(weights)
    hidden = torch.zeros((rows, 128), dtype=torch.bfloat16)
    head = _bf16(np.random.default_rng(0).normal(size=(128, vocab)))
    nll, weight_sum, lse = ref.cut_forward(hidden, head, torch.arange(rows) % vocab, torch.tensor(weights))
    assert float(nll) == pytest.approx(expected, rel=1e-6)
    assert float(weight_sum) == pytest.approx(sum(weights))
    active = torch.tensor(weights) != 0
    assert torch.allclose(lse[active], torch.full((int(active.sum()),), math.log(vocab)))
    assert (lse[~active] == 0).all()


def test_mean_loss_normalisation():
    assert ref.mean_loss(6.0, 0.5) == 6.0      # max(weight_sum, 1)
    assert ref.mean_loss(6.0, 3.0) == 2.0


# ---- library cross-checks -------------------------------------------------------------------
def _random_case(seed, rows=64, width=128, vocab=97):
    rng = np.random.default_rng(seed)
    hidden = _bf16(rng.normal(scale=0.5, size=(rows, width)))
    head = _bf16(rng.normal(scale=0.2, size=(width, vocab)))
    targets = torch.from_numpy(rng.integers(vocab, size=rows).astype(np.int32))
    weights = torch.from_numpy(rng.choice([0.0, 0.25, 1.0, 2.0], size=rows).astype(np.float32))
    return hidden, head, targets, weights


def test_forward_matches_library_cross_entropy():
    # same identity as tests/training/test_maskgit.py:216-236 (fused == -sum w log_softmax[target])
    hidden, head, targets, weights = _random_case(1)
    nll, weight_sum, lse = ref.cut_forward(hidden, head, targets, weights)
    logits = hidden.double() @ head.double()
    per_row = torch.nn.functional.cross_entropy(logits, targets.long(), reduction="none")
    assert float(nll) == pytest.approx(float((per_row * weights.double()).sum()), rel=1e-6)
    assert float(weight_sum) == float(weights.sum())
    active = weights != 0
    torch.testing.assert_close(lse[active].double(), torch.logsumexp(logits, -1)[active], atol=1e-5, rtol=0)


def test_f64_gradients_match_autograd_and_rows_sum_to_zero():
    hidden, head, targets, weights = _random_case(2)
    dy = 0.37
    nll, _, _, dhidden, dhead = ref.cut_f64(hidden, head, targets, weights, dy)
    h = hidden.double().requires_grad_(True)
    w = head.double().requires_grad_(True)
    loss = (torch.nn.functional.cross_entropy(h @ w, targets.long(), reduction="none") * weights.double()).sum()
    (loss * dy).backward()
    assert float(nll) == pytest.approx(float(loss), rel=1e-12)
    torch.testing.assert_close(dhidden, h.grad, atol=1e-12, rtol=1e-9)
    torch.testing.assert_close(dhead, w.grad, atol=1e-12, rtol=1e-9)


def test_bf16_backward_close_to_f64_and_exact_zeros():
    hidden, head, targets, weights = _random_case(3, rows=200, vocab=258)
    targets = targets.clone()
    targets[weights == 0] = -100          # raw ignore labels reach the kernel on zero-weight rows
    dy = 0.37
    _, _, lse = ref.cut_forward(hidden, head, targets, weights)
    dhidden, dhead = ref.cut_backward(hidden, head, targets, weights, lse, dy)
    _, _, _, dhidden64, dhead64 = ref.cut_f64(hidden, head, targets, weights, dy)
    assert relative_l2(dhidden, dhidden64) < 1e-2
    assert relative_l2(dhead, dhead64) < 1e-2
    assert (dhidden[weights == 0] == 0).all()
    assert ref.cut_backward(hidden, head, targets, weights, lse, dy, head_trainable=False)[1] is None


def test_analytic_logits_vjp_matches_autograd():
    # src/causal_trainer/kernels/fused_cross_entropy.py:88-103 vs autograd of :64-76
    hidden, head, targets, weights = _random_case(4)
    logits = (hidden.float() @ head.float()).requires_grad_(True)
    cotangent = torch.linspace(0.1, 1.0, logits.shape[0])
    ref.xla_sparse_cross_entropy(logits, targets, weights).backward(cotangent)
    analytic = ref.xla_sparse_cross_entropy_vjp(logits.detach(), targets, weights, cotangent)
    torch.testing.assert_close(analytic, logits.grad, atol=1e-6, rtol=1e-5)
    # softmax minus one-hot sums to zero along the vocabulary
    assert float(analytic.sum(-1).abs().max()) < 1e-5


def test_all_masked_gives_zero_loss_and_grads():
    # tests/kernels/test_tiled_cut.py:138-155
    hidden, head, targets, _ = _random_case(5)
    weights = torch.zeros(hidden.shape[0])
    nll, weight_sum, lse = ref.cut_forward(hidden, head, targets, weights)
    assert float(nll) == 0 and float(weight_sum) == 0 and not lse.any()
    dhidden, dhead = ref.cut_backward(hidden, head, targets, weights, lse, 1.0)
    assert not dhidden.any() and not dhead.any()


def test_compaction_is_stable_and_loss_invariant():
    # tests/kernels/test_cross_entropy_tpu.py:166-239 weight patterns
    hidden, head, targets, _ = _random_case(6, rows=96)
    patterns = {
        "trailing": np.r_[np.ones(40), np.zeros(56)],
        "inactive": np.zeros(96),
        "alternating": np.arange(96) % 2,
        "middle": np.r_[np.zeros(30), np.ones(20), np.zeros(46)],
        "dense": np.ones(96),
    }
    for name, pattern in patterns.items():
        weights = torch.from_numpy(pattern.astype(np.float32))
        base = ref.cut_forward(hidden, head, targets, weights)
        c_hidden, c_targets, c_weights, indices, slot_valid = ref.compact_active_rows(hidden, targets, weights)
        active = int((weights != 0).sum())
        assert indices[:active].tolist() == torch.nonzero(weights != 0).flatten().tolist(), name
        assert int(slot_valid.sum()) == active
        assert (c_weights[active:] == 0).all() and (c_targets[active:] == 0).all()
        compacted = ref.cut_forward(c_hidden, head, c_targets, c_weights)
        assert float(compacted[0]) == pytest.approx(float(base[0]), rel=1e-6, abs=1e-6), name
        assert float(compacted[1]) == float(base[1]), name


def test_reference_seeded_fixture_regenerates():
    # tests/kernels/test_tiled_cut.py:66-128, rng = default_rng(460)
    from tests.golden import make_golden

    fixture = make_golden.cutce_fixture()
    golden = np.load(make_golden.GOLDEN_DIR / "cutce_rng460.npz")
    np.testing.assert_array_equal(fixture["hidden"].view(torch.int16).numpy(), golden["hidden"])
    np.testing.assert_array_equal(fixture["head"].view(torch.int16).numpy(), golden["head"])
    np.testing.assert_array_equal(fixture["targets"], golden["targets"])
    np.testing.assert_array_equal(fixture["weights"], golden["weights"])
    hidden = fixture["hidden"].reshape(-1, 128)
    targets = torch.from_numpy(fixture["targets"].reshape(-1))
    weights = torch.from_numpy(fixture["weights"].reshape(-1))
    nll, weight_sum, lse = ref.cut_forward(hidden, fixture["head"], targets, weights)
    # expectations stated by the reference test: nll vs log_softmax reference rtol 2e-5 / atol 2e-3,
    # weight_sum exact
    logp = torch.log_softmax(hidden.double() @ fixture["head"].double(), -1)
    safe = targets.long().clamp(min=0)
    expected = -(logp.gather(1, safe[:, None])[:, 0] * weights.double()).sum()
    assert float(nll) == pytest.approx(float(expected), rel=2e-5, abs=2e-3)
    assert float(weight_sum) == float(weights.sum()) == float(golden["weight_sum"])
    assert float(nll) == float(golden["nll_sum"])
    np.testing.assert_array_equal(lse.numpy(), golden["lse"])


def test_streaming_sparse_ce_oracle_agrees_with_the_xla_path_and_its_ignore_rules():
    # the setup of the reference's tests/kernels/test_cross_entropy_tpu.py:50-98 (vocab 1280,
    # 256 rows, weight 0.5 on the first 96 rows, target 220 kept valid), with own seeds
    rng = np.random.default_rng(50)
    logits = torch.from_numpy((rng.standard_normal((256, 1280)) * 0.25).astype(np.float32)).to(torch.bfloat16)
    targets = torch.from_numpy(rng.integers(0, 1280, size=256).astype(np.int64))
    targets[0] = 220
    weights = torch.where(torch.arange(256) < 96, torch.tensor(0.5), torch.tensor(0.0))
    loss, lse = ref.pallas_sparse_cross_entropy(logits, targets, weights)
    want = ref.xla_sparse_cross_entropy(logits, targets, weights)
    torch.testing.assert_close(loss, want, rtol=0, atol=1e-6)
    assert torch.equal(lse[96:], torch.zeros(160)) and torch.equal(loss[96:], torch.zeros(160))
    cot = torch.from_numpy(rng.standard_normal(256).astype(np.float32))
    got = ref.pallas_sparse_cross_entropy_vjp(logits, targets, weights, cot)
    assert torch.equal(got, ref.xla_sparse_cross_entropy_vjp(logits, targets, weights, cot))
    # ignore_index rows and out-of-range targets: no loss / no one-hot, never an index error
    t2 = targets.clone()
    t2[1], t2[2], t2[3] = -100, 5000, -7
    loss2, lse2 = ref.pallas_sparse_cross_entropy(logits, t2, weights)
    assert float(loss2[1]) == 0.0 and float(lse2[1]) == 0.0
    torch.testing.assert_close(loss2[2], 0.5 * torch.logsumexp(logits[2].float(), -1))
    torch.testing.assert_close(loss2[3], 0.5 * torch.logsumexp(logits[3].float(), -1))
    grad2 = ref.pallas_sparse_cross_entropy_vjp(logits, t2, weights, cot)
    assert float(grad2[1].abs().max()) == 0.0
    torch.testing.assert_close(grad2[2].float().sum(), 0.5 * cot[2], rtol=2e-2, atol=2e-3)   # sum of softmax = 1
    # uniform logits: lse = log V exactly representable check
    flat = torch.zeros((2, 1024))
    l3, s3 = ref.pallas_sparse_cross_entropy(flat, torch.tensor([3, 4]), torch.tensor([2.0, 1.0]))
    torch.testing.assert_close(s3, torch.full((2,), float(np.log(1024.0))))
    torch.testing.assert_close(l3, torch.tensor([2.0, 1.0]) * float(np.log(1024.0)))


@pytest.mark.parametrize("compaction", [False, True])
def test_chunked_loop_meets_the_reference_expectations_on_its_seeded_data(compaction):
    # tests/kernels/test_tiled_cut.py:89-128 on a one-device mesh: chunks of 128 over 2 x 386
    # rows (a ragged last chunk), cotangent 0.37, checked against log_softmax + autograd
    from tests.golden import make_golden

    fixture = make_golden.cutce_fixture()
    hidden, head = fixture["hidden"].reshape(-1, 128), fixture["head"]
    targets = torch.from_numpy(fixture["targets"].reshape(-1))
    weights = torch.from_numpy(fixture["weights"].reshape(-1))
    nll, weight_sum, lse = ref.chunked_cut_forward(hidden, head, targets, weights, 128,
                                                  sparse_compaction=compaction)
    dhidden, dhead = ref.chunked_cut_backward(hidden, head, targets, weights, lse, 0.37, 128)

    h64 = hidden.double().requires_grad_(True)
    w64 = head.double().requires_grad_(True)
    logp = torch.log_softmax(h64 @ w64, -1)
    expected = -(logp.gather(1, targets.long().clamp(min=0)[:, None])[:, 0] * weights.double()).sum()
    (0.37 * expected).backward()
    assert float(nll) == pytest.approx(float(expected), rel=2e-5, abs=2e-3)
    assert float(weight_sum) == float(weights.sum())
    for got, want in ((dhidden, h64.grad), (dhead, w64.grad)):
        assert float((got.double() - want).norm() / want.norm()) < 0.025
    assert not dhidden[weights == 0].any()
    assert ref.chunked_cut_backward(hidden, head, targets, weights, lse, 0.37, 128, head_trainable=False)[1] is None

    # the chunk loop is the unchunked operator up to the order of f32 additions
    base_nll, base_weight, base_lse = ref.cut_forward(hidden, head, targets, weights)
    base_dhidden, base_dhead = ref.cut_backward(hidden, head, targets, weights, base_lse, 0.37)
    assert float(nll) == pytest.approx(float(base_nll), rel=1e-6)
    assert float(weight_sum) == float(base_weight)
    torch.testing.assert_close(lse, base_lse, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(dhidden.float(), base_dhidden.float(), rtol=0, atol=2.0 ** -8 * float(base_dhidden.abs().max()))
    assert float((dhead.float() - base_dhead.float()).norm() / base_dhead.float().norm()) < 4e-3


def test_chunked_loop_all_masked_rows():
    # tests/kernels/test_tiled_cut.py:138-155: 199 rows, every weight zero, frozen head
    from tests.golden import make_golden

    fixture = make_golden.cutce_fixture()
    hidden, head = fixture["hidden"].reshape(-1, 128)[:199], fixture["head"]
    targets = torch.full((199,), -100, dtype=torch.int32)
    weights = torch.zeros(199)
    nll, weight_sum, lse = ref.chunked_cut_forward(hidden, head, targets, weights, 128, sparse_compaction=True)
    assert float(nll) == float(weight_sum) == 0.0
    dhidden, dhead = ref.chunked_cut_backward(hidden, head, targets, weights, lse, 1.0, 128, head_trainable=False)
    assert dhead is None and not dhidden.any()
