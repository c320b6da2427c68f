"""The layer-neighbour oracle against the reference's own known answers and closed forms (CPU).

Known answers restated from the reference's tests/modeling/test_rotary.py (each test names the
reference test it repeats); RMSNorm has no known-answer test in the reference, so it is pinned by
torch's library routine, closed forms and a float64 formula.
"""

import numpy as np
import pytest
import torch

from oracle import layer_ref
from oracle.attention_ref import canonicalize_segment_ids


def test_rotary_defaults_to_gpt_j_adjacent_pairs_and_leaves_tail_unchanged():
    # test_rotary.py::test_rotary_defaults_to_gpt_j_adjacent_pairs_and_leaves_tail_unchanged
    query = torch.tensor([[[[1.0, 2.0, 3.0, 4.0]]]])
    rotated_q, rotated_k = layer_ref.apply_rotary_embedding(query, query.clone(), np.array([[1]]), np.array([1.0]))
    expected = torch.tensor([1.0 * np.cos(1.0) - 2.0 * np.sin(1.0), 2.0 * np.cos(1.0) + 1.0 * np.sin(1.0)],
                            dtype=torch.float32)
    assert torch.allclose(rotated_q[0, 0, 0, :2], expected)
    assert torch.equal(rotated_q[..., 2:], query[..., 2:])
    assert torch.equal(rotated_q, rotated_k)


def test_rotary_supports_gpt_neox_half_pairs_and_leaves_tail_unchanged():
    # test_rotary.py::test_rotary_supports_gpt_neox_half_pairs_and_leaves_tail_unchanged
    query = torch.tensor([[[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]]])
    rotated_q, rotated_k = layer_ref.apply_rotary_embedding(query, query.clone(), np.array([[1]]),
                                                            np.array([1.0, 0.5]), rope_style="gpt-neox")
    cosine = torch.cos(torch.tensor([1.0, 0.5]))
    sine = torch.sin(torch.tensor([1.0, 0.5]))
    expected = torch.cat((query[0, 0, 0, :2] * cosine - query[0, 0, 0, 2:4] * sine,
                          query[0, 0, 0, 2:4] * cosine + query[0, 0, 0, :2] * sine))
    assert torch.allclose(rotated_q[0, 0, 0, :4], expected)
    assert torch.equal(rotated_q[..., 4:], query[..., 4:])
    assert torch.equal(rotated_q, rotated_k)


def test_rotary_rejects_unknown_style():
    # test_rotary.py::test_rotary_rejects_unknown_style
    query = torch.ones((1, 1, 1, 2))
    with pytest.raises(ValueError, match="rope_style"):
        layer_ref.apply_rotary_embedding(query, query, np.array([[0]]), np.array([1.0]), rope_style="unknown")


def test_positions_reset_for_zero_label_and_reused_segment_runs():
    # test_rotary.py::test_positions_reset_for_zero_label_and_reused_segment_runs
    valid = np.array([[0, 1, 1, 1, 1, 1, 1]], dtype=bool)
    labels = np.array([[0, 0, 0, 7, 7, 0, 0]], dtype=np.int32)
    assert np.array_equal(canonicalize_segment_ids(valid, labels), [[0, 1, 1, 2, 2, 3, 3]])
    assert np.array_equal(layer_ref.make_position_ids(valid, labels), [[0, 0, 1, 0, 1, 0, 1]])


def test_positions_restart_after_an_internal_masked_gap_without_explicit_segments():
    # test_rotary.py::test_positions_restart_after_an_internal_masked_gap_without_explicit_segments
    valid = np.array([[1, 1, 0, 1, 1]], dtype=bool)
    assert np.array_equal(layer_ref.make_position_ids(valid), [[0, 1, 0, 0, 1]])


def test_precomputed_rotary_uses_actual_reset_and_jump_positions_without_a_cache():
    # test_rotary.py::test_precomputed_rotary_uses_actual_reset_and_jump_positions_without_a_cache
    positions = np.array([[0, 1, 0, 2_000_000]], dtype=np.int32)
    inv_freq = np.array([1.0, 0.01], dtype=np.float32)
    cosine, sine = layer_ref.rotary_cos_sin(positions, inv_freq, torch.bfloat16)
    assert cosine.shape == sine.shape == (1, 4, 2)
    assert cosine.dtype == sine.dtype == torch.bfloat16
    angles = positions.astype(np.float32)[..., None] * inv_freq[None, None, :]
    assert torch.equal(cosine, torch.from_numpy(np.cos(angles)).to(torch.bfloat16))
    assert torch.equal(sine, torch.from_numpy(np.sin(angles)).to(torch.bfloat16))
    # a float64 evaluation of the float32 angle agrees: the large argument is reduced correctly
    assert abs(float(cosine[0, 3, 0]) - np.cos(np.float64(angles[0, 3, 0]))) < 2.0 ** -8

    query = torch.arange(1 * 4 * 2 * 8, dtype=torch.float32).reshape(1, 4, 2, 8).to(torch.bfloat16)
    key = (query + torch.tensor(0.5, dtype=torch.bfloat16)).to(torch.bfloat16)
    pre_q, pre_k = layer_ref.apply_rotary_cos_sin(query, key, cosine, sine)
    direct_q, direct_k = layer_ref.apply_rotary_embedding(query, key, positions, inv_freq)
    assert torch.equal(pre_q, direct_q) and torch.equal(pre_k, direct_k)
    assert torch.equal(pre_q[..., 4:], query[..., 4:])
    assert torch.equal(pre_k[..., 4:], key[..., 4:])


def test_inverse_frequencies_follow_the_transformers_operation_order():
    # rotary.py:53-60; closed form 1 / theta^(2i/d) in float64
    got = layer_ref.inverse_frequencies(64, 10_000.0)
    want = 1.0 / np.power(10_000.0, np.arange(0, 64, 2, dtype=np.float64) / 64.0)
    assert got.dtype == np.float32 and got.shape == (32,)
    assert got[0] == 1.0
    np.testing.assert_allclose(got, want, rtol=3e-7)


@pytest.mark.parametrize("style", ["gpt-j", "gpt-neox"])
def test_rotation_preserves_pair_norms_and_its_transpose_undoes_it(style):
    rng = np.random.default_rng(5)
    x = torch.from_numpy(rng.standard_normal((2, 9, 3, 16))).double()
    positions = rng.integers(0, 5000, size=(2, 9))
    cosine, sine = layer_ref.rotary_cos_sin(positions, layer_ref.inverse_frequencies(8, 10_000.0), torch.float64)
    # float32 tables cast up: still unit vectors to 1e-7
    rotated = layer_ref.apply_rotary_f64(x, cosine, sine, rope_style=style)
    head, tail = rotated[..., :8], rotated[..., 8:]
    assert torch.equal(tail, x[..., 8:])
    torch.testing.assert_close(head.square().sum(-1), x[..., :8].square().sum(-1), rtol=1e-6, atol=1e-6)
    back = layer_ref.apply_rotary_f64(rotated, cosine, sine, rope_style=style, inverse=True)
    torch.testing.assert_close(back, x, rtol=1e-6, atol=1e-6)
    # position 0 is the identity
    zero_c, zero_s = layer_ref.rotary_cos_sin(np.zeros((2, 9), np.int32), layer_ref.inverse_frequencies(8, 1e4),
                                              torch.float64)
    assert torch.equal(layer_ref.apply_rotary_f64(x, zero_c, zero_s, rope_style=style), x)


def test_bf16_rotation_stays_within_its_rounding_of_the_exact_one():
    rng = np.random.default_rng(6)
    q = torch.from_numpy(rng.standard_normal((2, 33, 4, 32)).astype(np.float32)).to(torch.bfloat16)
    k = torch.from_numpy(rng.standard_normal((2, 33, 2, 32)).astype(np.float32)).to(torch.bfloat16)
    positions = rng.integers(0, 4096, size=(2, 33))
    cosine, sine = layer_ref.rotary_cos_sin(positions, layer_ref.inverse_frequencies(16, 1e4))
    for style in ("gpt-j", "gpt-neox"):
        got_q, got_k = layer_ref.apply_rotary_cos_sin(q, k, cosine, sine, rope_style=style)
        for got, x in ((got_q, q), (got_k, k)):
            exact = layer_ref.apply_rotary_f64(x, cosine, sine, rope_style=style)
            # three roundings of relative size 2^-9 on terms bounded by sqrt(2) max|x|
            assert float((got.double() - exact).abs().max()) <= 3 * 2.0 ** -9 * 1.5 * float(x.abs().max())


def test_rms_norm_matches_the_library_routine_and_closed_forms():
    rng = np.random.default_rng(7)
    x = torch.from_numpy(rng.standard_normal((3, 5, 64)).astype(np.float32))
    scale = torch.from_numpy(rng.uniform(0.5, 1.5, size=64).astype(np.float32))
    # float32 compute dtype: exactly the textbook operator
    got = layer_ref.rms_norm(x, scale, 1e-6, torch.float32)
    want = torch.nn.functional.rms_norm(x, (64,), scale, 1e-6)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(got.double(), layer_ref.rms_norm_f64(x, scale, 1e-6), rtol=1e-5, atol=1e-6)
    # a constant row normalises to +-1 times the scale; zero rows stay zero (eps keeps it finite)
    const = torch.full((1, 64), -3.0)
    torch.testing.assert_close(layer_ref.rms_norm(const, scale, 0.0, torch.float32), -scale[None, :])
    assert torch.equal(layer_ref.rms_norm(torch.zeros(2, 64), scale, 1e-6, torch.float32), torch.zeros(2, 64))
    # positive rescaling of the input leaves the output unchanged when eps = 0
    torch.testing.assert_close(layer_ref.rms_norm(4.0 * x, scale, 0.0, torch.float32),
                               layer_ref.rms_norm(x, scale, 0.0, torch.float32), rtol=1e-6, atol=1e-6)
    # bf16 compute dtype: normalised value and product each rounded once (architecture.py:160-161)
    xb = x.to(torch.bfloat16)
    r = torch.rsqrt(xb.float().square().mean(-1, keepdim=True) + 1e-6)
    want_b = ((xb.float() * r).to(torch.bfloat16) * scale.to(torch.bfloat16)).to(torch.bfloat16)
    assert torch.equal(layer_ref.rms_norm(xb, scale, 1e-6), want_b)


def test_rms_norm_gradients_match_the_closed_form():
    rng = np.random.default_rng(8)
    x = torch.from_numpy(rng.standard_normal((7, 128)).astype(np.float32))
    scale = torch.from_numpy(rng.uniform(0.5, 1.5, size=128).astype(np.float32))
    dy = torch.from_numpy(rng.standard_normal((7, 128)).astype(np.float32))
    dx, dscale = layer_ref.rms_norm_vjp(x, scale, 1e-6, dy, torch.float32)
    _, dx64, dscale64 = layer_ref.rms_norm_f64(x, scale, 1e-6, dy)
    torch.testing.assert_close(dx.double(), dx64, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dscale.double(), dscale64, rtol=1e-4, atol=1e-5)
    # dx is orthogonal to x for each row when eps = 0 (the output does not depend on |x|)
    dx0, _ = layer_ref.rms_norm_vjp(x, scale, 0.0, dy, torch.float32)
    assert float((dx0 * x).sum(-1).abs().max()) < 1e-4
