"""GPU parity of the decoder-layer neighbours of attention (through the C ABI) against the oracle.

Integer outputs (position ids) are bit-exact. Floating-point tolerances, stated where used:
rotary tables within one bf16 unit in the last place of the oracle's (f32 cos/sin implementations
may differ in the last f32 bit, which moves a bf16 rounding in ~1e-4 of the entries); the
rotation within the roundings that separate "round once from f32" (the kernel) from "round every
product and sum to bf16" (the oracle, as jnp evaluates the reference); RMSNorm within two bf16
units in the last place on a small fraction of entries (reduction order of the f32 mean);
gradients rel-L2 <= 2e-2 as for the other bf16 gradients of this library.
"""

import numpy as np
import pytest
import torch

from oracle import attention_ref, layer_ref

pytestmark = pytest.mark.gpu


def _bf16(array):
    return torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)


def test_position_ids_known_answers(ct, gpu):
    # reference tests/modeling/test_rotary.py:63-78
    valid = torch.tensor([[0, 1, 1, 1, 1, 1, 1]], dtype=torch.int32, device=gpu)
    labels = torch.tensor([[0, 0, 0, 7, 7, 0, 0]], dtype=torch.int32, device=gpu)
    assert ct.make_position_ids(valid, labels).cpu().tolist() == [[0, 0, 1, 0, 1, 0, 1]]
    gap = torch.tensor([[1, 1, 0, 1, 1]], dtype=torch.int32, device=gpu)
    assert ct.make_position_ids(gap).cpu().tolist() == [[0, 1, 0, 0, 1]]


@pytest.mark.parametrize("batch,seq", [(1, 1), (3, 7), (2, 64), (5, 1000), (2, 1025), (4, 4096), (1, 262144)])
def test_position_ids_match_oracle(ct, gpu, batch, seq):
    rng = np.random.default_rng(batch * 7919 + seq)
    for density in (0.0, 0.5, 0.97, 1.0):
        mask = (rng.random((batch, seq)) < density).astype(np.int32)
        run = np.maximum(1, seq // 29)
        labels = np.repeat(rng.integers(0, 5, (batch, seq // run + 1)), run, axis=1)[:, :seq].astype(np.int32)
        got = ct.make_position_ids(torch.from_numpy(mask).to(gpu), torch.from_numpy(labels).to(gpu))
        np.testing.assert_array_equal(got.cpu().numpy(), layer_ref.make_position_ids(mask, labels))
        got = ct.make_position_ids(torch.from_numpy(mask).to(gpu))
        np.testing.assert_array_equal(got.cpu().numpy(), layer_ref.make_position_ids(mask))


def test_rotary_tables_match_oracle_including_jump_positions(ct, gpu):
    # reference tests/modeling/test_rotary.py:81-90: reset and jump positions, no cache
    positions = np.array([[0, 1, 0, 2_000_000]], dtype=np.int32)
    inv_freq = np.array([1.0, 0.01], dtype=np.float32)
    cosine, sine = ct.rotary_cos_sin(torch.from_numpy(positions).to(gpu), torch.from_numpy(inv_freq).to(gpu))
    want_c, want_s = layer_ref.rotary_cos_sin(positions, inv_freq)
    assert cosine.shape == sine.shape == (1, 4, 2) and cosine.dtype == torch.bfloat16
    assert float((cosine.cpu().float() - want_c.float()).abs().max()) <= 2.0 ** -8
    assert float((sine.cpu().float() - want_s.float()).abs().max()) <= 2.0 ** -8

    rng = np.random.default_rng(11)
    positions = rng.integers(0, 131072, size=(4, 4096)).astype(np.int32)
    inv_freq = layer_ref.inverse_frequencies(64, 500_000.0)
    cosine, sine = ct.rotary_cos_sin(torch.from_numpy(positions).to(gpu), torch.from_numpy(inv_freq).to(gpu))
    want_c, want_s = layer_ref.rotary_cos_sin(positions, inv_freq)
    for got, want in ((cosine, want_c), (sine, want_s)):
        diff = (got.cpu().float() - want.float()).abs()
        assert float(diff.max()) <= 2.0 ** -8          # one bf16 unit in the last place below 1
        assert float((diff > 0).float().mean()) < 1e-3  # and only where an f32 last bit decides


def _pair_bound(x, rotary_dim, style):
    """max(|x_a|, |x_b|) of each rotated channel's pair, broadcast back to the channel layout."""
    head = x[..., :rotary_dim].float().abs()
    if style == "gpt-j":
        m = torch.maximum(head[..., ::2], head[..., 1::2])
        return torch.stack((m, m), dim=-1).reshape(head.shape)
    a, b = torch.chunk(head, 2, dim=-1)
    m = torch.maximum(a, b)
    return torch.cat((m, m), dim=-1)


@pytest.mark.parametrize("style", ["gpt-j", "gpt-neox"])
@pytest.mark.parametrize("shape", [(1, 5, 2, 1, 16, 16), (2, 130, 8, 2, 64, 32), (2, 512, 32, 8, 128, 64),
                                   (1, 64, 4, 4, 128, 128),
                                   # outside the 16-byte kernel's granularity: the element-wise kernel
                                   (1, 4, 2, 2, 8, 4), (2, 37, 3, 1, 12, 6), (1, 9, 2, 1, 64, 24), (1, 3, 1, 1, 10, 10)])
def test_rotary_matches_oracle(ct, gpu, style, shape):
    batch, seq, q_heads, kv_heads, head_dim, rotary_dim = shape
    rng = np.random.default_rng(sum(shape))
    q = _bf16(rng.standard_normal((batch, seq, q_heads, head_dim)) * 3.0)
    k = _bf16(rng.standard_normal((batch, seq, kv_heads, head_dim)) * 3.0)
    positions = rng.integers(0, 100_000, size=(batch, seq)).astype(np.int32)
    cosine, sine = layer_ref.rotary_cos_sin(positions, layer_ref.inverse_frequencies(rotary_dim, 1e4))
    want_q, want_k = layer_ref.apply_rotary_cos_sin(q, k, cosine, sine, rope_style=style)
    got_q, got_k = ct.apply_rotary_cos_sin(q.to(gpu), k.to(gpu), cosine.to(gpu), sine.to(gpu), rope_style=style)
    for got, want, x in ((got_q.cpu(), want_q, q), (got_k.cpu(), want_k, k)):
        # channels past the rotated ones pass through exactly
        assert torch.equal(got[..., rotary_dim:], x[..., rotary_dim:])
        # kernel: one rounding of the f32 result; oracle: two rounded products and a rounded sum.
        # Each rounding is <= 2^-8 relative (half a unit in the last place of an 8-bit significand)
        # on a term <= sqrt(2) m, m the larger of the pair.
        bound = 4 * 2.0 ** -8 * 1.4143 * _pair_bound(x, rotary_dim, style) + 1e-30
        assert bool(((got[..., :rotary_dim].float() - want[..., :rotary_dim].float()).abs() <= bound).all())
        # and the kernel is the more exact of the two
        exact = layer_ref.apply_rotary_f64(x, cosine, sine, rope_style=style)
        assert float((got.double() - exact).abs().max()) <= float((want.double() - exact).abs().max()) + 1e-12
        assert bool(((got.double() - exact).abs()[..., :rotary_dim]
                     <= 2.0 ** -8 * 1.4143 * _pair_bound(x, rotary_dim, style).double() + 1e-30).all())


@pytest.mark.parametrize("head_dim,rotary_dim", [(8, 4), (32, 16)])
def test_rotary_reference_example_with_tail_channels(ct, gpu, head_dim, rotary_dim):
    # reference tests/modeling/test_rotary.py:92-98 (rotary_dim 4 of 8: the element-wise kernel) and the
    # same construction at 16 of 32 channels (the 16-byte kernel)
    positions = np.array([[0, 1, 0, 2_000_000]], dtype=np.int32)
    inv_freq = layer_ref.inverse_frequencies(rotary_dim, 1e4)
    query = torch.arange(1 * 4 * 2 * head_dim, dtype=torch.float32).reshape(1, 4, 2, head_dim).to(torch.bfloat16)
    key = (query + torch.tensor(0.5, dtype=torch.bfloat16)).to(torch.bfloat16)
    cosine, sine = ct.rotary_cos_sin(torch.from_numpy(positions).to(gpu), torch.from_numpy(inv_freq).to(gpu))
    pre_q, pre_k = ct.apply_rotary_cos_sin(query.to(gpu), key.to(gpu), cosine, sine)
    direct_q, direct_k = ct.apply_rotary_embedding(query.to(gpu), key.to(gpu), torch.from_numpy(positions).to(gpu),
                                                   torch.from_numpy(inv_freq).to(gpu))
    assert torch.equal(pre_q, direct_q) and torch.equal(pre_k, direct_k)
    assert torch.equal(pre_q[..., rotary_dim:].cpu(), query[..., rotary_dim:])
    assert torch.equal(pre_k[..., rotary_dim:].cpu(), key[..., rotary_dim:])
    # position 0 rotates by nothing
    assert torch.equal(pre_q[:, 0].cpu(), query[:, 0]) and torch.equal(pre_q[:, 2].cpu(), query[:, 2])


def test_rotary_argument_errors_are_the_references(ct, gpu):
    q = torch.ones((1, 2, 2, 16), dtype=torch.bfloat16, device=gpu)
    table = torch.ones((1, 2, 8), dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError, match="rope_style"):
        ct.apply_rotary_cos_sin(q, q, table, table, rope_style="unknown")
    with pytest.raises(ValueError, match="must have shape"):
        ct.apply_rotary_cos_sin(q[0], q[0], table, table)
    with pytest.raises(ValueError, match="cosine and sine shapes differ"):
        ct.apply_rotary_cos_sin(q, q, table, table[..., :4])
    with pytest.raises(ValueError, match="invalid rotary dimension"):
        ct.apply_rotary_cos_sin(q, q, torch.ones((1, 2, 16), dtype=torch.bfloat16, device=gpu),
                                torch.ones((1, 2, 16), dtype=torch.bfloat16, device=gpu))
    with pytest.raises(ValueError, match="non-empty vector"):
        ct.rotary_cos_sin(torch.zeros((1, 2), dtype=torch.int32, device=gpu), torch.zeros((0,), device=gpu))


@pytest.mark.parametrize("style", ["gpt-j", "gpt-neox"])
def test_fused_query_scale_and_gradients(ct, gpu, style):
    rng = np.random.default_rng(21)
    q = _bf16(rng.standard_normal((2, 96, 8, 128))).to(gpu)
    k = _bf16(rng.standard_normal((2, 96, 2, 128))).to(gpu)
    positions = rng.integers(0, 8192, size=(2, 96)).astype(np.int32)
    cosine, sine = layer_ref.rotary_cos_sin(positions, layer_ref.inverse_frequencies(64, 1e4))
    cosine, sine = cosine.to(gpu), sine.to(gpu)
    scale = 128 ** -0.5
    plain_q, plain_k = ct.apply_rotary_cos_sin(q, k, cosine, sine, rope_style=style)
    fused_q, fused_k = ct.apply_rotary_cos_sin(q, k, cosine, sine, rope_style=style, q_scale=scale)
    # the attention operator's pre-scale (src/modeling/attention.py:124): a bf16 product with the
    # bf16-rounded scale, bit for bit
    scale_b = torch.tensor(scale, dtype=torch.bfloat16, device=gpu)
    assert torch.equal(fused_q, plain_q * scale_b)
    assert torch.equal(fused_k, plain_k)

    # gradients: the transpose rotation; against autograd of the oracle's chain
    qg, kg = q.clone().requires_grad_(True), k.clone().requires_grad_(True)
    out_q, out_k = ct.apply_rotary_cos_sin(qg, kg, cosine, sine, rope_style=style)
    dq_up = _bf16(rng.standard_normal(tuple(q.shape))).to(gpu)
    dk_up = _bf16(rng.standard_normal(tuple(k.shape))).to(gpu)
    torch.autograd.backward((out_q, out_k), (dq_up, dk_up))
    qc, kc = q.cpu().clone().requires_grad_(True), k.cpu().clone().requires_grad_(True)
    ref_q, ref_k = layer_ref.apply_rotary_cos_sin(qc, kc, cosine.cpu(), sine.cpu(), rope_style=style)
    torch.autograd.backward((ref_q, ref_k), (dq_up.cpu(), dk_up.cpu()))
    assert attention_ref.relative_l2(qg.grad.cpu(), qc.grad) <= 2e-2
    assert attention_ref.relative_l2(kg.grad.cpu(), kc.grad) <= 2e-2
    # exact structure: the backward is the forward with the sine negated
    neg_q, neg_k = ct.apply_rotary_cos_sin(dq_up, dk_up, cosine, -sine, rope_style=style)
    assert torch.equal(qg.grad, neg_q) and torch.equal(kg.grad, neg_k)


@pytest.mark.parametrize("rows,hidden", [(1, 8), (5, 136), (37, 512), (300, 4096), (16384, 4096), (9, 8192)])
def test_rms_norm_forward_matches_oracle(ct, gpu, rows, hidden):
    rng = np.random.default_rng(rows + hidden)
    x = _bf16(rng.standard_normal((rows, hidden)) * rng.uniform(0.1, 8.0, size=(rows, 1)))
    scale = _bf16(rng.uniform(0.5, 1.5, size=hidden))
    want = layer_ref.rms_norm(x, scale, 1e-6)
    got = ct.rms_norm(x.to(gpu), scale.to(gpu), 1e-6).cpu()
    diff = (got.float() - want.float()).abs()
    # two bf16 units in the last place at most (a last-bit difference in the f32 statistic can move
    # the rounded normalised value by one unit, and the rounding of the product by another), on few entries
    assert bool((diff <= 2 * 2.0 ** -7 * want.float().abs() + 1e-30).all())
    assert float((diff > 0).float().mean()) < 2e-3
    torch.testing.assert_close(got.double(), layer_ref.rms_norm_f64(x, scale, 1e-6), rtol=2.0 ** -7, atol=1e-6)


def test_rms_norm_special_rows(ct, gpu):
    scale = _bf16(np.linspace(0.5, 1.5, 512)).to(gpu)
    x = torch.zeros((3, 512), dtype=torch.bfloat16, device=gpu)
    x[1] = -3.0
    y = ct.rms_norm(x, scale, 1e-6)
    assert torch.equal(y[0], torch.zeros(512, dtype=torch.bfloat16, device=gpu))   # eps keeps 0/0 away
    assert torch.equal(y[1], -scale)                                              # constant row -> -1 * scale
    with pytest.raises(ValueError, match="scale must have shape"):
        ct.rms_norm(x, scale[:8], 1e-6)
    assert ct.rms_norm(x[:0], scale, 1e-6).shape == (0, 512)


@pytest.mark.parametrize("rows,hidden", [(3, 512), (257, 1024), (4100, 4096), (33, 8192),
                                         # sizes outside 512 * 2^k: the kernel that walks the row
                                         (2, 8), (700, 136), (1030, 768), (65, 5120), (5, 16384)])
def test_rms_norm_gradients_match_oracle(ct, gpu, rows, hidden):
    rng = np.random.default_rng(rows * 3 + hidden)
    x = _bf16(rng.standard_normal((rows, hidden)) * rng.uniform(0.1, 4.0, size=(rows, 1)))
    scale = _bf16(rng.uniform(0.5, 1.5, size=hidden))
    dy = _bf16(rng.standard_normal((rows, hidden)))
    xg, sg = x.to(gpu).requires_grad_(True), scale.to(gpu).requires_grad_(True)
    ct.rms_norm(xg, sg, 1e-6).backward(dy.to(gpu))
    want_dx, want_dscale = layer_ref.rms_norm_vjp(x, scale, 1e-6, dy)
    _, dx64, dscale64 = layer_ref.rms_norm_f64(x, scale, 1e-6, dy)
    assert attention_ref.relative_l2(xg.grad.cpu(), want_dx) <= 2e-2
    assert attention_ref.relative_l2(xg.grad.cpu(), dx64) <= 1e-2
    assert attention_ref.relative_l2(sg.grad.cpu(), want_dscale) <= 2e-2
    assert attention_ref.relative_l2(sg.grad.cpu(), dscale64) <= 1e-2
    with pytest.raises((RuntimeError, ValueError), match="multiple of 8"):
        bad = torch.ones((2, 132), dtype=torch.bfloat16, device=gpu, requires_grad=True)
        ct.rms_norm(bad, torch.ones(132, dtype=torch.bfloat16, device=gpu), 1e-6).sum().backward()
