"""Pins for oracle/attention_ref.py: the reference's own known answers, brute force and library routines.

Each test names the reference test (path:line, relative to the reference root) whose expected
values it reuses, or the independent computation it checks against.
"""

import math

import numpy as np
import pytest
import torch

from oracle import attention_ref as ref


def _bf16(array):
    return torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)


# ---- integer side ---------------------------------------------------------------------------
def test_canonical_ids_known_answer():
    # tests/modeling/test_attention.py:61-74
    valid = np.array([[0, 1, 1, 1, 1, 1, 1]], bool)
    labels = np.array([[0, 0, 0, 8, 8, 0, 0]], np.int32)
    normalized = ref.canonicalize_segment_ids(valid, labels)
    np.testing.assert_array_equal(normalized, [[0, 1, 1, 2, 2, 3, 3]])
    allowed = ref.allowed_mask(valid, normalized)[0]
    assert not allowed[5, 1] and not allowed[5, 3]
    assert allowed[5, 5] and allowed[6, 5]
    assert not allowed[0].any()


def test_canonical_ids_identity_on_packer_output():
    ids = np.array([[1, 1, 2, 2, 2, 3, 0, 0]], np.int32)
    np.testing.assert_array_equal(ref.canonicalize_segment_ids(ids != 0, ids), ids)


def test_tile_summaries_known_answer():
    # tests/kernels/test_efficient_attention.py:446-480
    ids = np.concatenate((np.zeros(130), np.ones(49), np.full(122, 2), np.full(211, 3))).astype(np.int32)[None]
    q_summary, kv_summary = ref.block_summaries(ids, 128, 256)
    np.testing.assert_array_equal(q_summary, [[[0, 0], [1, 2], [2, 3], [3, 3]]])
    np.testing.assert_array_equal(kv_summary, [[[1, 2], [2, 3]]])
    # :483-503 all-padding input -> all-zero summaries
    q0, kv0 = ref.block_summaries(np.zeros((2, 512), np.int32), 128, 256)
    assert q0.shape == (2, 4, 2) and kv0.shape == (2, 2, 2)
    assert not q0.any() and not kv0.any()


def _maskgit_fixture():
    # tests/kernels/test_maskgit_attention.py:21-30
    segments = np.zeros((2, 512), np.int32)
    segments[0, 20:350] = 1
    segments[0, 350:500] = 2
    segments[1, :150] = 1
    segments[1, 150:] = 2
    ends = np.broadcast_to(np.arange(512, dtype=np.int32), segments.shape).copy()
    ends[0, 80:330] = 329
    ends[0, 390:470] = 469
    return segments, ends


def test_hybrid_skip_predicate_known_answer():
    # tests/kernels/test_maskgit_attention.py:74-95
    segments, ends = _maskgit_fixture()
    q_summary, kv_summary = ref.block_summaries(segments, 128, 128, ends)
    assert q_summary.reshape(2, -1).shape == (2, 12)
    assert ref.summary_should_run(q_summary, kv_summary, 0, 0, 2, block_q=128, block_kv=128)
    assert not ref.summary_should_run(q_summary, kv_summary, 0, 0, 3, block_q=128, block_kv=128)


def test_skip_predicate_never_drops_an_allowed_pair():
    # Soundness of the conservative predicate against the exact mask, random ragged layouts.
    rng = np.random.default_rng(7)
    for _ in range(20):
        seq, bq, bkv = 256, 32, 64
        ids = np.zeros((1, seq), np.int32)
        position, segment = int(rng.integers(0, 40)), 1
        while position < seq:
            length = int(rng.integers(1, 90))
            if rng.random() < 0.2:
                position += length  # a hole of padding
                continue
            ids[0, position:position + length] = segment
            position += length
            segment += 1
        ends = np.arange(seq, dtype=np.int32)[None].copy()
        start = int(rng.integers(0, seq - 30))
        sid = ids[0, start]
        if sid:
            stop = start
            while stop < seq and stop < start + 40 and ids[0, stop] == sid:
                stop += 1
            ends[0, start:stop] = stop - 1
        allowed = ref.allowed_from_canonical(ids, ends)[0]
        q_summary, kv_summary = ref.block_summaries(ids, bq, bkv, ends)
        for qb in range(seq // bq):
            for kb in range(seq // bkv):
                tile = allowed[qb * bq:(qb + 1) * bq, kb * bkv:(kb + 1) * bkv]
                if tile.any():
                    assert ref.summary_should_run(q_summary, kv_summary, 0, qb, kb, block_q=bq, block_kv=bkv)


def test_attention_end_semantics():
    # tests/training/test_maskgit.py:116-125, :159-163
    seq = 24
    ids = np.array([[1] * 16 + [2] * 8], np.int32)
    start, stop = 4, 10
    ends = ref.attention_end_from_blocks(seq, [(start, stop)])[None]
    allowed = ref.allowed_from_canonical(ids, ends)[0]
    assert allowed[start, stop - 1]
    assert not allowed[start - 1, start]
    assert not allowed[start, stop]
    assert not allowed[ids[0][:, None] != ids[0][None, :]].any()
    plain = ref.allowed_from_canonical(ids, np.arange(seq, dtype=np.int32)[None])
    np.testing.assert_array_equal(plain, ref.allowed_from_canonical(ids))


def test_default_scale_is_representable_choice():
    # tests/kernels/test_efficient_attention.py:387-392: bf16(D ** -0.5)
    for dim in (64, 128, 256):
        value = float(torch.tensor(dim ** -0.5, dtype=torch.bfloat16))
        assert abs(value - dim ** -0.5) <= dim ** -0.5 * 2 ** -8
    assert float(torch.tensor(128 ** -0.5, dtype=torch.bfloat16)) == 0.08837890625


# ---- floating point side --------------------------------------------------------------------
def _brute_force(q, k, v, allowed, scale):
    """Triple loop in Python floats (float64): O and LSE."""

    batch, seq, q_heads, dim = q.shape
    groups = q_heads // k.shape[2]
    out = np.zeros((batch, seq, q_heads, dim))
    lse = np.zeros((batch, seq, q_heads))
    for b in range(batch):
        for h in range(q_heads):
            for i in range(seq):
                keys = [j for j in range(seq) if allowed[b, i, j]]
                if not keys:
                    continue
                scores = [scale * sum(float(q[b, i, h, d]) * float(k[b, j, h // groups, d]) for d in range(dim))
                          for j in keys]
                top = max(scores)
                weights = [math.exp(s - top) for s in scores]
                total = sum(weights)
                lse[b, i, h] = math.log(total) + top
                for wgt, j in zip(weights, keys):
                    for d in range(dim):
                        out[b, i, h, d] += wgt / total * float(v[b, j, h // groups, d])
    return out, lse


def test_f64_attention_matches_brute_force_with_gqa_and_ends():
    rng = np.random.default_rng(3)
    batch, seq, q_heads, kv_heads, dim = 1, 12, 4, 2, 4
    q, k, v = (_bf16(rng.normal(size=s)) for s in ((batch, seq, q_heads, dim), (batch, seq, kv_heads, dim),
                                                   (batch, seq, kv_heads, dim)))
    ids = np.array([[0, 1, 1, 1, 1, 1, 2, 2, 2, 0, 3, 3]], np.int32)
    ends = ref.attention_end_from_blocks(seq, [(2, 5)])[None]
    allowed = ref.allowed_from_canonical(ids, ends)
    scale = float(torch.tensor(0.5, dtype=torch.bfloat16))
    out, lse = ref.attention_f64(q, k, v, allowed, scale=scale)
    expected_out, expected_lse = _brute_force(q.float().numpy(), k.float().numpy(), v.float().numpy(), allowed, scale)
    np.testing.assert_allclose(out.numpy(), expected_out, atol=1e-12)
    np.testing.assert_allclose(lse.numpy(), expected_lse, atol=1e-12)
    # a wrong GQA map (h % Hkv) must fail this pin: heads 1 and 2 read different kv heads
    assert not np.allclose(expected_out[0, :, 1], expected_out[0, :, 2])


def test_f64_backward_matches_autograd():
    rng = np.random.default_rng(4)
    batch, seq, q_heads, kv_heads, dim = 2, 16, 4, 2, 8
    q = _bf16(rng.normal(size=(batch, seq, q_heads, dim)))
    k = _bf16(rng.normal(size=(batch, seq, kv_heads, dim)))
    v = _bf16(rng.normal(size=(batch, seq, kv_heads, dim)))
    dout = _bf16(rng.normal(size=(batch, seq, q_heads, dim)))
    ids = np.array([[1] * 7 + [2] * 6 + [0] * 3, [0] * 2 + [1] * 14], np.int32)
    allowed = ref.allowed_from_canonical(ids)
    scale = 0.25
    _, _, dq, dk, dv = ref.attention_f64(q, k, v, allowed, scale=scale, dout=dout)

    q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
    groups = q_heads // kv_heads
    scores = torch.einsum("bqhd,bkhd->bhqk", q64, k64.repeat_interleave(groups, 2)) * scale
    mask = torch.from_numpy(allowed)[:, None]
    prob = torch.softmax(torch.where(mask, scores, -1e300), dim=-1)
    prob = torch.where(mask.any(-1, keepdim=True), prob, 0.0)
    out = torch.einsum("bhqk,bkhd->bqhd", prob, v64.repeat_interleave(groups, 2))
    out.backward(dout.double())
    np.testing.assert_allclose(dq.numpy(), q64.grad.numpy(), atol=1e-10)
    np.testing.assert_allclose(dk.numpy(), k64.grad.numpy(), atol=1e-10)
    np.testing.assert_allclose(dv.numpy(), v64.grad.numpy(), atol=1e-10)


def test_single_segment_reduces_to_library_causal_attention():
    rng = np.random.default_rng(5)
    batch, seq, heads, dim = 2, 32, 2, 16
    q, k, v = (_bf16(rng.normal(size=(batch, seq, heads, dim))) for _ in range(3))
    ids = np.ones((batch, seq), np.int32)
    allowed = ref.allowed_from_canonical(ids)
    scale = 0.25  # exactly representable in bf16
    out, _ = ref.attention_f64(q, k, v, allowed, scale=scale)
    expected = torch.nn.functional.scaled_dot_product_attention(
        q.double().transpose(1, 2), k.double().transpose(1, 2), v.double().transpose(1, 2),
        is_causal=True, scale=scale).transpose(1, 2)
    np.testing.assert_allclose(out.numpy(), expected.numpy(), atol=1e-10)


def test_bf16_restatements_agree_with_f64_within_rounding():
    rng = np.random.default_rng(6)
    batch, seq, q_heads, kv_heads, dim = 2, 128, 4, 2, 64
    q = _bf16(rng.normal(size=(batch, seq, q_heads, dim)))
    k = _bf16(rng.normal(size=(batch, seq, kv_heads, dim)))
    v = _bf16(rng.normal(size=(batch, seq, kv_heads, dim)))
    dout = _bf16(rng.normal(size=(batch, seq, q_heads, dim)))
    ids = np.zeros((batch, seq), np.int32)
    ids[0, 5:60], ids[0, 60:128] = 1, 2
    ids[1, :100] = 1
    allowed = ref.allowed_from_canonical(ids)
    scale = dim ** -0.5
    out64, lse64, dq64, dk64, dv64 = ref.attention_f64(q, k, v, allowed, scale=scale, dout=dout)
    out, dq, dk, dv = ref.vanilla_attention_vjp(q, k, v, allowed, dout, scale=scale)
    for name, got, want in (("o", out, out64), ("dq", dq, dq64), ("dk", dk, dk64), ("dv", dv, dv64)):
        assert ref.relative_l2(got, want) < 1e-2, name
    out_e, lse_e = ref.efficient_forward(q, k, v, allowed, scale=scale)
    assert ref.relative_l2(out_e, out64) < 5e-3
    # LSE differs from f64 only by the bf16 rounding of q * scale
    assert float((lse_e.double() - lse64).abs().max()) < 2e-2
    grads_e = ref.efficient_backward(q, k, v, allowed, out_e, lse_e, dout, scale=scale)
    for got, want in zip(grads_e, (dq64, dk64, dv64)):
        assert ref.relative_l2(got, want) < 1e-2
    # padding rows: exact zeros (tests/kernels/test_efficient_attention.py:220-223)
    pad = torch.from_numpy(ids == 0)
    for tensor in (out, dq, out_e, grads_e[0]):
        assert (tensor[pad] == 0).all()
    assert (lse_e[pad] == 0).all()


def test_efficient_lse_uses_bf16_prescaled_query():
    # The scale is folded into q in bf16 before the dot product
    # (src/causal_trainer/kernels/efficient_attention.py:906-907).
    q = _bf16(np.full((1, 1, 1, 2), 1.00390625))  # 1 + 2^-8, exactly representable
    k = _bf16(np.ones((1, 1, 1, 2)))
    allowed = np.ones((1, 1, 1), bool)
    scale = 0.08837890625
    expected = float((q[0, 0, 0, 0] * torch.tensor(scale, dtype=torch.bfloat16)).float()) * 2
    got = float(ref.efficient_lse(q, k, allowed, scale=scale))
    assert got == pytest.approx(expected, abs=1e-7)
    assert got != pytest.approx(1.00390625 * scale * 2, abs=1e-7)  # unrounded product differs


def test_isolation_in_both_directions():
    # tests/modeling/test_attention.py:19-58 (values from NumPy instead of jax.random)
    rng = np.random.default_rng(0)
    q = _bf16(rng.normal(size=(1, 6, 4, 2)))
    k = _bf16(rng.normal(size=(1, 6, 1, 2)))
    v = _bf16(rng.normal(size=(1, 6, 1, 2)))
    ids = np.array([[1, 1, 1, 2, 2, 2]], np.int32)
    allowed = ref.allowed_from_canonical(ids)
    scale = 2 ** -0.5
    baseline = ref.vanilla_attention(q, k, v, allowed, scale=scale)
    q2, k2, v2 = q.clone(), k.clone(), v.clone()
    q2[:, 3:], k2[:, 3:], v2[:, 3:] = 100.0, -100.0, 50.0
    later = ref.vanilla_attention(q2, k2, v2, allowed, scale=scale)
    assert torch.equal(later[:, :3], baseline[:, :3])
    q3, k3, v3 = q.clone(), k.clone(), v.clone()
    q3[:, :3], k3[:, :3], v3[:, :3] = -70.0, 80.0, -90.0
    earlier = ref.vanilla_attention(q3, k3, v3, allowed, scale=scale)
    assert torch.equal(earlier[:, 3:], baseline[:, 3:])


def test_bidirectional_dependency_known_answer():
    # tests/training/test_maskgit.py:200-213
    rng = np.random.default_rng(3)
    q, k, v = (_bf16(rng.normal(size=(1, 8, 1, 4))) for _ in range(3))
    ids = np.array([[1, 1, 1, 1, 1, 2, 2, 2]], np.int32)
    ends = np.array([[0, 1, 4, 4, 4, 5, 6, 7]], np.int32)
    allowed = ref.allowed_from_canonical(ids, ends)

    def grad_of_row(row):
        dout = torch.zeros_like(q)
        dout[:, row] = 1.0
        return ref.vanilla_attention_vjp(q, k, v, allowed, dout, scale=0.5)[3].float()

    gradient = grad_of_row(2)
    assert float(gradient[:, 4].norm()) > 0
    assert (gradient[:, 5:] == 0).all()
    assert (grad_of_row(1)[:, 2:] == 0).all()


def test_reference_seeded_fixture_regenerates(tmp_path):
    # tests/kernels/test_efficient_attention.py:187-223, rng = default_rng(931); the committed
    # golden file holds this restatement's outputs on those inputs (restatement-derived).
    from tests.golden import make_golden

    fixture = make_golden.attention_fixture()
    golden = np.load(make_golden.GOLDEN_DIR / "attention_rng931.npz")
    for name in ("q", "k", "v", "dout"):
        np.testing.assert_array_equal(fixture[name].view(torch.int16).numpy(), golden[name])
    np.testing.assert_array_equal(fixture["segment_ids"], golden["segment_ids"])
    allowed = ref.allowed_from_canonical(fixture["segment_ids"])
    out, dq, dk, dv = ref.vanilla_attention_vjp(fixture["q"], fixture["k"], fixture["v"], allowed,
                                                fixture["dout"], scale=128 ** -0.5)
    for name, tensor in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        np.testing.assert_array_equal(tensor.view(torch.int16).numpy(), golden[name])
    seg = fixture["segment_ids"][0]
    # expectations stated by the reference test (:216-223): zeros on padding for all four;
    # dK and dV nonzero inside [71, 128) and zero outside segment 2
    for tensor in (out, dq, dk, dv):
        assert (tensor[:, seg == 0] == 0).all()
    for grad in (dk, dv):
        assert (grad[:, seg != 2] == 0).all()
        assert grad[0, 71:128].float().abs().sum() > 0
    assert (dq[:, seg != 2] == 0).all()


def test_sampled_rows_of_a_segment_agree_with_the_full_restatement():
    """segment_sampled_rows (chunked, sampled) against efficient_forward / efficient_backward
    evaluated on the whole segment, for plain causal and for bidirectional blocks."""

    rng = np.random.default_rng(77)
    length, groups, dim = 300, 3, 64
    for hybrid in (False, True):
        q = _bf16(rng.standard_normal((1, length, groups, dim)))
        k = _bf16(rng.standard_normal((1, length, 1, dim)))
        v = _bf16(rng.standard_normal((1, length, 1, dim)))
        dout = _bf16(rng.standard_normal((1, length, groups, dim)))
        ends = np.arange(length, dtype=np.int32)
        if hybrid:
            ends[40:111] = 110
            ends[200:290] = 289
        ids = np.ones((1, length), np.int32)
        allowed = ref.allowed_from_canonical(ids, ends[None])
        scale = dim ** -0.5
        out, lse = ref.efficient_forward(q, k, v, allowed, scale=scale)
        dq, dk, dv = ref.efficient_backward(q, k, v, allowed, out, lse, dout, scale=scale)
        query_rows = np.sort(rng.choice(length, 37, replace=False))
        key_rows = np.sort(rng.choice(length, 29, replace=False))
        got = ref.segment_sampled_rows(q[0], k[0, :, 0], v[0, :, 0], dout[0], ends, scale=scale,
                                       query_rows=query_rows, key_rows=key_rows, chunk=64)
        torch.testing.assert_close(got[1], lse[0, query_rows], atol=2e-5, rtol=0)
        # the full restatement rounds its results to bf16: half an ulp (2^-9 relative) each
        assert ref.relative_l2(got[0], out[0, query_rows].float()) < 3e-3
        assert ref.relative_l2(got[2], dq[0, query_rows].float()) < 3e-3
        assert ref.relative_l2(got[3], dk[0, key_rows, 0].float()) < 3e-3
        assert ref.relative_l2(got[4], dv[0, key_rows, 0].float()) < 3e-3
