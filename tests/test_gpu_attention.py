"""GPU parity of the attention hot path (through the C ABI) against oracle/attention_ref.py.

Tolerances are the stated ones: O max-abs <= 2e-2 (bf16), LSE max-abs <= 1e-3 (f32),
dQ / dK / dV relative L2 <= 2e-2; mask handling is exact (zeros are bitwise zeros).
"""

import numpy as np
import pytest
import torch

from oracle import attention_ref as ref

pytestmark = pytest.mark.gpu

O_ATOL, LSE_ATOL, GRAD_RTOL = 2e-2, 1e-3, 2e-2


def _bf16(array):
    return torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)


def _layout(rng, batch, seq, *, holes=False, max_len=200):
    ids = np.zeros((batch, seq), np.int32)
    for row in range(batch):
        position, segment = (int(rng.integers(0, 70)) if holes else 0), 1
        while position < seq:
            length = int(rng.integers(1, max_len))
            if holes and rng.random() < 0.25:
                position += length
                continue
            ids[row, position:position + length] = segment
            position += length
            segment += 1
    return ids


def _random_ends(rng, ids, blocks_per_row=5):
    batch, seq = ids.shape
    ends = np.broadcast_to(np.arange(seq, dtype=np.int32), ids.shape).copy()
    for row in range(batch):
        for _ in range(blocks_per_row):
            start = int(rng.integers(0, seq - 2))
            sid = ids[row, start]
            if sid == 0:
                continue
            stop = start
            limit = start + int(rng.integers(2, 150))
            while stop < seq and stop < limit and ids[row, stop] == sid:
                stop += 1
            ends[row, start:stop] = stop - 1
    return ends


# how the backward of _run_gpu is pinned (set by the bwd_variant fixture; empty = the library's choice)
_BWD = {}


def _run_gpu(ct, device, q, k, v, dout, ids, ends, scale, **bwd):
    profile = ct.resolve_attention_profile(q.shape, k.shape, None, has_attention_end=ends is not None)
    metadata = ct.prepare_attention_metadata(
        torch.from_numpy(ids).to(device), mesh=None, profile=profile,
        attention_end=None if ends is None else torch.from_numpy(ends).to(device))
    qd, kd, vd, dod = (t.to(device) for t in (q, k, v, dout))
    out, lse = ct.attention_forward_with_lse(qd, kd, vd, metadata, scale=scale)
    dq, dk, dv = ct.attention_backward(qd, kd, vd, metadata, out, lse, dod, scale=scale, **(bwd or _BWD))
    torch.cuda.synchronize()
    return tuple(t.cpu() for t in (out, lse, dq, dk, dv))


def _check_against_oracle(results, q, k, v, dout, ids, ends, scale):
    out, lse, dq, dk, dv = results
    allowed = ref.allowed_from_canonical(ids, ends)
    out_ref, dq_ref, dk_ref, dv_ref = ref.vanilla_attention_vjp(q, k, v, allowed, dout, scale=scale)
    lse_ref = ref.efficient_lse(q, k, allowed, scale=scale)
    assert float((out.float() - out_ref.float()).abs().max()) <= O_ATOL
    assert float((lse - lse_ref).abs().max()) <= LSE_ATOL
    for name, got, want in (("dq", dq, dq_ref), ("dk", dk, dk_ref), ("dv", dv, dv_ref)):
        assert ref.relative_l2(got, want) <= GRAD_RTOL, name
    # and against the analytic backward of the kernel being replaced
    for got, want in zip((dq, dk, dv), ref.efficient_backward(q, k, v, allowed, out, lse, dout, scale=scale)):
        assert ref.relative_l2(got, want) <= GRAD_RTOL
    pad = torch.from_numpy(ids == 0)
    assert (out[pad] == 0).all() and (lse[pad] == 0).all()
    assert (dq[pad] == 0).all() and (dk[pad] == 0).all() and (dv[pad] == 0).all()
    for tensor in results:
        assert torch.isfinite(tensor.float()).all()


CASES = [
    # batch, seq, Hq, Hkv, D, holes, ends
    (1, 128, 1, 1, 128, False, False),
    (2, 256, 4, 1, 128, False, False),    # MQA as in the reference kernel
    (2, 512, 8, 2, 128, True, False),     # GQA group 4, padding holes and leading padding
    (1, 512, 2, 2, 128, True, True),      # MHA with bidirectional blocks
    (2, 256, 8, 8, 64, False, False),     # head_dim 64
    (1, 384, 6, 3, 128, True, True),      # group 2
    (1, 256, 3, 1, 64, False, True),      # group 3 (one head per workgroup)
    (1, 384, 16, 2, 128, True, False),    # group 8
]


@pytest.fixture(params=[("narrow", "recompute"), ("wide", "recompute"), ("narrow", "from_ds")],
                ids=["dkv32", "dkv64", "from_ds"])
def bwd_variant(request):
    """Every form of the backward: dQ from a second evaluation of S and dP beside either dK/dV
    kernel (two wavefronts of 32 keys per SIMD, or one wavefront of 64 keys: head dimension 128
    only, other dimensions run the first), and dQ from the dS blocks the narrow dK/dV kernel
    stores. Tests without this fixture run what the library chooses by itself."""

    _BWD.clear()
    _BWD.update(dkv_kernel=request.param[0], dq_form=request.param[1])
    try:
        yield request.param
    finally:
        _BWD.clear()


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d_S%d_Hq%d_Hkv%d_D%d_%s%s" % (
    c[0], c[1], c[2], c[3], c[4], "holes" if c[5] else "packed", "_ends" if c[6] else ""))
def test_forward_backward_match_oracle(ct, gpu, case, bwd_variant):
    batch, seq, q_heads, kv_heads, dim, holes, with_ends = case
    rng = np.random.default_rng(hash(case) % (2 ** 31))
    ids = _layout(rng, batch, seq, holes=holes)
    ends = _random_ends(rng, ids) if with_ends else None
    q = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    k = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    v = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    dout = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    scale = dim ** -0.5
    print("case", case, flush=True)
    results = _run_gpu(ct, gpu, q, k, v, dout, ids, ends, scale)
    _check_against_oracle(results, q, k, v, dout, ids, ends, scale)


def test_several_query_tiles_per_workgroup_with_empty_ones(ct, gpu, bwd_variant):
    """Rows long enough for every forward workgroup to walk several query tiles one after the other
    (a tile's first K rows are copied while the tile before it finishes), with stretches of padding
    that leave whole 64-row tiles without a single key between tiles that have many, over three
    batch rows: the hand-over between tiles, including to and from a tile with nothing to do."""

    rng = np.random.default_rng(77)
    batch, seq = 3, 2048
    ids = np.zeros((batch, seq), np.int32)
    for row in range(batch):
        position, segment = int(rng.integers(0, 200)), 1
        while position < seq:
            length = int(rng.integers(1, 300))
            if rng.random() < 0.3:
                position += int(rng.integers(64, 260))      # padding: up to four whole tiles
                continue
            ids[row, position:position + length] = segment
            position += length
            segment += 1
    blocks = ids.reshape(batch, seq // 64, 64)
    assert ((blocks == 0).all(-1).sum(-1) >= 2).all()       # every row has tiles without any key
    q = _bf16(rng.standard_normal((batch, seq, 4, 128)))
    k = _bf16(rng.standard_normal((batch, seq, 1, 128)))
    v = _bf16(rng.standard_normal((batch, seq, 1, 128)))
    dout = _bf16(rng.standard_normal((batch, seq, 4, 128)))
    scale = 128 ** -0.5
    results = _run_gpu(ct, gpu, q, k, v, dout, ids, None, scale)
    _check_against_oracle(results, q, k, v, dout, ids, None, scale)
    again = _run_gpu(ct, gpu, q, k, v, dout, ids, None, scale)
    for first, second in zip(results, again):
        assert torch.equal(first, second)


@pytest.mark.parametrize("seq,expected", [(4096, "from_ds"), (8192, "narrow"), (16384, "wide")])
def test_default_choices_of_the_backward(ct, gpu, seq, expected):
    """Left to itself the backward takes dQ from stored dS blocks at rows of up to 4096 positions (the
    Python operator then offers the workspace for it) and recomputes S and dP in its dQ kernel
    above, beside the wide dK/dV kernel from 16384 positions on and the narrow one below: seen in
    the kernels the library launches. Every kernel is deterministic, so the default's results are
    bitwise those of the form it chose. The two dK/dV kernels sum in the same order (both start their
    S and dP products from the per-row terms) and give the same bits; the stored-dS form takes delta
    from a pass of its own and sums bf16 dS blocks for dQ, so its results differ in the last bits. With the small workspace the default
    recomputes at any length; asked for by name, the stored-dS form needs a workspace that holds at
    least one KV head's blocks."""

    rng = np.random.default_rng(seq)
    ids = _layout(rng, 1, seq, max_len=3000)
    q, dout = (_bf16(rng.standard_normal((1, seq, 2, 128))) for _ in range(2))
    k, v = (_bf16(rng.standard_normal((1, seq, 1, 128))) for _ in range(2))
    library = ct._lib.load()
    small = int(library.ct_attn_bwd_workspace_bytes(1, seq, 2, 1, 128))
    assert small < int(library.ct_attn_bwd_workspace_bytes_from_ds(1, seq, 2, 1, 128, 0))
    runs = {
        "default": dict(dq_form=None),
        "from_ds": dict(dq_form="from_ds"),
        "narrow": dict(dkv_kernel="narrow", dq_form="recompute"),
        "wide": dict(dkv_kernel="wide", dq_form="recompute"),
    }
    kernels_of = {
        "from_ds": {"attn_dkv_kernel", "attn_dq_blocks_kernel"},
        "narrow": {"attn_dkv_kernel", "attn_dq_kernel"},
        "wide": {"attn_dkv_wide_kernel", "attn_dq_kernel"},
    }
    backward_kernels = set().union(*kernels_of.values())
    results, launched = {}, {}

    def run(name, **pins):
        print("seq", seq, name, flush=True)
        with ct.profiling.KernelTimer() as timer:
            outcome = _run_gpu(ct, gpu, q, k, v, dout, ids, None, 128 ** -0.5, **pins)
        launched[name] = set(timer.durations_ms()) & backward_kernels
        return outcome

    for name, pins in runs.items():
        results[name] = run(name, **pins)
        assert launched[name] == kernels_of[expected if name == "default" else name], (name, launched[name])
    for index in (2, 3, 4):
        assert torch.equal(results["default"][index], results[expected][index])
        assert ref.relative_l2(results["from_ds"][index], results["narrow"][index]) <= 1e-2
    for index in (3, 4):
        assert torch.equal(results["narrow"][index], results["wide"][index])
    assert not torch.equal(results["from_ds"][2], results["narrow"][2])
    if expected == "from_ds":
        recomputed = run("default with the small workspace", dq_form=None, workspace_bytes=small)
        assert launched["default with the small workspace"] == kernels_of["narrow"]
        for index in (2, 3, 4):
            assert torch.equal(recomputed[index], results["narrow"][index])
    with pytest.raises(ct._lib.CtError, match="stored-dS form needs"):
        _run_gpu(ct, gpu, q, k, v, dout, ids, None, 128 ** -0.5, dq_form="from_ds", workspace_bytes=small)
    with pytest.raises(ct._lib.CtError, match="no stored-dS form"):
        _run_gpu(ct, gpu, q, k, v, dout, ids, None, 128 ** -0.5, dq_form="from_ds", dkv_kernel="wide")


@pytest.mark.parametrize("form", ["recompute", "from_ds"])
def test_kept_work_list(ct, gpu, form):
    """Layers that share a packing can share the backward's scratch buffer and the dK/dV work list
    in it (CT_ATTN_BWD_WORK_LIST_KEPT through ct.BackwardWorkspace): the first call builds the list,
    the next ones launch one kernel less and give the same bits, also with other tensors; another
    packing builds it again."""

    from causal_trainer_dev_amd import profiling

    rng = np.random.default_rng(77)
    batch, seq, q_heads, kv_heads, dim = 2, 1024, 4, 2, 128
    scale = dim ** -0.5
    layouts = [_layout(rng, batch, seq, max_len=700), _layout(rng, batch, seq, max_len=300)]
    profile = ct.resolve_attention_profile((batch, seq, q_heads, dim), (batch, seq, kv_heads, dim), None,
                                           has_attention_end=False)
    kept = ct.BackwardWorkspace()
    launches = []
    for ids, layers in ((layouts[0], 3), (layouts[1], 2)):
        metadata = ct.prepare_attention_metadata(torch.from_numpy(ids).to(gpu), mesh=None, profile=profile)
        for layer in range(layers):
            q, dout = (_bf16(rng.standard_normal((batch, seq, q_heads, dim))).to(gpu) for _ in range(2))
            k, v = (_bf16(rng.standard_normal((batch, seq, kv_heads, dim))).to(gpu) for _ in range(2))
            out, lse = ct.attention_forward_with_lse(q, k, v, metadata, scale=scale)
            print("layout", len(launches), "layer", layer, form, flush=True)
            expected = ct.attention_backward(q, k, v, metadata, out, lse, dout, scale=scale, dq_form=form)
            with profiling.KernelTimer() as timer:
                got = ct.attention_backward(q, k, v, metadata, out, lse, dout, scale=scale, dq_form=form,
                                            workspace=kept)
            launches.append(sorted(timer.durations_ms()))
            for a, b in zip(expected, got):
                assert torch.equal(a, b)
    built = ["attn_dkv_schedule_kernel" in names for names in launches]
    assert built == [True, False, False, True, False], launches


@pytest.mark.parametrize("scale", [0.0, 1e-37, -0.09, 1.0])
@pytest.mark.parametrize("dim", [64, 128])
def test_any_finite_scale(ct, gpu, bwd_variant, scale, dim):
    """The operator accepts any finite scale (src/kernels/efficient_attention.py:1947-1957): 0 gives
    uniform attention over the allowed keys (dQ and dK exactly 0), a negative one turns the order of
    the scores around; the dK/dV kernels, which carry the scale in the exponent, must follow. A scale
    so small that lse / scale would overflow (1e-37) behaves like 0: finite results, uniform
    attention, dQ and dK vanishingly small."""

    rng = np.random.default_rng(int(abs(scale) * 100) + dim)
    batch, seq, q_heads, kv_heads = 2, 256, 4, 2
    ids = _layout(rng, batch, seq, holes=True)
    ends = _random_ends(rng, ids)
    # scale 1 needs small scores to stay inside the stated tolerances of bf16 probabilities
    spread = 0.25 if scale == 1.0 else 1.0
    q = _bf16(rng.standard_normal((batch, seq, q_heads, dim)) * spread)
    k = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)) * spread)
    v = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    dout = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    results = _run_gpu(ct, gpu, q, k, v, dout, ids, ends, scale)
    if abs(scale) < 1e-30:
        if scale == 0.0:
            assert not results[2].any() and not results[3].any()
        else:
            assert all(torch.isfinite(t.float()).all() for t in results)
            assert float(results[2].float().abs().max()) <= 1e-30 and float(results[3].float().abs().max()) <= 1e-30
        out, lse, _, _, dv = results
        allowed = ref.allowed_from_canonical(ids, ends)
        out_ref, _, _, dv_ref = ref.vanilla_attention_vjp(q, k, v, allowed, dout, scale=scale)
        assert float((out.float() - out_ref.float()).abs().max()) <= O_ATOL
        assert float((lse - ref.efficient_lse(q, k, allowed, scale=scale)).abs().max()) <= LSE_ATOL
        assert ref.relative_l2(dv, dv_ref) <= GRAD_RTOL
    else:
        _check_against_oracle(results, q, k, v, dout, ids, ends, scale)


def test_edge_layouts(ct, gpu, bwd_variant):
    rng = np.random.default_rng(11)
    batch, seq, q_heads, kv_heads, dim = 4, 256, 4, 2, 128
    ids = np.zeros((batch, seq), np.int32)
    ids[1, :] = 1                       # one full-length segment
    ids[2, 200:] = 1                    # whole leading tiles of padding
    ids[3] = np.arange(seq) % 7 + 1     # ids that are not contiguous runs: length-1 "segments"
    ids[3, 100:160] = 9                 # ... with one real run; row 0 stays all padding
    q = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    k = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    v = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    dout = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    results = _run_gpu(ct, gpu, q, k, v, dout, ids, None, dim ** -0.5)
    _check_against_oracle(results, q, k, v, dout, ids, None, dim ** -0.5)
    assert not results[0][0].any() and not results[2][0].any()


def test_reference_seeded_fixture(ct, gpu):
    # inputs of the reference's tests/kernels/test_efficient_attention.py:187-223; its own bar is
    # relative L2 < 0.03 against vanilla attention
    golden = np.load("tests/golden/attention_rng931.npz")

    def tensor(name):
        return torch.from_numpy(golden[name]).view(torch.bfloat16)

    q, k, v, dout = (tensor(n) for n in ("q", "k", "v", "dout"))
    ids = golden["segment_ids"]
    out, lse, dq, dk, dv = _run_gpu(ct, gpu, q, k, v, dout, ids, None, 128 ** -0.5)
    for name, got in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert ref.relative_l2(got, tensor(name)) < 0.02, name
        assert (got[:, ids[0] == 0] == 0).all()
    assert float((lse - torch.from_numpy(golden["lse"])).abs().max()) <= LSE_ATOL
    for grad in (dk, dv):
        assert grad[0, 71:128].float().abs().sum() > 0
        assert (grad[:, ids[0] != 2] == 0).all()


def test_neighbour_perturbation_leaves_other_segment_bitwise_unchanged(ct, gpu, bwd_variant):
    # reference: tests/kernels/test_efficient_attention_tpu.py:395-424
    rng = np.random.default_rng(21)
    batch, seq, q_heads, kv_heads, dim = 1, 512, 4, 2, 128
    ids = np.zeros((batch, seq), np.int32)
    ids[0, 10:230], ids[0, 230:500] = 1, 2
    q = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    k = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    v = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    dout = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    base = _run_gpu(ct, gpu, q, k, v, dout, ids, None, dim ** -0.5)
    q2, k2, v2, d2 = q.clone(), k.clone(), v.clone(), dout.clone()
    q2[:, 10:230], k2[:, 10:230], v2[:, 10:230], d2[:, 10:230] = 3.0, -2.0, 5.0, -1.0
    other = _run_gpu(ct, gpu, q2, k2, v2, d2, ids, None, dim ** -0.5)
    for a, b in zip(base, other):
        assert torch.equal(a[:, 230:500], b[:, 230:500])
    again = _run_gpu(ct, gpu, q, k, v, dout, ids, None, dim ** -0.5)
    for a, b in zip(base, again):
        assert torch.equal(a, b)        # fixed summation order: bitwise reproducible


def test_zero_cross_segment_mass(ct, gpu, bwd_variant):
    # V carries a one-hot of the key's segment id: any attention mass that leaks to another
    # segment shows up as a nonzero in a column that must be exactly 0.
    rng = np.random.default_rng(31)
    batch, seq, q_heads, kv_heads, dim = 2, 1024, 8, 2, 128
    ids = _layout(rng, batch, seq, holes=True, max_len=120)
    assert ids.max() < dim
    ends = _random_ends(rng, ids, 8)
    q = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    k = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    onehot = np.zeros((batch, seq, kv_heads, dim), np.float32)
    b_idx, s_idx = np.nonzero(ids)
    onehot[b_idx, s_idx, :, ids[b_idx, s_idx]] = 1.0
    v = _bf16(onehot)
    out = _run_gpu(ct, gpu, q, k, v, torch.zeros_like(q), ids, ends, dim ** -0.5)[0].float()
    own = torch.zeros((batch, seq, dim), dtype=torch.bool)
    own[torch.from_numpy(b_idx), torch.from_numpy(s_idx), torch.from_numpy(ids[b_idx, s_idx]).long()] = True
    own = own[:, :, None, :].expand_as(out)
    assert (out[~own] == 0).all()
    valid = torch.from_numpy(ids != 0)
    assert float((out[own].reshape(-1) - 1).abs().max()) <= 2 ** -7     # probabilities sum to 1
    assert own.sum() == valid.sum() * q_heads


def test_custom_vjp_through_autograd(ct, gpu):
    rng = np.random.default_rng(41)
    batch, seq, q_heads, kv_heads, dim = 1, 256, 4, 2, 128
    ids = _layout(rng, batch, seq)
    q, k, v, dout = (_bf16(rng.standard_normal(s)).to(gpu) for s in (
        (batch, seq, q_heads, dim), (batch, seq, kv_heads, dim), (batch, seq, kv_heads, dim),
        (batch, seq, q_heads, dim)))
    profile = ct.resolve_attention_profile(q.shape, k.shape, None)
    metadata = ct.prepare_attention_metadata(torch.from_numpy(ids).to(gpu), mesh=None, profile=profile)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    out = ct.efficient_attention(q, k, v, metadata, mesh=None)
    out.backward(dout)
    lse_out, lse = ct.attention_forward_with_lse(q.detach(), k.detach(), v.detach(), metadata)
    assert torch.equal(out.detach(), lse_out)
    dq, dk, dv = ct.attention_backward(q.detach(), k.detach(), v.detach(), metadata, lse_out, lse, dout)
    assert torch.equal(q.grad, dq) and torch.equal(k.grad, dk) and torch.equal(v.grad, dv)
    with pytest.raises(ValueError, match="metadata.q_block_segments must have shape"):
        ct.efficient_attention(q, k, v, metadata, profile=ct.AttentionKernelProfile(4, 128, 128, 128))


def test_metadata_matches_oracle_bit_exact(ct, gpu):
    rng = np.random.default_rng(51)
    # known answers of the reference first (tests/kernels/test_efficient_attention.py:446-480)
    ids = np.concatenate((np.zeros(130), np.ones(49), np.full(122, 2), np.full(211, 3))).astype(np.int32)[None]
    metadata = ct.prepare_attention_metadata(torch.from_numpy(ids).to(gpu), mesh=None,
                                             profile=ct.AttentionKernelProfile(1, 128, 256, 128))
    assert metadata.q_block_segments.cpu().tolist() == [[[0, 0], [1, 2], [2, 3], [3, 3]]]
    assert metadata.kv_block_segments.cpu().tolist() == [[[1, 2], [2, 3]]]
    for _ in range(5):
        ids = _layout(rng, 2, 1024, holes=True)
        ends = _random_ends(rng, ids, 10)
        metadata = ct.prepare_attention_metadata(
            torch.from_numpy(ids).to(gpu), mesh=None, profile=ct.AttentionKernelProfile(1, 128, 256, 128),
            attention_end=torch.from_numpy(ends).to(gpu))
        q_summary, kv_summary = ref.block_summaries(ids, 128, 256, ends)
        np.testing.assert_array_equal(metadata.q_block_segments.cpu().numpy(), q_summary)
        np.testing.assert_array_equal(metadata.kv_block_segments.cpu().numpy(), kv_summary)
        # tile bounds: every allowed pair lies inside the advertised visit ranges
        bounds = ct.tile_bounds_table(metadata).cpu().numpy()
        allowed = ref.allowed_from_canonical(ids, ends)
        for b in range(2):
            for rb in range(1024 // 32):
                rows = allowed[b, rb * 32:(rb + 1) * 32]
                keys = np.flatnonzero(rows.any(0))
                if len(keys):
                    assert bounds[b, rb, 5] <= keys[0] // 64 and keys[-1] // 64 <= bounds[b, rb, 6]
                cols = allowed[b, :, rb * 32:(rb + 1) * 32]
                queries = np.flatnonzero(cols.any(1))
                if len(queries):
                    assert bounds[b, rb, 7] <= queries[0] // 32 and queries[-1] // 32 <= bounds[b, rb, 8]
                block = ids[b, rb * 32:(rb + 1) * 32]
                assert bounds[b, rb, 2] == (block[0] if (block == block[0]).all() and block[0] != 0 else 0)
        # where the dS blocks of a key block start: exclusive prefix sum of its visitors' range lengths
        for b in range(2):
            visitors = np.where(bounds[b, :, 8] >= bounds[b, :, 7], bounds[b, :, 8] - bounds[b, :, 7] + 1, 0)
            np.testing.assert_array_equal(bounds[b, :, 9], np.concatenate(([0], np.cumsum(visitors)[:-1])))
            assert visitors.sum() <= (1024 // 32) ** 2
        # schedules: permutations, ordered by non-increasing work
        blocks = 1024 // 32
        per_row = 2 * blocks + blocks // 4
        flat = metadata.tile_bounds.cpu().numpy()
        schedules = flat[2 * blocks * 12:2 * blocks * 12 + 2 * per_row].reshape(2, per_row)
        for b in range(2):
            spans = np.where(bounds[b, :, 6] >= bounds[b, :, 5], bounds[b, :, 6] - bounds[b, :, 5] + 1, 0)
            order = schedules[b, :blocks]
            assert sorted(order.tolist()) == list(range(blocks))
            assert (np.diff(spans[order]) <= 0).all()
            for offset, count in ((blocks, blocks // 2), (blocks + blocks // 2, blocks // 4),
                                  (blocks + blocks // 2 + blocks // 4, blocks // 4),
                                  (2 * blocks, (blocks + 7) // 8)):
                assert sorted(schedules[b, offset:offset + count].tolist()) == list(range(count))
        # work bins: every (batch row, query tile) item appears in exactly one of the 32 bins,
        # and the bins are balanced to within the heaviest item (longest-first packing)
        cursor = 2 * blocks * 12 + 2 * per_row
        for tile_blocks in (2, 4, 8):
            tiles_per_row = (blocks + tile_blocks - 1) // tile_blocks
            items = 2 * tiles_per_row
            offsets = flat[cursor:cursor + 33]
            listed = flat[cursor + 33:cursor + 33 + items]
            assert offsets[0] == 0 and offsets[32] == items and (np.diff(offsets) >= 0).all()
            assert sorted(listed.tolist()) == list(range(items))
            work = np.zeros(items, dtype=np.int64)
            for item in range(items):
                b, tile = divmod(item, tiles_per_row)
                rows = bounds[b, tile * tile_blocks:(tile + 1) * tile_blocks]
                first, last = rows[:, 5].min(), rows[:, 6].max()
                work[item] = (last - first + 1 if last >= first else 0) + 3
            loads = np.array([work[listed[offsets[j]:offsets[j + 1]]].sum() for j in range(32)])
            assert loads.max() - loads.min() <= work.max()
            cursor += 33 + items
        assert cursor == flat.size


def test_delta_pass_matches_torch(ct, gpu):
    rng = np.random.default_rng(61)
    rows = 4 * 300 * 3
    for dim in (64, 128):
        out = _bf16(rng.standard_normal((rows, dim))).to(gpu)
        dout = _bf16(rng.standard_normal((rows, dim))).to(gpu)
        delta = torch.empty(rows, dtype=torch.float32, device=gpu)
        ct._lib.check(ct._lib.load().ct_attn_delta(ct._lib.current_stream(), out.data_ptr(), dout.data_ptr(),
                                                   delta.data_ptr(), rows, dim))
        expected = (out.float() * dout.float()).sum(-1)
        torch.testing.assert_close(delta, expected, atol=1e-4, rtol=1e-5)


def test_backward_leaves_delta_and_matches_the_pass_on_its_own(ct, gpu):
    """The backward forms delta = rowsum(out * dout) inside its dQ kernel and leaves -delta in its
    head-major scratch (the dK/dV kernel adds it to its dP blocks); it has to agree with the closed
    form on every row, padding rows and hybrid ends included."""

    rng = np.random.default_rng(67)
    for (batch, seq, hq, hkv, dim, hybrid) in ((2, 256, 4, 1, 128, False), (1, 384, 8, 2, 64, True),
                                                (2, 128, 2, 2, 128, False)):
        ids = _layout(rng, batch, seq, holes=True)
        ends = _random_ends(rng, ids) if hybrid else None
        q = _bf16(rng.standard_normal((batch, seq, hq, dim)))
        k = _bf16(rng.standard_normal((batch, seq, hkv, dim)))
        v = _bf16(rng.standard_normal((batch, seq, hkv, dim)))
        dout = _bf16(rng.standard_normal((batch, seq, hq, dim)))
        profile = ct.resolve_attention_profile(q.shape, k.shape, None, has_attention_end=hybrid)
        metadata = ct.prepare_attention_metadata(
            torch.from_numpy(ids).to(gpu), mesh=None, profile=profile,
            attention_end=None if ends is None else torch.from_numpy(ends).to(gpu))
        qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
        out, lse = ct.attention_forward_with_lse(qd, kd, vd, metadata, scale=dim ** -0.5)
        *_, delta = ct.attention_backward(qd, kd, vd, metadata, out, lse, dod, scale=dim ** -0.5, with_delta=True)
        expected = (out.float() * dod.float()).sum(-1).permute(0, 2, 1)  # [B, Hq, S]
        torch.testing.assert_close(-delta, expected, atol=1e-4, rtol=1e-5)


def test_split_key_tiles_match_oracle(ct, gpu, bwd_variant):
    """One 2048-position segment, one KV head, a small batch: the dK/dV work list is far below
    one compute slot's share, so the chunk target sits at its minimum and the key tiles with the
    longest query lists are split into several chunks whose f32 partial sums the reduce kernel
    adds. Checked against the oracle like any other case, and for run-to-run equality."""

    rng = np.random.default_rng(71)
    batch, seq, q_heads, kv_heads, dim = 1, 2048, 2, 1, 128
    ids = np.ones((batch, seq), np.int32)
    ids[0, 2000:] = 0
    q = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    k = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    v = _bf16(rng.standard_normal((batch, seq, kv_heads, dim)))
    dout = _bf16(rng.standard_normal((batch, seq, q_heads, dim)))
    # 16 key tiles of 128; the first has (2048 / 32) * 2 = 128 (head, query block) items against
    # a minimum chunk of 16: it is cut into 8 chunks
    results = _run_gpu(ct, gpu, q, k, v, dout, ids, None, dim ** -0.5)
    _check_against_oracle(results, q, k, v, dout, ids, None, dim ** -0.5)
    again = _run_gpu(ct, gpu, q, k, v, dout, ids, None, dim ** -0.5)
    for a, b in zip(results, again):
        assert torch.equal(a, b)


def _visit_ranges_of_canonical_ids(ids_row, ends_row):
    """Columns 5..8 of the tile table (first / last 64-key tile a 32-row query block visits, first /
    last query block that visits a 32-key block) for one row of canonical ids, i.e. nonzero ids
    that never decrease along the sequence. Two blocks interact iff both hold a nonzero id, their
    id ranges overlap and the key block starts at or before the query block's largest visible
    end (the skip test of src/kernels/efficient_attention.py:377-412); with non-decreasing ids the
    blocks whose id range overlaps a given range are consecutive among the blocks that hold an id,
    so each bound is a binary search."""

    seq = len(ids_row)
    big = np.iinfo(np.int32).max

    def summary(block):
        blocks = ids_row.reshape(-1, block)
        has = (blocks != 0).any(1)
        return has, np.where(blocks != 0, blocks, big).min(1), blocks.max(1)

    nrb, nt = seq // 32, seq // 64
    q_has, q_min, q_max = summary(32)
    end_max = np.where(ids_row != 0, ends_row, -1).reshape(-1, 32).max(1)
    out = np.empty((nrb, 4), np.int64)
    t_has, t_min, t_max = summary(64)
    tiles = np.flatnonzero(t_has)
    lo = np.searchsorted(t_max[tiles], q_min, "left")                       # first tile with max >= q_min
    hi = np.searchsorted(t_min[tiles], q_max, "right") - 1                  # last tile with min <= q_max
    hi = np.minimum(hi, np.searchsorted(tiles, np.minimum(end_max // 64, nt - 1), "right") - 1)
    some = q_has & (lo <= hi) & (lo < len(tiles))
    out[:, 0] = np.where(some, tiles[np.minimum(lo, len(tiles) - 1)], big)
    out[:, 1] = np.where(some, tiles[np.clip(hi, 0, len(tiles) - 1)], -1)
    # as keys: query blocks qb with overlapping ids and end_max[qb] >= first key of this block.
    # end_max is not monotone (bidirectional blocks), so the reach condition is applied on the
    # candidates' running maximum from the right / left.
    blocks = np.flatnonzero(q_has)
    b_min, b_max, b_end = q_min[blocks], q_max[blocks], end_max[blocks]
    first = np.searchsorted(b_max, q_min, "left")
    last = np.searchsorted(b_min, q_max, "right") - 1
    key_start = np.arange(nrb) * 32
    for rb in np.flatnonzero(q_has):
        cand = np.arange(first[rb], last[rb] + 1)
        ok = cand[b_end[cand] >= key_start[rb]]
        out[rb, 2] = blocks[ok[0]] if len(ok) else big
        out[rb, 3] = blocks[ok[-1]] if len(ok) else -1
    out[~q_has, 2], out[~q_has, 3] = big, -1
    return out


def test_million_token_sequence(ct, gpu):
    """S = 1 048 576 (the longest sequence the reference's tests compile,
    tests/kernels/test_efficient_attention_tpu.py:195-231): the metadata kernels keep their
    working arrays in the scratch region of the metadata buffer instead of LDS. Tile table
    against the oracle's summaries and the closed form of the visit ranges, schedules and
    bins as permutations, then a forward + backward with short segments against the oracle on
    a window of whole segments."""

    rng = np.random.default_rng(81)
    # the closed form of the visit ranges, pinned by brute force on a short row first
    small = _layout(rng, 1, 2048, holes=True)
    small_ends = _random_ends(rng, small, 12)
    want = _visit_ranges_of_canonical_ids(small[0], small_ends[0])
    allowed_blocks = np.zeros((64, 32), bool), np.zeros((64, 64), bool)
    meta_small = ct.prepare_attention_metadata(torch.from_numpy(small).to(gpu), mesh=None,
                                               profile=ct.AttentionKernelProfile(1, 128, 256, 128),
                                               attention_end=torch.from_numpy(small_ends).to(gpu))
    np.testing.assert_array_equal(ct.tile_bounds_table(meta_small).cpu().numpy()[0, :, 5:9], want)
    del allowed_blocks

    seq, q_heads, kv_heads, dim = 1 << 20, 2, 1, 64
    ids = _layout(rng, 1, seq, holes=True, max_len=1500)
    ends = _random_ends(rng, ids, 400)
    print("million-token metadata", flush=True)
    metadata = ct.prepare_attention_metadata(torch.from_numpy(ids).to(gpu), mesh=None,
                                             profile=ct.AttentionKernelProfile(1, 128, 256, 128),
                                             attention_end=torch.from_numpy(ends).to(gpu))
    torch.cuda.synchronize()
    q_summary, kv_summary = ref.block_summaries(ids, 128, 256, ends)
    np.testing.assert_array_equal(metadata.q_block_segments.cpu().numpy(), q_summary)
    np.testing.assert_array_equal(metadata.kv_block_segments.cpu().numpy(), kv_summary)
    bounds = ct.tile_bounds_table(metadata).cpu().numpy()[0]
    blocks = seq // 32
    per_block = ids.reshape(blocks, 32)
    np.testing.assert_array_equal(bounds[:, 1], per_block.max(1))
    np.testing.assert_array_equal(bounds[:, 5:9], _visit_ranges_of_canonical_ids(ids[0], ends[0]))
    visitors = np.where(bounds[:, 8] >= bounds[:, 7], bounds[:, 8] - bounds[:, 7] + 1, 0).astype(np.int64)
    np.testing.assert_array_equal(bounds[:, 9], np.minimum(np.concatenate(([0], np.cumsum(visitors)[:-1])),
                                                           2 ** 31 - 1))
    flat = metadata.tile_bounds.cpu().numpy()
    per_row = 2 * blocks + blocks // 4
    schedules = flat[blocks * 12:blocks * 12 + per_row]
    spans = np.where(bounds[:, 6] >= bounds[:, 5], bounds[:, 6] - bounds[:, 5] + 1, 0)
    order = schedules[:blocks]
    assert np.array_equal(np.sort(order), np.arange(blocks)) and (np.diff(spans[order]) <= 0).all()
    cursor = blocks * 12 + per_row
    for tile_blocks in (2, 4, 8):
        items = (blocks + tile_blocks - 1) // tile_blocks
        offsets = flat[cursor:cursor + 33]
        listed = flat[cursor + 33:cursor + 33 + items]
        assert offsets[0] == 0 and offsets[32] == items and (np.diff(offsets) >= 0).all()
        assert np.array_equal(np.sort(listed), np.arange(items))
        first = bounds[:, 5].reshape(items, tile_blocks).min(1)
        last = bounds[:, 6].reshape(items, tile_blocks).max(1)
        work = np.where(last >= first, last - first + 1, 0) + 3
        loads = np.add.reduceat(work[listed], offsets[:32])
        assert loads.max() - loads.min() <= work.max()
        cursor += 33 + items
    assert cursor <= flat.size          # what follows is the kernels' scratch region

    print("million-token attention", flush=True)
    q = _bf16(rng.standard_normal((1, seq, q_heads, dim), dtype=np.float32))
    k = _bf16(rng.standard_normal((1, seq, kv_heads, dim), dtype=np.float32))
    v = _bf16(rng.standard_normal((1, seq, kv_heads, dim), dtype=np.float32))
    dout = _bf16(rng.standard_normal((1, seq, q_heads, dim), dtype=np.float32))
    out, lse, dq, dk, dv = _run_gpu(ct, gpu, q, k, v, dout, ids, ends, dim ** -0.5)
    pad = torch.from_numpy(ids == 0)
    for tensor in (out, lse, dq, dk, dv):
        assert torch.isfinite(tensor.float()).all() and (tensor[pad] == 0).all()
    for origin in (0, seq // 2 + 77, seq - 5000):
        start, stop = _self_contained_window(ids[0, origin:origin + 5000], 4096)
        window = slice(origin + start, origin + stop)
        got = tuple(t[:, window] for t in (out, lse, dq, dk, dv))
        _check_against_oracle(got, q[:, window], k[:, window], v[:, window], dout[:, window], ids[:, window],
                              ends[:, window] - window.start, dim ** -0.5)


def _longest_segment(ids):
    """(batch row, start, stop) of the longest run of one nonzero id."""

    best = (0, 0, 0)
    for row in range(ids.shape[0]):
        cuts = np.flatnonzero(np.diff(ids[row])) + 1
        edges = np.concatenate(([0], cuts, [ids.shape[1]]))
        for a, c in zip(edges[:-1], edges[1:]):
            if ids[row, a] != 0 and c - a > best[2] - best[1]:
                best = (row, int(a), int(c))
    return best


def _self_contained_window(ids_row, limit):
    """Largest run of whole segments (and padding) of at most `limit` positions: (start, stop)."""

    seq = len(ids_row)
    cuts = [0] + [i for i in range(1, seq) if ids_row[i] != ids_row[i - 1]] + [seq]
    best = (0, 0)
    for a in range(len(cuts) - 1):
        for c in range(a + 1, len(cuts)):
            if cuts[c] - cuts[a] > limit:
                break
            if cuts[c] - cuts[a] > best[1] - best[0]:
                best = (cuts[a], cuts[c])
    return best


@pytest.mark.parametrize("name", ["packed_small", "llama3_8b", "maskgit", "long_70b"])
def test_benchmark_shapes(ct, gpu, name, bwd_variant):
    """Full benchmark shapes: size-independent properties everywhere, and the oracle on a
    self-contained window (whole segments) of one KV head with its query group."""

    W = ct.workloads
    config = W.ATTENTION_CONFIGS[name]
    inputs = W.make_attention_inputs(config)
    ids = inputs["segment_ids"].numpy()
    ends = None if inputs["attention_end"] is None else inputs["attention_end"].numpy()
    print("shape", name, flush=True)
    out, lse, dq, dk, dv = _run_gpu(ct, gpu, inputs["q"], inputs["k"], inputs["v"], inputs["dout"], ids, ends,
                                    config.scale)
    pad = torch.from_numpy(ids == 0)
    for tensor in (out, lse, dq, dk, dv):
        assert torch.isfinite(tensor.float()).all()
        assert (tensor[pad] == 0).all()
    assert (lse[~pad] != 0).any()

    # The oracle on three (batch row, KV head) pairs: the first, the last and one drawn at random
    # (workgroups, work bins and split chunks place different rows and heads differently).
    group = config.q_heads // config.kv_heads
    pick = np.random.default_rng(config.seed + 1)
    corners = [(0, 0), (config.batch - 1, config.kv_heads - 1),
               (int(pick.integers(config.batch)), int(pick.integers(config.kv_heads)))]
    for index, (b, kvh) in enumerate(dict.fromkeys(corners)):
        heads = slice(kvh * group, (kvh + 1) * group)
        # a self-contained window (whole segments) of this row
        start, stop = _self_contained_window(ids[b], 4096)
        assert stop - start >= 512, "no whole segment short enough for the oracle"
        window = slice(start, stop)
        w_ids = ids[b:b + 1, window]
        w_ends = None if ends is None else ends[b:b + 1, window] - start
        q = inputs["q"][b:b + 1, window, heads]
        k = inputs["k"][b:b + 1, window, kvh:kvh + 1]
        v = inputs["v"][b:b + 1, window, kvh:kvh + 1]
        dout = inputs["dout"][b:b + 1, window, heads]
        got = (out[b:b + 1, window, heads], lse[b:b + 1, window, heads], dq[b:b + 1, window, heads],
               dk[b:b + 1, window, kvh:kvh + 1], dv[b:b + 1, window, kvh:kvh + 1])
        print("window", name, b, kvh, start, stop, flush=True)
        _check_against_oracle(got, q, k, v, dout, w_ids, w_ends, config.scale)

        # The longest segment of this row (up to the whole sequence): sampled query rows with every
        # head of the group for O, LSE and dQ; sampled key rows for dK and dV, which sum over every
        # query of the segment and every head of the group.
        _, start, stop = _longest_segment(ids[b:b + 1])
        length = stop - start
        assert length >= 64
        samples = 64 if index == 0 else 32
        edge = np.array([0, 1, 31, 32, 63, 64, 127, 128, length - 129, length - 65, length - 33, length - 2,
                         length - 1])
        edge = edge[(edge >= 0) & (edge < length)]
        query_rows = np.unique(np.concatenate((edge, pick.choice(length, samples - len(edge), replace=False))))
        key_rows = np.unique(np.concatenate((edge, pick.choice(length, samples - len(edge), replace=False))))
        seg_ends = (np.arange(length) if ends is None else ends[b, start:stop] - start)
        want = ref.segment_sampled_rows(
            inputs["q"][b, start:stop, heads], inputs["k"][b, start:stop, kvh], inputs["v"][b, start:stop, kvh],
            inputs["dout"][b, start:stop, heads], seg_ends, scale=config.scale, query_rows=query_rows,
            key_rows=key_rows)
        print("longest segment", name, b, kvh, start, stop, flush=True)
        rows, cols = start + query_rows, start + key_rows
        assert float((out[b, rows][:, heads].float() - want[0]).abs().max()) <= O_ATOL
        assert float((lse[b, rows][:, heads] - want[1]).abs().max()) <= LSE_ATOL
        assert ref.relative_l2(dq[b, rows][:, heads], want[2]) <= GRAD_RTOL
        assert ref.relative_l2(dk[b, cols, kvh], want[3]) <= GRAD_RTOL
        assert ref.relative_l2(dv[b, cols, kvh], want[4]) <= GRAD_RTOL
