"""CPU-only checks of the host-side mirror and of the C ABI surface (no compute calls)."""

import ctypes
import re
from pathlib import Path

import numpy as np
import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]


def test_library_exports_every_declared_symbol(ct):
    header = (ROOT / "include" / "ct_hotpath.h").read_text()
    declared = set(re.findall(r"\b(ct_[a-z0-9_]+)\s*\(", header))
    assert declared == set(ct._lib.SYMBOLS), declared ^ set(ct._lib.SYMBOLS)
    library = ct._lib.load()
    for name in declared:
        assert hasattr(library, name), name
    assert library.ct_abi_version() == ct._lib.ABI_VERSION
    assert library.ct_last_error() == b"" or isinstance(library.ct_last_error(), bytes)


def test_size_queries_need_no_gpu(ct):
    library = ct._lib.load()
    nrb = 4096 // 32
    bins = sum(33 + 4 * ((nrb + pb - 1) // pb) for pb in (2, 4, 8))
    assert library.ct_attn_meta_bytes(4, 4096) == (4 * (nrb * 12 + 2 * nrb + nrb // 4) + bins) * 4
    assert library.ct_attn_meta_bytes(0, 128) == 0
    # the backward's scratch: the work list, statistics and partial sums alone are small ...
    least = library.ct_attn_bwd_workspace_bytes(4, 4096, 32, 8, 128)
    assert 0 < least < 1 << 30
    assert library.ct_attn_bwd_workspace_bytes(4, 4000, 32, 8, 128) == 0
    assert library.ct_attn_bwd_workspace_bytes_from_ds(4, 4000, 32, 8, 128, 0) == 0
    # ... the stored-dS form adds 2 KB per (key block, query block at or after it) pair of every
    # batch row and query head (nrb^2 pairs with visible ends)
    causal = library.ct_attn_bwd_workspace_bytes_from_ds(4, 4096, 32, 8, 128, 0)
    hybrid = library.ct_attn_bwd_workspace_bytes_from_ds(4, 4096, 32, 8, 128, 1)
    assert causal - least == 4 * 32 * (nrb * (nrb + 1) // 2) * 2048
    assert hybrid - least == 4 * 32 * nrb * nrb * 2048
    # the region is capped at 16 GiB but never below one KV head's blocks: 64 query heads over 8 KV heads
    # at S = 32768 take 8.6 GB per KV head, so the backward runs in 8 passes of one KV head
    long_blocks = (32768 // 32) * (32768 // 32 + 1) // 2
    long_total = library.ct_attn_bwd_workspace_bytes_from_ds(1, 32768, 64, 8, 128, 0)
    long_least = library.ct_attn_bwd_workspace_bytes(1, 32768, 64, 8, 128)
    assert 8 * long_blocks * 2048 <= long_total - long_least + (1 << 30) and long_total < 10 << 30
    # one KV head beyond 64 GiB: that form is not available
    assert library.ct_attn_bwd_workspace_bytes_from_ds(1, 1 << 20, 2, 1, 64, 1) == 0
    shape = ct._lib.CutceShape(16384, 4096, 128256)
    fwd = library.ct_cutce_fwd_workspace_bytes(ctypes.byref(shape))
    full = library.ct_cutce_bwd_workspace_bytes(ctypes.byref(shape))
    least = library.ct_cutce_bwd_workspace_min_bytes(ctypes.byref(shape))
    assert 0 < fwd < 64 << 20
    assert full >= 16384 * 128256 * 2
    assert 0 < least < full


def test_argument_validation_happens_before_any_launch(ct):
    library = ct._lib.load()
    args = ct._lib.AttnFwdArgs(batch=1, seq=100, q_heads=4, kv_heads=2, head_dim=128, scale=0.1)
    assert library.ct_attn_fwd(None, ctypes.byref(args)) == ct._lib.CT_INVALID_ARGUMENT
    assert b"null pointer" in library.ct_last_error()
    for field in ("q", "k", "v", "segment_ids", "tile_meta", "out", "lse"):
        setattr(args, field, 4096)       # never dereferenced: validation fails first
    assert library.ct_attn_fwd(None, ctypes.byref(args)) == ct._lib.CT_INVALID_ARGUMENT
    assert b"128-aligned" in library.ct_last_error()
    args.seq, args.q_heads, args.kv_heads = 128, 5, 2
    assert library.ct_attn_fwd(None, ctypes.byref(args)) == ct._lib.CT_INVALID_ARGUMENT
    assert b"divisible by the KV head count" in library.ct_last_error()
    args.q_heads, args.head_dim = 4, 96
    assert library.ct_attn_fwd(None, ctypes.byref(args)) == ct._lib.CT_UNSUPPORTED
    args.head_dim, args.k = 128, 4096 + 8
    assert library.ct_attn_fwd(None, ctypes.byref(args)) == ct._lib.CT_INVALID_ARGUMENT
    assert b"16-byte aligned" in library.ct_last_error()
    shape = ct._lib.CutceShape(10, 100, 50)
    cargs = ct._lib.CutceFwdArgs(shape=shape)
    for field in ("hidden", "head", "targets", "weights", "nll_sum", "weight_sum", "lse", "workspace"):
        setattr(cargs, field, 4096)
    assert library.ct_cutce_fwd(None, ctypes.byref(cargs)) == ct._lib.CT_INVALID_ARGUMENT
    assert b"divisible by 128" in library.ct_last_error()
    cargs.shape = ct._lib.CutceShape(10, 128, 50)
    cargs.workspace_bytes = 16
    assert library.ct_cutce_fwd(None, ctypes.byref(cargs)) == ct._lib.CT_WORKSPACE_TOO_SMALL


def test_profile_resolution_matches_reference_tiers(ct):
    # tests/kernels/test_efficient_attention.py:226-249: S=4096, 32 heads, tp=4 -> h8, q256, kv 512/256
    profile = ct.resolve_attention_profile((4, 4096, 32, 128), (4, 4096, 1, 128), {"tp": 4})
    assert (profile.block_h, profile.block_q, profile.block_kv_outer, profile.block_kv_compute) == (8, 256, 512, 256)
    long_profile = ct.resolve_attention_profile((1, 32768, 64, 128), (1, 32768, 8, 128), None)
    assert (long_profile.block_kv_outer, long_profile.block_kv_compute) == (1024, 256)
    hybrid = ct.resolve_attention_profile((2, 8192, 16, 128), (2, 8192, 16, 128), None, has_attention_end=True)
    assert hybrid.block_h * hybrid.block_q <= 2048 and hybrid.block_q % 128 == 0
    assert ct.default_attention_scale(128) == 128 ** -0.5
    with pytest.raises(ValueError, match="128-aligned"):
        ct.resolve_attention_profile((1, 100, 2, 128), (1, 100, 1, 128), None)
    with pytest.raises(ValueError, match="divisible by the KV head count"):
        ct.resolve_attention_profile((1, 128, 3, 128), (1, 128, 2, 128), None)


def test_attention_argument_errors(ct):
    q = torch.zeros((1, 128, 2, 128), dtype=torch.bfloat16)
    k = torch.zeros((1, 128, 1, 128), dtype=torch.bfloat16)
    meta = ct.AttentionMetadata(*(torch.zeros((1, 128), dtype=torch.int32),) * 2,
                                torch.zeros((1, 1, 2), dtype=torch.int32),
                                torch.zeros((1, 1, 2), dtype=torch.int32))
    # tests/kernels/test_efficient_attention.py:420-441: non-causal is rejected
    with pytest.raises(ValueError, match="implements causal attention only"):
        ct.efficient_attention(q, k, k, meta, causal=False)
    with pytest.raises(TypeError, match="compile-time bool"):
        ct.efficient_attention(q, k, k, meta, causal=1)
    with pytest.raises(TypeError, match="requires BF16"):
        ct.efficient_attention(q.float(), k.float(), k.float(), meta)
    with pytest.raises(ValueError, match="key and value shapes differ"):
        ct.efficient_attention(q, k, k[:, :64], meta)
    with pytest.raises(ValueError, match="head_dim"):
        ct.efficient_attention(q[..., :32], k[..., :32], k[..., :32], meta)
    with pytest.raises(ValueError, match="one GPU"):
        ct.efficient_attention(q, k, k, meta, mesh={"tp": 2})
    with pytest.raises(RuntimeError, match="only on a ROCm GPU"):
        ct.efficient_attention(q, k, k, meta)


def test_cutce_argument_errors(ct):
    fn = ct.pallas_cut_linear_cross_entropy
    hidden = torch.zeros((1, 4, 128), dtype=torch.bfloat16)
    head = torch.zeros((128, 10), dtype=torch.bfloat16)
    targets = torch.zeros((1, 4), dtype=torch.int32)
    weights = torch.ones((1, 4))
    with pytest.raises(ValueError, match=r"\[batch, sequence, hidden\]"):
        fn(hidden[0], head, targets, weights)
    with pytest.raises(ValueError, match=r"\[hidden, vocab\]"):
        fn(hidden, head.T, targets, weights)
    with pytest.raises(ValueError, match="must match hidden_states"):
        fn(hidden, head, targets[:, :2], weights)
    with pytest.raises(ValueError, match="divisible by 128"):
        fn(hidden[..., :100], head[:100], targets, weights)
    with pytest.raises(TypeError, match="same compute dtype"):
        fn(hidden, head.float(), targets, weights)
    with pytest.raises(TypeError, match="non-negative integer"):
        fn(hidden, head, targets, weights, local_chunk_size=True)
    with pytest.raises(ValueError, match="non-negative"):
        fn(hidden, head, targets, weights, local_chunk_size=-1)
    # tests/kernels/test_tiled_cut.py:158-166: every invalid chunk size names the option
    for invalid in (True, 1.5, "128", -1):
        with pytest.raises((TypeError, ValueError), match="local_chunk_size"):
            fn(hidden, head, targets, weights, local_chunk_size=invalid)
    # the head as [vocab, hidden]: named by the option, checked like the other layout
    with pytest.raises(ValueError, match="head_layout"):
        fn(hidden, head, targets, weights, head_layout="vocab_major")
    with pytest.raises(ValueError, match=r"\[hidden, vocab\]"):
        fn(hidden, head, targets, weights, head_layout="vd")
    with pytest.raises(RuntimeError, match="only on a ROCm GPU"):
        fn(hidden, head.T.contiguous(), targets, weights, head_layout="vd")
    with pytest.raises(RuntimeError, match="only on a ROCm GPU"):
        fn(hidden, head, targets, weights)


def test_local_chunk_size_bounds_the_backward_workspace(ct):
    # cut_cross_entropy.py:697-825: the chunk option exists to bound transient memory
    from causal_trainer_dev_amd.cut_cross_entropy import backward_workspace_bytes

    rows, hidden, vocab = 16384, 4096, 128256
    library = ct._lib.load()
    shape = ct._lib.CutceShape(rows, hidden, vocab)
    full = library.ct_cutce_bwd_workspace_bytes(ctypes.byref(shape))
    least = library.ct_cutce_bwd_workspace_min_bytes(ctypes.byref(shape))
    assert backward_workspace_bytes(rows, hidden, vocab, 0) == full
    assert backward_workspace_bytes(rows, hidden, vocab, rows) == full
    sizes = [backward_workspace_bytes(rows, hidden, vocab, chunk) for chunk in (8192, 2048, 512, 1)]
    assert sizes == sorted(sizes, reverse=True) and all(least <= size < full for size in sizes)
    assert sizes[1] < full // 4 and sizes[-1] < least + (1 << 20)
    # the slab part shrinks in proportion to the chunk
    assert abs((sizes[1] - least) - (full - least) // 8) <= 1


def _ffi_handlers_in_source():
    """name -> (operands, results, attribute names) from the XLA_FFI_DEFINE_HANDLER_SYMBOL blocks."""

    source = (ROOT / "causal-trainer-dev_amd" / "csrc" / "ct_ffi.cc").read_text()
    found = {}
    for block in re.findall(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\((.*?)\);\n", source, flags=re.S):
        name = block.split(",", 1)[0].strip()
        attributes = tuple(re.findall(r'\.Attr<[^>]+>\("(\w+)"\)', block))
        found[name] = (len(re.findall(r"\.Arg<", block)), len(re.findall(r"\.Ret<", block)), attributes)
    return found


def test_jax_binding_matches_the_ffi_handlers_and_the_documentation(ct):
    """The JAX side cannot run here (no jax): what can be held is static agreement between the
    handlers csrc/ct_ffi.cc defines, the table and call sites of jax_ffi.py, and the integration document."""

    import ast
    import inspect

    from causal_trainer_dev_amd import jax_ffi

    in_source = _ffi_handlers_in_source()
    assert len(in_source) == 14
    assert {name: tuple(handler) for name, handler in jax_ffi.HANDLERS.items()} == in_source
    documented = set(re.findall(r"`(ct_ffi_\w+)`", (ROOT / "INTEGRATION.md").read_text()))
    assert documented == set(in_source)

    # every _call site names a known handler and passes the operand / result / attribute counts
    tree = ast.parse(inspect.getsource(jax_ffi))
    sites = [node for node in ast.walk(tree)
             if isinstance(node, ast.Call) and getattr(node.func, "id", None) == "_call"]
    assert len(sites) >= 5
    for site in sites:
        name = site.args[0].value
        operands, results, attributes = in_source[name]
        assert isinstance(site.args[1], ast.List) and len(site.args[1].elts) == results, name
        assert len(site.args) - 2 == operands, name
        assert tuple(keyword.arg for keyword in site.keywords) == attributes, name
    # every registered handler has a caller: no symbol is handed to a maintainer without its glue
    used = {site.args[0].value for site in sites}
    assert used == set(in_source)

    # the operators keep the reference's signatures (efficient_attention.py:326-331, :1890-1900;
    # cut_cross_entropy.py:828-838)
    def parameters(function):
        return [(p.name, p.kind.name, p.default) for p in inspect.signature(function).parameters.values()]

    empty = inspect.Parameter.empty
    assert parameters(jax_ffi.efficient_attention) == [
        ("query", "POSITIONAL_OR_KEYWORD", empty), ("key", "POSITIONAL_OR_KEYWORD", empty),
        ("value", "POSITIONAL_OR_KEYWORD", empty), ("metadata", "POSITIONAL_OR_KEYWORD", empty),
        ("mesh", "KEYWORD_ONLY", empty), ("profile", "KEYWORD_ONLY", None), ("scale", "KEYWORD_ONLY", None),
        ("causal", "KEYWORD_ONLY", True)]
    assert parameters(jax_ffi.prepare_attention_metadata) == [
        ("canonical_segment_ids", "POSITIONAL_OR_KEYWORD", empty), ("mesh", "KEYWORD_ONLY", empty),
        ("profile", "KEYWORD_ONLY", empty), ("attention_end", "KEYWORD_ONLY", None)]
    assert parameters(jax_ffi.pallas_cut_linear_cross_entropy) == [
        ("hidden_states", "POSITIONAL_OR_KEYWORD", empty), ("lm_head_kernel", "POSITIONAL_OR_KEYWORD", empty),
        ("targets", "POSITIONAL_OR_KEYWORD", empty), ("weights", "POSITIONAL_OR_KEYWORD", empty),
        ("mesh", "KEYWORD_ONLY", empty), ("sparse_compaction", "KEYWORD_ONLY", False),
        ("lm_head_trainable", "KEYWORD_ONLY", True), ("local_chunk_size", "KEYWORD_ONLY", 0)]
    # the rows either side of the two paths (rotary.py:13-16, :63-66, :132-136, :160-167, :207-214;
    # architecture.py:155; losses.py:21-30; cross_entropy.py:600-606)
    assert parameters(jax_ffi.canonicalize_segment_ids) == [
        ("attention_mask", "POSITIONAL_OR_KEYWORD", empty), ("segment_ids", "POSITIONAL_OR_KEYWORD", None)]
    assert parameters(jax_ffi.make_position_ids) == parameters(jax_ffi.canonicalize_segment_ids)
    assert parameters(jax_ffi.rotary_cos_sin) == [
        ("position_ids", "POSITIONAL_OR_KEYWORD", empty), ("inv_freq", "POSITIONAL_OR_KEYWORD", empty),
        ("dtype", "POSITIONAL_OR_KEYWORD", empty)]
    assert parameters(jax_ffi.apply_rotary_cos_sin)[:5] == [
        ("query", "POSITIONAL_OR_KEYWORD", empty), ("key", "POSITIONAL_OR_KEYWORD", empty),
        ("cosine", "POSITIONAL_OR_KEYWORD", empty), ("sine", "POSITIONAL_OR_KEYWORD", empty),
        ("rope_style", "KEYWORD_ONLY", "gpt-j")]
    assert parameters(jax_ffi.apply_rotary_embedding) == [
        ("query", "POSITIONAL_OR_KEYWORD", empty), ("key", "POSITIONAL_OR_KEYWORD", empty),
        ("position_ids", "POSITIONAL_OR_KEYWORD", empty), ("inv_freq", "POSITIONAL_OR_KEYWORD", empty),
        ("rope_style", "KEYWORD_ONLY", "gpt-j")]
    assert parameters(jax_ffi.rms_norm) == [
        ("x", "POSITIONAL_OR_KEYWORD", empty), ("scale", "POSITIONAL_OR_KEYWORD", empty),
        ("eps", "POSITIONAL_OR_KEYWORD", empty), ("compute_dtype", "POSITIONAL_OR_KEYWORD", empty)]
    assert parameters(jax_ffi.shifted_targets_and_weights) == [
        ("input_ids", "POSITIONAL_OR_KEYWORD", empty), ("attention_mask", "POSITIONAL_OR_KEYWORD", empty),
        ("segment_ids", "POSITIONAL_OR_KEYWORD", None), ("assistant_mask", "POSITIONAL_OR_KEYWORD", None),
        ("loss_mask", "POSITIONAL_OR_KEYWORD", None), ("labels", "POSITIONAL_OR_KEYWORD", None),
        ("ignore_index", "KEYWORD_ONLY", -100)]
    assert parameters(jax_ffi.pallas_fused_sparse_cross_entropy) == [
        ("logits", "POSITIONAL_OR_KEYWORD", empty), ("targets", "POSITIONAL_OR_KEYWORD", empty),
        ("weights", "POSITIONAL_OR_KEYWORD", empty), ("mesh", "KEYWORD_ONLY", empty)]
    assert jax_ffi.AttentionMetadata._fields[:5] == (
        "query_segment_ids", "kv_segment_ids", "q_block_segments", "kv_block_segments", "attention_end")
    assert jax_ffi.AttentionMetadata._fields[5:] == ("tile_bounds",)
    # a frozen head asks XLA for a placeholder, not for a [d, V] gradient
    source = inspect.getsource(jax_ffi)
    assert "head.shape if lm_head_trainable else (8,)" in source and "np.float32(scale)" in source


def test_workload_generators_and_flop_accounting(ct):
    from oracle import attention_ref

    W = ct.workloads
    config = W.ATTENTION_CONFIGS["packed_small"]
    inputs = W.make_attention_inputs(config)
    ids = inputs["segment_ids"].numpy()
    assert ids.shape == (2, 1024) and inputs["q"].shape == (2, 1024, 8, 64)
    np.testing.assert_array_equal(attention_ref.canonicalize_segment_ids(ids != 0, ids), ids)
    pairs = W.count_allowed_pairs(ids)
    assert pairs == attention_ref.count_allowed_pairs(ids)
    assert W.attention_flops(config, pairs)["total"] == 14 * 64 * 8 * pairs
    rng = np.random.default_rng(0)
    seg, end = W.maskgit_layout(rng, 1, 4096)
    assert W.count_allowed_pairs(seg, end) == attention_ref.count_allowed_pairs(seg, end)
    blocks = np.flatnonzero(end[0] != np.arange(4096))
    assert len(blocks) % 1055 == 0 and len(blocks) > 0  # the last token of a block keeps end == itself
    cfg = W.CUTCE_CONFIGS["llama3_8b_head"]
    assert W.cutce_flops(cfg, 16384)["total"] == 6 * 16384 * 4096 * 128256
    assert W.attention_delta_bytes(W.ATTENTION_CONFIGS["llama3_8b"]) == 2 * 4 * 4096 * 32 * 128 * 2 + 4 * 4 * 4096 * 32
