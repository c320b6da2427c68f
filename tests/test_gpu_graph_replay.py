"""The hot paths under HIP graph capture: every entry point only enqueues kernels on the stream it
is given (no allocation, no memset node, no synchronisation), so a captured forward + backward
must replay correctly. Each replay is checked against the eager result on fresh inputs, with the
program's own eager work and synchronisations between the replays."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _bf16(array):
    return torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)


def test_attention_forward_backward_replay(ct, gpu):
    rng = np.random.default_rng(5)
    batch, seq, q_heads, kv_heads, dim = 2, 512, 8, 2, 128
    ids = np.zeros((batch, seq), np.int32)
    ids[0, :300], ids[0, 300:490] = 1, 2
    ids[1, 17:200], ids[1, 200:512] = 1, 2
    profile = ct.resolve_attention_profile((batch, seq, q_heads, dim), (batch, seq, kv_heads, dim), None,
                                           has_attention_end=False)
    metadata = ct.prepare_attention_metadata(torch.from_numpy(ids).to(gpu), mesh=None, profile=profile)
    scale = dim ** -0.5

    def fresh():
        return (_bf16(rng.standard_normal((batch, seq, q_heads, dim))).to(gpu),
                _bf16(rng.standard_normal((batch, seq, kv_heads, dim))).to(gpu),
                _bf16(rng.standard_normal((batch, seq, kv_heads, dim))).to(gpu),
                _bf16(rng.standard_normal((batch, seq, q_heads, dim))).to(gpu))

    def step(q, k, v, dout):
        out, lse = ct.attention_forward_with_lse(q, k, v, metadata, scale=scale)
        dq, dk, dv = ct.attention_backward(q, k, v, metadata, out, lse, dout, scale=scale)
        return out, lse, dq, dk, dv

    static = fresh()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm-up outside the capture, as torch asks
        step(*static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(*static)
    for _ in range(3):
        inputs = fresh()
        eager = step(*inputs)              # the program's own eager work between replays
        torch.cuda.synchronize()
        for slot, value in zip(static, inputs):
            slot.copy_(value)
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want)


def test_cut_cross_entropy_replay(ct, gpu):
    rng = np.random.default_rng(6)
    rows, width, vocab = 700, 256, 3000

    def fresh():
        hidden = _bf16(rng.normal(scale=0.5, size=(rows, width))).to(gpu)
        head = _bf16(rng.normal(scale=0.05, size=(width, vocab))).to(gpu)
        targets = torch.from_numpy(rng.integers(vocab, size=rows).astype(np.int32)).to(gpu)
        weights = torch.from_numpy(rng.choice(np.asarray([0, 0.5, 1], np.float32), size=rows)).to(gpu)
        return hidden, head, targets, weights

    dy = torch.tensor([0.37], dtype=torch.float32, device=gpu)

    def step(hidden, head, targets, weights):
        nll, weight_sum, lse = ct.cutce_forward(hidden, head, targets, weights, sparse_compaction=True)
        dhidden, dhead = ct.cutce_backward(hidden, head, targets, weights, lse, dy, sparse_compaction=True)
        return nll.reshape(1), weight_sum.reshape(1), lse, dhidden, dhead

    static = fresh()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(*static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(*static)
    for _ in range(3):
        inputs = fresh()
        eager = step(*inputs)
        torch.cuda.synchronize()
        for slot, value in zip(static, inputs):
            slot.copy_(value)
        graph.replay()
        torch.cuda.synchronize()
        # the loss sum, lse and dHidden do not depend on which workgroup took which unit; dHead's
        # f32 sums do not either (one workgroup per output tile), so replays match eager bit for bit
        for got, want in zip(captured, eager):
            assert torch.equal(got, want)
