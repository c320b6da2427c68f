"""GPU parity of the logits-level sparse cross-entropy (through the C ABI) against the oracle.

Tolerances: per-row loss and lse within 1e-5 relative + 1e-5 absolute of the f32 oracle (both sum
~1e5 f32 terms in different orders); summed loss within the reference's own 8e-3 (it is far inside);
bf16 gradients within one unit in the last place of the oracle's, f32 gradients 1e-6 absolute.
The ignored set (target -100 or weight 0) is exact: loss, lse and gradient rows are exactly 0.
"""

import numpy as np
import pytest
import torch

from oracle import cutce_ref

pytestmark = pytest.mark.gpu


def _case(rng, rows, vocab, dtype, scale=0.25):
    logits = torch.from_numpy((rng.standard_normal((rows, vocab)) * scale).astype(np.float32)).to(dtype)
    targets = torch.from_numpy(rng.integers(0, vocab, size=rows).astype(np.int32))
    weights = torch.from_numpy(rng.choice([0.0, 0.25, 0.5, 1.0, 2.0], size=rows).astype(np.float32))
    return logits, targets, weights


def _run(ct, gpu, logits, targets, weights, cot):
    x = logits.to(gpu)[None].requires_grad_(True)
    loss = ct.pallas_fused_sparse_cross_entropy(x, targets.to(gpu)[None], weights.to(gpu)[None], mesh=None)
    loss.backward(cot.to(gpu)[None])
    return loss[0].detach().cpu(), x.grad[0].cpu()


def test_reference_test_setup_value_and_gradient(ct, gpu):
    # reference tests/kernels/test_cross_entropy_tpu.py:50-98: vocab 1280 (not a multiple of the
    # reference's 128-lane tile times TP), 256 rows, weight 0.5 on the first 96, target 220 valid
    rng = np.random.default_rng(0)
    logits = torch.from_numpy((rng.standard_normal((256, 1280)) * 0.25).astype(np.float32)).to(torch.bfloat16)
    targets = torch.from_numpy(rng.integers(0, 1280, size=256).astype(np.int32))
    targets[0] = 220
    weights = torch.where(torch.arange(256) < 96, torch.tensor(0.5), torch.tensor(0.0))
    cot = torch.ones(256)
    loss, grad = _run(ct, gpu, logits, targets, weights, cot)
    want = cutce_ref.xla_sparse_cross_entropy(logits, targets, weights)
    want_grad = cutce_ref.xla_sparse_cross_entropy_vjp(logits, targets, weights, cot)
    assert abs(float(loss.sum()) - float(want.sum())) <= 8e-3          # the reference's own bound
    np.testing.assert_allclose(grad.float().numpy(), want_grad.float().numpy(), rtol=0.0, atol=3e-3)
    torch.testing.assert_close(loss, want, rtol=1e-5, atol=1e-5)
    assert torch.equal(loss[96:], torch.zeros(160)) and float(grad[96:].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,vocab", [(1, 1), (3, 7), (17, 1000), (64, 4096), (33, 128256), (5, 185600),
                                        (9, 32003)])
def test_matches_oracle(ct, gpu, dtype, rows, vocab):
    rng = np.random.default_rng(rows * 1009 + vocab)
    logits, targets, weights = _case(rng, rows, vocab, dtype, scale=2.0)
    if rows > 2:
        targets[0] = -100                  # ignored by the index rule
        targets[1] = vocab + 5             # counted row, target outside the vocabulary
        weights[1] = 1.0
    cot = torch.from_numpy(rng.standard_normal(rows).astype(np.float32))
    loss, grad = _run(ct, gpu, logits, targets, weights, cot)
    want_loss, _ = cutce_ref.pallas_sparse_cross_entropy(logits, targets, weights)
    want_grad = cutce_ref.pallas_sparse_cross_entropy_vjp(logits, targets, weights, cot)
    torch.testing.assert_close(loss, want_loss, rtol=1e-5, atol=1e-5)
    ignored = (targets == -100) | (weights == 0)
    assert torch.equal(loss[ignored], torch.zeros(int(ignored.sum())))
    assert float(grad[ignored].abs().max()) == 0.0 if bool(ignored.any()) else True
    if dtype == torch.float32:
        torch.testing.assert_close(grad, want_grad, rtol=1e-4, atol=1e-6)
    else:
        # one bf16 unit in the last place of the oracle's value (2^-7 relative), plus f32 noise
        diff = (grad.float() - want_grad.float()).abs()
        assert bool((diff <= 2.0 ** -7 * want_grad.float().abs() + 1e-7).all())
        assert float((diff > 0).float().mean()) < 5e-3


def test_full_size_properties(ct, gpu):
    # BASELINE-size logits [16384, 128256] bf16 would be 4.2 GB; 4096 rows keep the test in seconds.
    # Size-independent properties: gradient rows sum to ~0 (softmax sums to 1), lse of a row of
    # equal logits is log V, ignored rows are exactly 0.
    rows, vocab = 4096, 128256
    g = torch.Generator(device="cuda").manual_seed(3)
    logits = torch.randn((1, rows, vocab), generator=g, device=gpu).bfloat16()
    logits[0, 7] = 1.5
    targets = torch.randint(0, vocab, (1, rows), generator=g, device=gpu, dtype=torch.int32)
    weights = (torch.rand((1, rows), generator=g, device=gpu) > 0.3).float()
    weights[0, 7] = 1.0
    x = logits.clone().requires_grad_(True)
    loss = ct.pallas_fused_sparse_cross_entropy(x, targets, weights, mesh=None)
    loss.sum().backward()
    assert abs(float(loss[0, 7]) - (float(np.log(vocab)))) < 1e-4       # lse - 1.5 with logits = 1.5
    ignored = weights[0] == 0
    assert float(loss[0][ignored].abs().max()) == 0.0 and float(x.grad[0][ignored].abs().max()) == 0.0
    sums = x.grad[0].float().sum(-1)
    assert float(sums.abs().max()) < 2e-2                                # bf16 rounding of 128256 terms


def test_argument_errors(ct, gpu):
    logits = torch.zeros((2, 3, 8), dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError, match="Pallas CE expects logits"):
        ct.pallas_fused_sparse_cross_entropy(logits[0], torch.zeros((3,), device=gpu), torch.zeros((3,), device=gpu))
    with pytest.raises(ValueError, match="Pallas CE expects logits"):
        ct.pallas_fused_sparse_cross_entropy(logits, torch.zeros((2, 4), device=gpu), torch.zeros((2, 4), device=gpu))
    out = ct.pallas_fused_sparse_cross_entropy(logits[:, :0], torch.zeros((2, 0), device=gpu),
                                               torch.zeros((2, 0), device=gpu))
    assert out.shape == (2, 0)
