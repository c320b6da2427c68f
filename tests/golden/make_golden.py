"""Regenerates the golden fixtures under tests/golden/.

The reference's JAX code cannot be imported in this environment, so the vectors are
*restatement-derived*: the inputs are the reference tests' own NumPy-seeded fixtures,
regenerated bit for bit, and the expected outputs come from oracle/ on those inputs.

  attention_rng931.npz  inputs of tests/kernels/test_efficient_attention.py:187-196
                        (rng = default_rng(931), draw order q, k, v, dO; batch 2, tp = sp = 1)
  cutce_rng460.npz      inputs of tests/kernels/test_tiled_cut.py:74-86
                        (rng = default_rng(460), draw order hidden, W, targets, weights)

Run from the repository root:  python -m tests.golden.make_golden
"""

from __future__ import annotations

from pathlib import Path

import numpy as np
import torch

GOLDEN_DIR = Path(__file__).resolve().parent


def _bf16(array) -> torch.Tensor:
    # float64 -> float32 -> bf16, both round-to-nearest-even
    return torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)


def _bits(tensor: torch.Tensor) -> np.ndarray:
    return tensor.contiguous().view(torch.int16).numpy()


def attention_fixture(batch: int = 2, heads: int = 2) -> dict:
    rng = np.random.default_rng(931)
    seq, dim = 256, 128
    q = _bf16(rng.normal(scale=0.05, size=(batch, seq, heads, dim)))
    k = _bf16(rng.normal(scale=0.05, size=(batch, seq, 1, dim)))
    v = _bf16(rng.normal(scale=0.05, size=(batch, seq, 1, dim)))
    positions = np.arange(seq)
    segment_row = np.where(positions < 17, 0, np.where(positions < 71, 1, np.where(positions < 211, 2, 3)))
    segment_ids = np.broadcast_to(segment_row.astype(np.int32), (batch, seq)).copy()
    dout = rng.normal(scale=0.02, size=(batch, seq, heads, dim))
    dout = np.where(((positions >= 160) & (positions < 211))[None, :, None, None], dout, 0.0)
    return {"q": q, "k": k, "v": v, "dout": _bf16(dout), "segment_ids": segment_ids}


def cutce_fixture(batch: int = 2, sequence: int = 386, vocab: int = 258) -> dict:
    rng = np.random.default_rng(460)
    hidden = _bf16(rng.normal(scale=0.06, size=(batch, sequence, 128)))
    head = _bf16(rng.normal(scale=0.05, size=(128, vocab)))
    targets = rng.integers(vocab, size=(batch, sequence), dtype=np.int32)
    weights = rng.choice(np.asarray([0.0, 0.25, 1.0, 2.0], np.float32), size=(batch, sequence)).astype(np.float32)
    weights[:, :17] = 0
    weights[:, 71:72] = 0
    weights[:, 121:159] = 0
    targets[weights == 0] = -100
    return {"hidden": hidden, "head": head, "targets": targets, "weights": weights, "cotangent": 0.37}


def main() -> None:
    from oracle import attention_ref, cutce_ref

    fixture = attention_fixture()
    allowed = attention_ref.allowed_from_canonical(fixture["segment_ids"])
    out, dq, dk, dv = attention_ref.vanilla_attention_vjp(
        fixture["q"], fixture["k"], fixture["v"], allowed, fixture["dout"], scale=128 ** -0.5)
    lse = attention_ref.efficient_lse(fixture["q"], fixture["k"], allowed, scale=128 ** -0.5)
    np.savez_compressed(
        GOLDEN_DIR / "attention_rng931.npz",
        q=_bits(fixture["q"]), k=_bits(fixture["k"]), v=_bits(fixture["v"]), dout=_bits(fixture["dout"]),
        segment_ids=fixture["segment_ids"], out=_bits(out), dq=_bits(dq), dk=_bits(dk), dv=_bits(dv),
        lse=lse.numpy(),
    )

    fixture = cutce_fixture()
    hidden = fixture["hidden"].reshape(-1, 128)
    targets = torch.from_numpy(fixture["targets"].reshape(-1))
    weights = torch.from_numpy(fixture["weights"].reshape(-1))
    nll, weight_sum, lse = cutce_ref.cut_forward(hidden, fixture["head"], targets, weights)
    dhidden, dhead = cutce_ref.cut_backward(hidden, fixture["head"], targets, weights, lse, fixture["cotangent"])
    np.savez_compressed(
        GOLDEN_DIR / "cutce_rng460.npz",
        hidden=_bits(fixture["hidden"]), head=_bits(fixture["head"]), targets=fixture["targets"],
        weights=fixture["weights"], nll_sum=np.float32(nll), weight_sum=np.float32(weight_sum),
        lse=lse.numpy(), dhidden=_bits(dhidden), dhead=_bits(dhead),
    )
    print("wrote", sorted(p.name for p in GOLDEN_DIR.glob("*.npz")))


if __name__ == "__main__":
    main()
