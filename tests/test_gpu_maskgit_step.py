"""One MaskGIT step end to end on the GPU: packed ChatML records -> MaskGITBatchTransform ->
segment-isolated attention with ``attention_end`` and cut cross-entropy on the aligned targets,
each against its oracle on the same arrays (the step of the reference's
tests/training/test_maskgit.py:239-290, without the model around the two operators).
"""

import numpy as np
import pytest
import torch

from oracle import attention_ref, cutce_ref
from tests.golden.chatml_tokenizer import ByteChatTokenizer, image_grid, record

pytestmark = pytest.mark.gpu


def _bf16(array):
    return torch.from_numpy(np.asarray(array, dtype=np.float32)).to(torch.bfloat16)


def test_packed_maskgit_batch_through_both_operators(ct, gpu):
    tokenizer = ByteChatTokenizer()
    records = [record(tokenizer, image_grid(8, 4)), record(tokenizer, "plain answer"),
               record(tokenizer, image_grid() + "\n\nnext:\n" + image_grid(2, 2, first=8)),
               record(tokenizer, image_grid(4, 3, first=2)), record(tokenizer, "text " * 20)]
    rows = ct.pack_examples(records, max_length=256, pad_token_id=tokenizer.pad_token_id)
    batch = ct.collate(rows, assistant_only_loss=True)
    mixed = ct.MaskGITBatchTransform(tokenizer, probability=1.0, seed=5)(batch, step=3)
    ids, ends = mixed["segment_ids"], mixed["attention_end"]
    assert (ends != np.arange(ids.shape[1])[None]).any()  # some block is bidirectional

    # attention: forward and backward with the transform's attention_end
    rng = np.random.default_rng(12)
    B, S, Hq, Hkv, D = ids.shape[0], ids.shape[1], 4, 2, 128
    q, k, v, dout = (_bf16(rng.standard_normal(shape) * 0.5) for shape in
                     ((B, S, Hq, D), (B, S, Hkv, D), (B, S, Hkv, D), (B, S, Hq, D)))
    scale = float(ct.default_attention_scale(D))
    profile = ct.resolve_attention_profile(q.shape, k.shape, None, has_attention_end=True)
    canonical = ct.canonicalize_segment_ids(torch.from_numpy(mixed["attention_mask"]).to(gpu),
                                            torch.from_numpy(ids).to(gpu))
    assert np.array_equal(canonical.cpu().numpy(), ids)  # packing already emits canonical ids
    metadata = ct.prepare_attention_metadata(canonical, mesh=None, profile=profile,
                                             attention_end=torch.from_numpy(ends).to(gpu))
    qd, kd, vd, dod = (t.to(gpu) for t in (q, k, v, dout))
    out, lse = ct.attention_forward_with_lse(qd, kd, vd, metadata, scale=scale)
    dq, dk, dv = ct.attention_backward(qd, kd, vd, metadata, out, lse, dod, scale=scale)
    allowed = attention_ref.allowed_mask(mixed["attention_mask"], ids, ends)
    assert np.array_equal(allowed, attention_ref.allowed_from_canonical(ids, ends))
    out_ref, dq_ref, dk_ref, dv_ref = attention_ref.vanilla_attention_vjp(q, k, v, allowed, dout, scale=scale)
    assert float((out.cpu().float() - out_ref.float()).abs().max()) <= 2e-2
    assert float((lse.cpu() - attention_ref.efficient_lse(q, k, allowed, scale=scale)).abs().max()) <= 1e-3
    for got, want in ((dq, dq_ref), (dk, dk_ref), (dv, dv_ref)):
        assert attention_ref.relative_l2(got.cpu(), want) <= 2e-2
    pad = torch.from_numpy(ids == 0)
    assert (out.cpu()[pad] == 0).all() and (dq.cpu()[pad] == 0).all()

    # loss: the aligned targets / weights go to the cut cross-entropy operator as they are
    d, V = 128, len(tokenizer)
    hidden = _bf16(rng.standard_normal((B, S, d)) * 0.06)
    head = _bf16(rng.standard_normal((d, V)) * 0.05)
    targets, weights = mixed["prediction_targets"], mixed["prediction_weights"]
    assert (weights[mixed["input_ids"] == tokenizer.get_vocab()["[MASK]"]] > 0).all()
    hd = hidden.to(gpu).requires_grad_(True)
    wd = head.to(gpu).requires_grad_(True)
    nll, weight_sum = ct.pallas_cut_linear_cross_entropy(hd, wd, torch.from_numpy(targets).to(gpu),
                                                         torch.from_numpy(weights).to(gpu), mesh=None,
                                                         sparse_compaction=True)
    dy = 1.0 / max(float(weights.sum()), 1.0)
    (nll * dy).backward()
    flat_t, flat_w = torch.from_numpy(targets.reshape(-1)), torch.from_numpy(weights.reshape(-1))
    nll_ref, weight_ref, lse_ref = cutce_ref.cut_forward(hidden.reshape(-1, d), head, flat_t, flat_w)
    dh_ref, dw_ref = cutce_ref.cut_backward(hidden.reshape(-1, d), head, flat_t, flat_w, lse_ref, dy)
    assert float(nll) == pytest.approx(float(nll_ref), rel=1e-4)
    assert float(weight_sum) == float(weight_ref) == float(weights.sum())
    assert attention_ref.relative_l2(hd.grad.cpu().reshape(-1, d), dh_ref) <= 2e-2
    assert attention_ref.relative_l2(wd.grad.cpu(), dw_ref) <= 2e-2
    assert (hd.grad.cpu().reshape(-1, d)[flat_w == 0] == 0).all()
