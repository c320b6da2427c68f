"""ct_cutce_fwd_noalloc (the forward whose workspace is a static device array) against
ct_cutce_fwd, through the C ABI: same kernels, so the results must be bitwise equal. Two calls
in a row, the second on a smaller input, so that what the first call left in the shared array
(a longer index list, more statistics) would show if the second call read any of it."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(seed, rows, width, vocab, device):
    rng = np.random.default_rng(seed)
    hidden = torch.from_numpy(rng.normal(size=(rows, width)).astype(np.float32)).to(torch.bfloat16)
    head = torch.from_numpy(rng.normal(scale=0.05, size=(width, vocab)).astype(np.float32)).to(torch.bfloat16)
    targets = rng.integers(vocab, size=rows).astype(np.int32)
    weights = rng.choice(np.asarray([0.0, 0.25, 1.0, 2.0], np.float32), size=rows).astype(np.float32)
    targets[weights == 0] = -100
    return (hidden.to(device), head.to(device), torch.from_numpy(targets).to(device),
            torch.from_numpy(weights).to(device))


def _forward(ct, entry, hidden, head, targets, weights, *, with_workspace):
    lib = ct._lib.load()
    rows, width = hidden.shape
    shape = ct._lib.CutceShape(rows=rows, hidden=width, vocab=head.shape[1])
    scalars = torch.full((2,), float("nan"), dtype=torch.float32, device=hidden.device)
    lse = torch.full((rows,), float("nan"), dtype=torch.float32, device=hidden.device)
    workspace = None
    if with_workspace:
        workspace = torch.empty(lib.ct_cutce_fwd_workspace_bytes(shape), dtype=torch.uint8, device=hidden.device)
    args = ct._lib.CutceFwdArgs(
        hidden=hidden.data_ptr(), head=head.data_ptr(), targets=targets.data_ptr(), weights=weights.data_ptr(),
        nll_sum=scalars[0:].data_ptr(), weight_sum=scalars[1:].data_ptr(), lse=lse.data_ptr(),
        workspace=ct._lib.pointer(workspace), workspace_bytes=0 if workspace is None else workspace.numel(),
        shape=shape, sparse_compaction=1, logits_cache=None, logits_cache_bytes=0)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    ct._lib.check(getattr(lib, entry)(ct._lib.current_stream(), args))
    torch.cuda.synchronize()
    allocated = free_before - torch.cuda.mem_get_info()[0]
    return scalars.cpu(), lse.cpu(), allocated


def test_noalloc_forward_matches_the_workspace_forward_on_two_calls_in_a_row(ct, gpu):
    lib = ct._lib.load()
    assert lib.ct_cutce_fwd_noalloc_max_bytes() == 32 << 20
    for seed, rows, width, vocab in ((5, 1500, 256, 3001), (6, 300, 128, 258)):
        print("noalloc case", seed, rows, width, vocab, flush=True)
        inputs = _inputs(seed, rows, width, vocab, gpu)
        want_scalars, want_lse, _ = _forward(ct, "ct_cutce_fwd", *inputs, with_workspace=True)
        got_scalars, got_lse, allocated = _forward(ct, "ct_cutce_fwd_noalloc", *inputs, with_workspace=False)
        assert allocated == 0      # device memory in use did not change across the call
        assert torch.equal(got_scalars, want_scalars) and torch.equal(got_lse, want_lse)
        assert torch.isfinite(got_scalars).all() and torch.isfinite(got_lse).all()
        assert (got_lse[inputs[3].cpu() == 0] == 0).all() and float(got_scalars[1]) == float(inputs[3].sum())


def test_noalloc_forward_rejects_shapes_beyond_its_array(ct, gpu):
    lib = ct._lib.load()
    shape = ct._lib.CutceShape(rows=65536, hidden=128, vocab=128256)
    assert lib.ct_cutce_fwd_workspace_bytes(shape) > lib.ct_cutce_fwd_noalloc_max_bytes()
    one = torch.zeros(16, dtype=torch.float32, device=gpu)
    args = ct._lib.CutceFwdArgs(
        hidden=one.data_ptr(), head=one.data_ptr(), targets=one.data_ptr(), weights=one.data_ptr(),
        nll_sum=one.data_ptr(), weight_sum=one.data_ptr(), lse=one.data_ptr(), workspace=None,
        workspace_bytes=0, shape=shape, sparse_compaction=0, logits_cache=None, logits_cache_bytes=0)
    with pytest.raises(ct._lib.CtError, match="static array holds"):
        ct._lib.check(lib.ct_cutce_fwd_noalloc(ct._lib.current_stream(), args))
