"""Host-side mirror of the reference's Cut cross-entropy operator for MI355X.

``pallas_cut_linear_cross_entropy`` keeps the reference's name, argument
meaning, validation errors and custom-VJP contract
(src/causal_trainer/kernels/cut_cross_entropy.py:828-958, :524-670): it
returns ``(nll_sum, weight_sum)`` as f32 scalars, saves
``(hidden, head, targets, weights, lse)``, gives no cotangent to
targets / weights, ignores the cotangent of ``weight_sum``, and with
``lm_head_trainable=False`` never launches the dHead kernel and returns no
head gradient. Tensors are torch tensors on a ROCm device; the work is done by
libct_hotpath.so through its C ABI.

``loss = nll_sum / max(weight_sum, 1)`` stays with the caller
(src/causal_trainer/training/losses.py:234-237).

One deliberate difference in the residual. The reference keeps no logits because
a TPU core has little memory, and pays for it by recomputing the projection in
each backward kernel. A MI355X has 288 GB: when the f32 logits of the active
rows fit in ``LOGITS_CACHE_LIMIT_BYTES`` the forward also leaves them in a cache
that lives until the backward of the loss (the adjacent step of a training
iteration), and the backward then runs 3 GEMMs instead of 4. Above the limit, or
with ``logits_cache=False``, nothing but ``lse`` is kept and logits are recomputed.

``local_chunk_size`` (:697-825). The reference's chunk loop bounds what one TPU core holds at
a time: it walks the rows in chunks, compacts inside the chunk and accumulates the head
gradient in f32 across chunks. What the option buys is a bound on transient memory, and that
is what it selects here: with ``local_chunk_size = C > 0`` the backward's dlogits slab is no
larger than the dlogits of C rows over the whole vocabulary would be (``backward_workspace_bytes``;
never below the kernels' minimum of one 256-wide vocabulary tile), the vocabulary is walked in
slabs of that size with dHidden accumulated in f32 across slabs and rounded once, and no logits
cache is kept. A row's statistics and gradients do not depend on which slab or slot it sits in;
only the order of f32 additions differs, inside the operator's tolerances. ``0`` (the default)
keeps the single full-vocabulary slab.
"""

from __future__ import annotations


import torch

from . import _lib
from .efficient_attention import _Axes, _integer

_HIDDEN_ALIGN = 128
# Largest logits cache the operator allocates by itself (f32 [vocab, rows], both padded to 256).
LOGITS_CACHE_LIMIT_BYTES = 24 << 30


def _shape_struct(rows: int, hidden: int, vocab: int) -> _lib.CutceShape:
    return _lib.CutceShape(rows=rows, hidden=hidden, vocab=vocab)


def logits_cache_bytes(rows: int, hidden: int, vocab: int) -> int:
    """Size of the optional f32 logits cache for this problem."""

    return int(_lib.load().ct_cutce_logits_cache_bytes(_shape_struct(rows, hidden, vocab)))


def backward_workspace_bytes(rows: int, hidden: int, vocab: int, local_chunk_size: int = 0) -> int:
    """Workspace of the backward: the full-vocabulary slab, or with ``local_chunk_size`` rows per
    chunk a slab as large as the dlogits of one chunk of rows (at least the kernels' minimum)."""

    lib = _lib.load()
    shape = _shape_struct(rows, hidden, vocab)
    full, least = int(lib.ct_cutce_bwd_workspace_bytes(shape)), int(lib.ct_cutce_bwd_workspace_min_bytes(shape))
    if local_chunk_size <= 0 or local_chunk_size >= rows:
        return full
    return max(least, min(full, least + (full - least) * local_chunk_size // rows))


def cutce_forward(hidden, head, targets, weights, *, sparse_compaction: bool = False,
                  logits_cache=None):
    """Flat forward: hidden [N, d], head [d, V] -> (nll_sum, weight_sum, lse [N]).

    ``logits_cache``: optional uint8 device tensor of ``logits_cache_bytes(...)`` bytes that
    the forward fills for ``cutce_backward``.
    """

    lib = _lib.load()
    rows, width = hidden.shape
    shape = _shape_struct(rows, width, head.shape[1])
    device = hidden.device
    workspace = torch.empty(lib.ct_cutce_fwd_workspace_bytes(shape), dtype=torch.uint8, device=device)
    scalars = torch.empty(2, dtype=torch.float32, device=device)
    lse = torch.empty(rows, dtype=torch.float32, device=device)
    args = _lib.CutceFwdArgs(
        hidden=hidden.data_ptr(), head=head.data_ptr(), targets=targets.data_ptr(),
        weights=weights.data_ptr(), nll_sum=scalars[0:].data_ptr(),
        weight_sum=scalars[1:].data_ptr(), lse=lse.data_ptr(),
        workspace=workspace.data_ptr(), workspace_bytes=workspace.numel(),
        shape=shape, sparse_compaction=int(bool(sparse_compaction)),
        logits_cache=_lib.pointer(logits_cache),
        logits_cache_bytes=0 if logits_cache is None else logits_cache.numel(),
    )
    with torch.cuda.device(device):
        _lib.check(lib.ct_cutce_fwd(_lib.current_stream(), args))
    return scalars[0], scalars[1], lse


def cutce_backward(hidden, head, targets, weights, lse, dy, *, sparse_compaction: bool = False,
                   lm_head_trainable: bool = True, workspace_bytes: int | None = None,
                   logits_cache=None):
    """Flat backward: returns (dhidden [N, d], dhead [d, V] or None).

    ``logits_cache``: the tensor a forward with the same ``sparse_compaction`` filled, or None
    to recompute the logits.
    """

    lib = _lib.load()
    rows, width = hidden.shape
    shape = _shape_struct(rows, width, head.shape[1])
    device = hidden.device
    if workspace_bytes is None:
        workspace_bytes = lib.ct_cutce_bwd_workspace_bytes(shape)
    workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=device)
    dhidden = torch.empty_like(hidden)
    dhead = torch.empty_like(head) if lm_head_trainable else None
    dy = dy.to(device=device, dtype=torch.float32).reshape(1).contiguous()
    args = _lib.CutceBwdArgs(
        hidden=hidden.data_ptr(), head=head.data_ptr(), targets=targets.data_ptr(),
        weights=weights.data_ptr(), lse=lse.data_ptr(), dy=dy.data_ptr(),
        dhidden=dhidden.data_ptr(), dhead=_lib.pointer(dhead),
        workspace=workspace.data_ptr(), workspace_bytes=workspace.numel(),
        shape=shape, sparse_compaction=int(bool(sparse_compaction)),
        logits_cache=_lib.pointer(logits_cache),
        logits_cache_bytes=0 if logits_cache is None else logits_cache.numel(),
    )
    with torch.cuda.device(device):
        _lib.check(lib.ct_cutce_bwd(_lib.current_stream(), args))
    return dhidden, dhead


class _CutCE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, head, targets, weights, lm_head_trainable, sparse_compaction,
                logits_cache, local_chunk_size):
        cache = None
        ctx.workspace_bytes = backward_workspace_bytes(hidden.shape[0], hidden.shape[1], head.shape[1],
                                                       local_chunk_size)
        if logits_cache and not local_chunk_size and (hidden.requires_grad or head.requires_grad):
            size = logits_cache_bytes(hidden.shape[0], hidden.shape[1], head.shape[1])
            if size <= LOGITS_CACHE_LIMIT_BYTES:
                cache = torch.empty(size, dtype=torch.uint8, device=hidden.device)
        nll_sum, weight_sum, lse = cutce_forward(hidden, head, targets, weights,
                                                 sparse_compaction=sparse_compaction,
                                                 logits_cache=cache)
        # The reference's residual (:587-593) plus, when it fits, the f32 logits cache.
        ctx.save_for_backward(hidden, head, targets, weights, lse)
        ctx.logits_cache = cache
        ctx.lm_head_trainable = lm_head_trainable
        ctx.sparse_compaction = sparse_compaction
        ctx.mark_non_differentiable(weight_sum)
        return nll_sum, weight_sum

    @staticmethod
    def backward(ctx, nll_cotangent, _weight_cotangent):
        hidden, head, targets, weights, lse = ctx.saved_tensors
        dhidden, dhead = cutce_backward(
            hidden, head, targets, weights, lse, nll_cotangent,
            sparse_compaction=ctx.sparse_compaction, lm_head_trainable=ctx.lm_head_trainable,
            logits_cache=ctx.logits_cache, workspace_bytes=ctx.workspace_bytes,
        )
        ctx.logits_cache = None
        return dhidden, dhead, None, None, None, None, None, None


def pallas_cut_linear_cross_entropy(hidden_states, lm_head_kernel, targets, weights, *, mesh=None,
                                    sparse_compaction: bool = False,
                                    lm_head_trainable: bool = True, local_chunk_size: int = 0,
                                    logits_cache: bool = True, head_layout: str = "dv"):
    """Return ``(nll_sum, weight_sum)``; logits are only ever kept in the bounded cache
    described in the module docstring (``logits_cache=False`` disables it).

    hidden_states ``[B, S, d]``, lm_head_kernel ``[d, V]`` (same float dtype, bf16),
    targets int32 ``[B, S]``, weights f32 ``[B, S]``; a row is ignored iff its weight is 0.

    ``head_layout="vd"``: lm_head_kernel is ``[V, d]`` (a checkpoint's ``[out, in]`` layout, which the
    reference transposes once at load, src/causal_trainer/checkpointing/huggingface.py:1-6). The
    kernels read ``[d, V]`` with the vocabulary contiguous, so this layout costs a transposing copy
    of the head per call and one of its gradient in the backward (2 B read + 2 B written per element
    each, about 0.4 ms per GB on this part); its gradient comes back as ``[V, d]``.
    """

    if head_layout not in ("dv", "vd"):
        raise ValueError("head_layout must be 'dv' ([hidden, vocab]) or 'vd' ([vocab, hidden])")
    if head_layout == "vd":
        if lm_head_kernel.ndim != 2:
            raise ValueError("lm_head_kernel must have shape [vocab, hidden]")
        lm_head_kernel = lm_head_kernel.t()   # (made contiguous below; autograd transposes the gradient back)

    local_chunk_size = _integer(local_chunk_size, "local_chunk_size must be a static non-negative integer")
    if local_chunk_size < 0:
        raise ValueError("local_chunk_size must be non-negative")
    layout_ok = hidden_states.ndim == 3
    if not layout_ok:
        raise ValueError("Cut cross-entropy expects hidden_states [batch, sequence, hidden]")
    batch, sequence, hidden = hidden_states.shape
    if tuple(lm_head_kernel.shape[:1]) != (hidden,) or lm_head_kernel.ndim != 2:
        raise ValueError("lm_head_kernel must have shape [hidden, vocab]")
    targets = torch.as_tensor(targets, device=hidden_states.device).to(torch.int32)
    weights = torch.as_tensor(weights, device=hidden_states.device).to(torch.float32)
    for broken, error in (
        (not (targets.shape == weights.shape == (batch, sequence)),
         ValueError("targets and weights must match hidden_states.shape[:-1]")),
        (batch * sequence == 0, ValueError("Cut cross-entropy requires at least one token row")),
        (hidden == 0 or hidden % _HIDDEN_ALIGN != 0,
         ValueError("Cut cross-entropy hidden size must be divisible by 128")),
        (lm_head_kernel.shape[1] == 0, ValueError("Cut cross-entropy requires a non-empty vocabulary")),
        (lm_head_kernel.dtype != hidden_states.dtype,
         TypeError("hidden_states and lm_head_kernel must use the same compute dtype")),
        (not hidden_states.dtype.is_floating_point, TypeError("Cut cross-entropy inputs must have a floating dtype")),
        (hidden_states.dtype != torch.bfloat16,
         TypeError("this build computes Cut cross-entropy in bfloat16 only")),
        (not hidden_states.is_cuda, RuntimeError("Cut cross-entropy is available only on a ROCm GPU")),
    ):
        if broken:
            raise error
    active = _Axes(mesh).beyond_one_device()
    sharded_rows = [axis for axis in ("fsdp", "ep") if axis in active]
    if sharded_rows:
        raise ValueError("Cut cross-entropy currently requires fsdp=ep=1; active unsupported axes: "
                         + ", ".join(sharded_rows))
    if active:
        raise ValueError(f"this build runs on one GPU; mesh axes larger than 1: {active}")
    width = hidden_states.shape[-1]
    return _CutCE.apply(
        hidden_states.reshape(-1, width).contiguous(), lm_head_kernel.contiguous(),
        targets.reshape(-1).contiguous(), weights.reshape(-1).contiguous(),
        bool(lm_head_trainable), bool(sparse_compaction), bool(logits_cache), local_chunk_size,
    )


__all__ = ["LOGITS_CACHE_LIMIT_BYTES", "backward_workspace_bytes", "cutce_backward", "cutce_forward", "logits_cache_bytes",
           "pallas_cut_linear_cross_entropy"]
