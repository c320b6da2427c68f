"""JAX binding of the hot paths through XLA FFI custom calls (needs jax + jaxlib on ROCm).

This is the reference-side glue: it registers the handlers exported by libct_ffi.so
(csrc/ct_ffi.cc) for platform "ROCM" and wraps them in ``jax.custom_vjp`` functions whose
signatures and residuals are those of the reference operators
(src/causal_trainer/kernels/efficient_attention.py:1807-1863,
src/causal_trainer/kernels/cut_cross_entropy.py:524-670), so the call sites at
src/causal_trainer/modeling/attention.py:435-444 and
src/causal_trainer/kernels/fused_cross_entropy.py:189-198 only change their import.

jax is not installed in the build environment of this repository, so this module is not
exercised by the test-suite here; the C ABI underneath it is, through ctypes.
"""

from __future__ import annotations

import ctypes
import functools
from pathlib import Path

_FFI_LIBRARY = Path(__file__).resolve().parent / "libct_ffi.so"
_TARGETS = ("ct_ffi_attn_prepare", "ct_ffi_attn_fwd", "ct_ffi_attn_bwd", "ct_ffi_cutce_fwd", "ct_ffi_cutce_bwd")


@functools.lru_cache(maxsize=1)
def register() -> None:
    import jax

    if not _FFI_LIBRARY.exists():
        raise RuntimeError(f"{_FFI_LIBRARY} is missing: build csrc/ct_ffi.cc against jaxlib's FFI headers")
    library = ctypes.CDLL(str(_FFI_LIBRARY))
    for name in _TARGETS:
        jax.ffi.register_ffi_target(name, jax.ffi.pycapsule(getattr(library, name)), platform="ROCM")


def _workspace_bytes(kind: str, rows: int, hidden: int, vocab: int) -> int:
    from . import _lib

    shape = _lib.CutceShape(rows, hidden, vocab)
    query = {"fwd": "ct_cutce_fwd_workspace_bytes", "bwd": "ct_cutce_bwd_workspace_bytes"}[kind]
    return int(getattr(_lib.load(), query)(ctypes.byref(shape)))


def tile_bounds(segment_ids, attention_end=None):
    """Flat int32 tile table + schedules (ct_attn_meta_bytes); call once per forward, next to
    prepare_attention_metadata, and reuse for every layer."""

    import jax
    import jax.numpy as jnp

    register()
    batch, seq = segment_ids.shape
    has_end = attention_end is not None
    from . import _lib

    words = int(_lib.load().ct_attn_meta_bytes(batch, seq)) // 4
    out = jax.ShapeDtypeStruct((words,), jnp.int32)
    return jax.ffi.ffi_call("ct_ffi_attn_prepare", out)(
        segment_ids, attention_end if has_end else segment_ids, has_end=has_end)


def make_efficient_attention():
    """Returns ``attention(q, k, v, segment_ids, attention_end, bounds, scale)`` with the custom VJP."""

    import jax
    import jax.numpy as jnp

    register()

    def forward(q, k, v, segment_ids, attention_end, bounds, scale):
        has_end = attention_end is not None
        shapes = (jax.ShapeDtypeStruct(q.shape, jnp.bfloat16), jax.ShapeDtypeStruct(q.shape[:3], jnp.float32))
        return jax.ffi.ffi_call("ct_ffi_attn_fwd", shapes)(
            q, k, v, segment_ids, attention_end if has_end else segment_ids, bounds,
            scale=jnp.float32(scale), has_end=has_end)

    @functools.partial(jax.custom_vjp, nondiff_argnums=(6,))
    def attention(q, k, v, segment_ids, attention_end, bounds, scale):
        return forward(q, k, v, segment_ids, attention_end, bounds, scale)[0]

    def attention_fwd(q, k, v, segment_ids, attention_end, bounds, scale):
        out, lse = forward(q, k, v, segment_ids, attention_end, bounds, scale)
        return out, (q, k, v, segment_ids, attention_end, bounds, out, lse)     # residual of the reference

    def attention_bwd(scale, residual, dout):
        q, k, v, segment_ids, attention_end, bounds, out, lse = residual
        has_end = attention_end is not None
        from . import _lib

        scratch = int(_lib.load().ct_attn_bwd_workspace_bytes(q.shape[0], q.shape[1], q.shape[2], k.shape[2], q.shape[3]))
        shapes = (jax.ShapeDtypeStruct(q.shape, q.dtype), jax.ShapeDtypeStruct(k.shape, k.dtype),
                  jax.ShapeDtypeStruct(v.shape, v.dtype), jax.ShapeDtypeStruct(lse.shape, jnp.float32),
                  jax.ShapeDtypeStruct((scratch,), jnp.uint8))
        dq, dk, dv, _, _ = jax.ffi.ffi_call("ct_ffi_attn_bwd", shapes)(
            q, k, v, segment_ids, attention_end if has_end else segment_ids, bounds, out, lse,
            dout.astype(jnp.bfloat16), scale=jnp.float32(scale), has_end=has_end)
        return dq, dk, dv, None, None, None

    attention.defvjp(attention_fwd, attention_bwd)
    return attention


def make_cut_cross_entropy(*, sparse_compaction: bool, lm_head_trainable: bool,
                           logits_cache_limit_bytes: int = 24 << 30):
    """Returns ``cut_ce(hidden[N, d], head[d, V], targets[N], weights[N]) -> (nll_sum, weight_sum)``.

    When the f32 logits cache of the problem fits in ``logits_cache_limit_bytes`` the forward
    under differentiation also returns it as a residual and the backward skips the logit
    recomputation; otherwise the residual is the reference's (no logits).
    """

    import jax
    import jax.numpy as jnp

    register()

    def forward(hidden, head, targets, weights, cache_bytes):
        rows, width = hidden.shape
        scalar = jax.ShapeDtypeStruct((1,), jnp.float32)
        shapes = (scalar, scalar, jax.ShapeDtypeStruct((rows,), jnp.float32),
                  jax.ShapeDtypeStruct((_workspace_bytes("fwd", rows, width, head.shape[1]),), jnp.uint8),
                  jax.ShapeDtypeStruct((max(cache_bytes, 16),), jnp.uint8))   # 16 bytes = "no cache"
        nll, weight_sum, lse, _, cache = jax.ffi.ffi_call("ct_ffi_cutce_fwd", shapes)(
            hidden, head, targets, weights, sparse_compaction=sparse_compaction)
        return nll[0], weight_sum[0], lse, cache

    def cache_bytes_for(hidden, head):
        from . import _lib

        shape = _lib.CutceShape(rows=hidden.shape[0], hidden=hidden.shape[1], vocab=head.shape[1])
        size = int(_lib.load().ct_cutce_logits_cache_bytes(shape))
        return size if size <= logits_cache_limit_bytes else 0

    @jax.custom_vjp
    def cut_ce(hidden, head, targets, weights):
        nll, weight_sum, _, _ = forward(hidden, head, targets, weights, 0)
        return nll, weight_sum

    def cut_ce_fwd(hidden, head, targets, weights):
        nll, weight_sum, lse, cache = forward(hidden, head, targets, weights, cache_bytes_for(hidden, head))
        return (nll, weight_sum), (hidden, head, targets, weights, lse, cache)

    def cut_ce_bwd(residual, cotangents):
        hidden, head, targets, weights, lse, cache = residual
        nll_cotangent, _ = cotangents
        rows, width = hidden.shape
        shapes = (jax.ShapeDtypeStruct(hidden.shape, hidden.dtype), jax.ShapeDtypeStruct(head.shape, head.dtype),
                  jax.ShapeDtypeStruct((_workspace_bytes("bwd", rows, width, head.shape[1]),), jnp.uint8))
        dhidden, dhead, _ = jax.ffi.ffi_call("ct_ffi_cutce_bwd", shapes)(
            hidden, head, targets, weights, lse, jnp.reshape(nll_cotangent.astype(jnp.float32), (1,)),
            cache, sparse_compaction=sparse_compaction, head_trainable=lm_head_trainable)
        return dhidden, (dhead if lm_head_trainable else None), None, None

    cut_ce.defvjp(cut_ce_fwd, cut_ce_bwd)
    return cut_ce
