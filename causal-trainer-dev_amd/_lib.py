"""ctypes binding of libct_hotpath.so (the C ABI declared in include/ct_hotpath.h).

The library is the only compute path: if it is missing or a symbol is absent
this module raises, it never falls back to another implementation.
"""

from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_float, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
LIBRARY_PATH = PACKAGE_DIR / "libct_hotpath.so"

CT_OK = 0
CT_INVALID_ARGUMENT = -1
CT_UNSUPPORTED = -2
CT_WORKSPACE_TOO_SMALL = -3
CT_LAUNCH_FAILED = -4

ATTN_META_WIDTH = 12
ABI_VERSION = 3

# ct_attn_bwd_args.variant (0 = every choice left to the library)
ATTN_BWD_DKV_NARROW = 1
ATTN_BWD_DKV_WIDE = 2
ATTN_BWD_DQ_RECOMPUTE = 0x10
ATTN_BWD_DQ_FROM_DS = 0x20
ATTN_BWD_WORK_LIST_KEPT = 0x100


class CtError(RuntimeError):
    """A C ABI call returned a negative status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"[ct_status {status}] {message}")
        self.status = status
        self.message = message


class AttnFwdArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p),
        ("segment_ids", c_void_p), ("attention_end", c_void_p), ("tile_meta", c_void_p),
        ("out", c_void_p), ("lse", c_void_p),
        ("batch", c_int32), ("seq", c_int32), ("q_heads", c_int32), ("kv_heads", c_int32),
        ("head_dim", c_int32), ("scale", c_float),
    ]


class AttnBwdArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p),
        ("segment_ids", c_void_p), ("attention_end", c_void_p), ("tile_meta", c_void_p),
        ("out", c_void_p), ("lse", c_void_p), ("dout", c_void_p),
        ("dq", c_void_p), ("dk", c_void_p), ("dv", c_void_p), ("delta", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("batch", c_int32), ("seq", c_int32), ("q_heads", c_int32), ("kv_heads", c_int32),
        ("head_dim", c_int32), ("scale", c_float), ("variant", c_int32),
    ]


class CutceShape(Structure):
    _fields_ = [("rows", c_int32), ("hidden", c_int32), ("vocab", c_int32)]


class CutceFwdArgs(Structure):
    _fields_ = [
        ("hidden", c_void_p), ("head", c_void_p), ("targets", c_void_p), ("weights", c_void_p),
        ("nll_sum", c_void_p), ("weight_sum", c_void_p), ("lse", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("shape", CutceShape), ("sparse_compaction", c_int32),
        ("logits_cache", c_void_p), ("logits_cache_bytes", c_size_t),
    ]


class CutceBwdArgs(Structure):
    _fields_ = [
        ("hidden", c_void_p), ("head", c_void_p), ("targets", c_void_p), ("weights", c_void_p),
        ("lse", c_void_p), ("dy", c_void_p), ("dhidden", c_void_p), ("dhead", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("shape", CutceShape), ("sparse_compaction", c_int32),
        ("logits_cache", c_void_p), ("logits_cache_bytes", c_size_t),
    ]


class ShiftedTargetsArgs(Structure):
    _fields_ = [
        ("input_ids", c_void_p), ("attention_mask", c_void_p), ("segment_ids", c_void_p),
        ("assistant_mask", c_void_p), ("loss_mask", c_void_p), ("labels", c_void_p),
        ("targets", c_void_p), ("weights", c_void_p),
        ("scratch", c_void_p), ("scratch_bytes", c_size_t),
        ("batch", c_int32), ("seq", c_int32), ("ignore_index", c_int32),
    ]


class RotaryArgs(Structure):
    _fields_ = [
        ("q_in", c_void_p), ("k_in", c_void_p), ("q_out", c_void_p), ("k_out", c_void_p),
        ("cosine", c_void_p), ("sine", c_void_p), ("tokens", c_int64),
        ("q_heads", c_int32), ("kv_heads", c_int32), ("head_dim", c_int32),
        ("rotary_pairs", c_int32), ("rope_style", c_int32), ("inverse", c_int32),
        ("q_scale", ctypes.c_float),
    ]


class SparseCeArgs(Structure):
    _fields_ = [
        ("logits", c_void_p), ("targets", c_void_p), ("weights", c_void_p), ("rows", c_int64),
        ("vocab", c_int32), ("logits_dtype", c_int32), ("ignore_index", c_int32),
    ]


LAUNCH_HOOK = ctypes.CFUNCTYPE(None, c_void_p, ctypes.c_char_p, c_int32, c_void_p)

# name -> (restype, argtypes); every symbol include/ct_hotpath.h declares.
SYMBOLS = {
    "ct_set_launch_hook": (None, [LAUNCH_HOOK, c_void_p]),
    "ct_last_error": (ctypes.c_char_p, []),
    "ct_abi_version": (c_int32, []),
    "ct_calibration_copy": (c_int32, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "ct_canonicalize_segment_ids": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
    "ct_shifted_targets_scratch_bytes": (c_size_t, [c_int32, c_int32]),
    "ct_shifted_targets_and_weights": (c_int32, [c_void_p, POINTER(ShiftedTargetsArgs)]),
    "ct_position_ids": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
    "ct_rotary_cos_sin": (c_int32, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_void_p]),
    "ct_apply_rotary": (c_int32, [c_void_p, POINTER(RotaryArgs)]),
    "ct_rms_norm_fwd": (c_int32, [c_void_p, c_void_p, c_void_p, ctypes.c_float, c_int64, c_int32,
                                  c_void_p, c_void_p]),
    "ct_rms_norm_bwd_workspace_bytes": (c_size_t, [c_int32]),
    "ct_rms_norm_bwd": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, ctypes.c_float, c_int64,
                                  c_int32, c_void_p, c_void_p, c_void_p, c_size_t]),
    "ct_sparse_ce_fwd": (c_int32, [c_void_p, POINTER(SparseCeArgs), c_void_p, c_void_p]),
    "ct_sparse_ce_bwd": (c_int32, [c_void_p, POINTER(SparseCeArgs), c_void_p, c_void_p, c_void_p]),
    "ct_attn_meta_bytes": (c_size_t, [c_int32, c_int32]),
    "ct_attn_bwd_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32, c_int32]),
    "ct_attn_bwd_workspace_bytes_from_ds": (c_size_t, [c_int32, c_int32, c_int32, c_int32, c_int32, c_int32]),
    "ct_attn_prepare": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
    "ct_attn_block_summary": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32,
                                        c_void_p]),
    "ct_attn_fwd": (c_int32, [c_void_p, POINTER(AttnFwdArgs)]),
    "ct_attn_bwd": (c_int32, [c_void_p, POINTER(AttnBwdArgs)]),
    "ct_attn_delta": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32]),
    "ct_cutce_fwd_workspace_bytes": (c_size_t, [POINTER(CutceShape)]),
    "ct_cutce_bwd_workspace_min_bytes": (c_size_t, [POINTER(CutceShape)]),
    "ct_cutce_bwd_workspace_bytes": (c_size_t, [POINTER(CutceShape)]),
    "ct_cutce_logits_cache_bytes": (c_size_t, [POINTER(CutceShape)]),
    "ct_cutce_fwd": (c_int32, [c_void_p, POINTER(CutceFwdArgs)]),
    "ct_cutce_bwd": (c_int32, [c_void_p, POINTER(CutceBwdArgs)]),
    "ct_cutce_fwd_noalloc_max_bytes": (c_size_t, []),
    "ct_cutce_fwd_noalloc": (c_int32, [c_void_p, POINTER(CutceFwdArgs)]),
}

_library = None


def load() -> ctypes.CDLL:
    """Load libct_hotpath.so and bind every declared symbol (raises if any is missing)."""

    global _library
    if _library is not None:
        return _library
    if not LIBRARY_PATH.exists():
        raise RuntimeError(
            f"{LIBRARY_PATH} is missing: build it with `python {PACKAGE_DIR / 'build.py'}` "
            "(needs hipcc). There is no fallback implementation."
        )
    library = ctypes.CDLL(str(LIBRARY_PATH))
    for name, (restype, argtypes) in SYMBOLS.items():
        try:
            function = getattr(library, name)
        except AttributeError as error:
            raise RuntimeError(f"{LIBRARY_PATH} does not export {name}") from error
        function.restype = restype
        function.argtypes = argtypes
    version = library.ct_abi_version()
    if version != ABI_VERSION:
        raise RuntimeError(f"libct_hotpath ABI {version} does not match binding ABI {ABI_VERSION}")
    _library = library
    return library


def check(status: int) -> None:
    """Raise CtError for a negative status."""

    if status != CT_OK:
        message = load().ct_last_error().decode("utf-8", "replace")
        raise CtError(status, message)


def pointer(tensor) -> int | None:
    """Device address of a tensor (None passes NULL)."""

    return None if tensor is None else tensor.data_ptr()


def current_stream() -> int:
    """The hipStream_t of torch's current stream, as an integer."""

    import torch

    return torch.cuda.current_stream().cuda_stream
