"""MI355X-native hot paths of Causal Trainer: segment-isolated attention and cut cross-entropy.

The directory name contains a hyphen, so the repository root carries the
symlink ``causal_trainer_dev_amd`` to it; import the package under that name.
"""

from . import _lib, workloads  # noqa: F401
from .efficient_attention import (  # noqa: F401
    AttentionKernelProfile,
    AttentionMetadata,
    BackwardWorkspace,
    attention_backward,
    attention_forward_with_lse,
    default_attention_scale,
    efficient_attention,
    prepare_attention_metadata,
    resolve_attention_profile,
    tile_bounds_table,
    validate_attention_profile,
)
from .cut_cross_entropy import (  # noqa: F401,E402
    cutce_backward,
    cutce_forward,
    pallas_cut_linear_cross_entropy,
)
from . import cut_cross_entropy, layer_ops, prep, profiling, sparse_cross_entropy  # noqa: F401,E402
from .sparse_cross_entropy import pallas_fused_sparse_cross_entropy  # noqa: F401,E402
from .prep import canonicalize_segment_ids, shifted_targets_and_weights  # noqa: F401,E402
from .layer_ops import (  # noqa: F401,E402
    apply_rotary_cos_sin, apply_rotary_embedding, make_position_ids, rms_norm, rotary_cos_sin,
)
from . import maskgit, packing  # noqa: F401,E402
from .maskgit import MaskGITBatchTransform  # noqa: F401,E402
from .packing import best_fit_decreasing, collate, pack_examples, pad_example, pad_examples  # noqa: F401,E402
