"""MI355X (gfx950) paged GQA decode attention behind the TileOPs operator contract.

Public surface: the four ops, the backend seam, the manifest loader.  The HIP library is opened lazily on
the first kernel build; importing this package touches no device.
"""

from .backend import (  # noqa: F401
    BUILTIN, AmbiguousTargetError, BackendError, OpNotAvailableError, TensorSpec, UnknownTargetError,
    default_target, load_failures, register_detector, register_kernel_builder, registered_targets, set_default_target,
)
from .ops import (  # noqa: F401
    GroupedQueryAttentionDecodeWithKVCacheFwdOp,
    GroupedQueryAttentionDecodePagedWithKVCacheFwdOp,
    GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp,
    GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp,
)

__all__ = [
    "GroupedQueryAttentionDecodeWithKVCacheFwdOp",
    "GroupedQueryAttentionDecodePagedWithKVCacheFwdOp",
    "GroupedQueryAttentionMultiTokenDecodePagedWithKVCacheFwdOp",
    "GroupedQueryAttentionPrefillPagedWithKVCacheFwdOp",
]
__version__ = "0.1.0"
