"""MI355X-native tree-based invariant kernels (TBIK) behind the reference's plugin API.

    from llm_reproducibility_amd import apply_patches
    apply_patches()          # reads VLLM_BATCH_INVARIANT / VLLM_TP_INVARIANT / ALIGN_TRAIN_INFERENCE

    from llm_reproducibility_amd.tbik.tree_based_matmul import matmul_tp_persistent
    from llm_reproducibility_amd.tbik.tree_based_all_reduce import tree_all_reduce_sum, tree_combine
    from llm_reproducibility_amd.bio.batch_invariant_ops import enable_batch_invariant_mode

All compute runs in hand-written HIP kernels for gfx950 loaded from libtbik_hip.so.
"""
__version__ = "0.1.0"

from . import utils  # noqa: F401
from .patch import apply_patches  # noqa: F401

__all__ = ["apply_patches", "utils"]
