"""Batch-invariant ops (mm/addmm, log_softmax/softmax, mean, RMSNorm) on gfx950."""
from .batch_invariant_ops import (  # noqa: F401
    set_batch_invariant_mode, is_batch_invariant_mode_enabled, disable_batch_invariant_mode,
    enable_batch_invariant_mode, matmul_persistent, log_softmax, mean_dim, rms_norm,
    get_batch_invariant_attention_block_size,
)
