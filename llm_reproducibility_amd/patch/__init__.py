"""Plugin boundary: `apply_patches()` reads the environment flags and installs the invariant kernels.

Same dispatch as the reference's src/patch/__init__.py:7-37.  Call it before the engine builds its
layers and in every worker process.
"""
from .patch_batch_invariant import patch_batch_invariant
from .patch_tp_invariant import patch_tp_invariant
from .patch_training_inference_align import patch_training_inference_align as patch_align, patch_training_baseline

__all__ = ["apply_patches"]


def apply_patches():
    from ..utils import batch_invariant_is_enabled, tp_invariant_is_enabled, compatible_mode_is_enabled
    bi, tp, align = batch_invariant_is_enabled(), tp_invariant_is_enabled(), compatible_mode_is_enabled()
    if not bi and not tp and not align:
        patch_training_baseline()
        print("No invariance patches applied. Only the baseline settings are in effect\n")
        return
    if bi:
        patch_batch_invariant()
    if tp:
        patch_tp_invariant()
    if align:
        if bi:
            patch_align()
        else:
            patch_training_baseline()
    print("Successfully applied patches\n")
    return
