"""Environment flags of the plugin boundary.

Same names and meaning as the reference's src/utils.py:4-60: every flag is an integer, anything that
does not parse counts as off, and VLLM_TP_INVARIANT requires VLLM_BATCH_INVARIANT.
TP_INVARIANT_MATMUL is the switch of the reference's smoke script (simple_matmul.py:8).
"""
import os


def _flag(name: str) -> bool:
    try:
        return int(os.getenv(name, "0")) != 0
    except ValueError:
        return False


def batch_invariant_is_enabled() -> bool:
    return _flag("VLLM_BATCH_INVARIANT")


def tp_invariant_is_enabled() -> bool:
    on = _flag("VLLM_TP_INVARIANT")
    if on:
        assert batch_invariant_is_enabled(), "Batch invariance must be enabled when TP invariance is enabled"
    return on


def check_invariant_compat() -> bool:
    return _flag("VLLM_BATCH_INVARIANT") and _flag("VLLM_TP_INVARIANT")


def compatible_mode_is_enabled() -> bool:
    return _flag("ALIGN_TRAIN_INFERENCE")


def tp_invariant_matmul_is_enabled() -> bool:
    return _flag("TP_INVARIANT_MATMUL")
