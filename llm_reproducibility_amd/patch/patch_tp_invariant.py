"""Installs the TP-invariant forward on row-split linear layers.

Counterpart of the reference's src/patch/patch_tp_invariant.py:10-52.  The package's own
`RowParallelLinear` is always patched; vLLM's class is patched too when vLLM is importable.
"""
from .. import layers

_original_forward = None


def patch_row_linear():
    global _original_forward
    if _original_forward is None:
        _original_forward = layers.RowParallelLinear.forward
    layers.RowParallelLinear.forward = layers.tbik_row_parallel_forward
    try:
        from vllm.model_executor.layers.linear import RowParallelLinear as VllmRowParallelLinear
    except ImportError:
        return
    VllmRowParallelLinear.forward = layers.tbik_row_parallel_forward


def unpatch_row_linear():
    """Restores the stock forward of the package's own layer (used by tests)."""
    global _original_forward
    if _original_forward is not None:
        layers.RowParallelLinear.forward = _original_forward
        _original_forward = None


def patch_tp_invariant():
    patch_row_linear()
    print("Successfully patched row-parallel linear layers to use the tp_invariant implementation")
