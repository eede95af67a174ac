"""Installs the batch-invariant operators.

Counterpart of the reference's src/patch/patch_batch_invariant.py:9-28: turn on the aten overrides,
route RMSNorm to the fixed-order implementation, and pin the engine settings the reference pins.
The reference sends RMSNorm through the unfused PyTorch formula so that its `.mean` hits the
batch-invariant kernel; here the same arithmetic runs in one fused kernel.
"""
import os

import torch

from .. import layers
from ..bio.batch_invariant_ops import enable_batch_invariant_mode, rms_norm


def patch_rms_norm():
    layers.RMSNorm.forward = layers.RMSNorm.forward_fused
    try:
        from vllm.model_executor.layers.layernorm import RMSNorm as VllmRMSNorm
    except ImportError:
        return

    def _forward_cuda(self, x, residual=None):
        # what the fused kernel does not take goes where the reference sends everything: the unfused formula, whose
        # mean runs through the batch-invariant override (src/patch/patch_batch_invariant.py:9-16)
        hidden = x.shape[-1]
        if (x.dtype not in (torch.bfloat16, torch.float16) or hidden > 8192 or hidden % 8 != 0
                or getattr(self, "variance_size_override", None) is not None):
            return self.forward_native(x, residual)
        weight = self.weight if getattr(self, "has_weight", True) else None
        return rms_norm(x, weight, self.variance_epsilon, residual)

    VllmRMSNorm.forward_cuda = _forward_cuda
    VllmRMSNorm.forward_hip = _forward_cuda


def patch_batch_invariant():
    enable_batch_invariant_mode()
    os.environ["VLLM_USE_V1"] = "1"
    patch_rms_norm()
    os.environ["VLLM_ATTENTION_BACKEND"] = "TRITON_ATTN"
    print("Successfully patched to use the batch_invariant implementation")
