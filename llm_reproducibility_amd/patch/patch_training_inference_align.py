"""Train/inference alignment switches.

The reference's src/patch/patch_training_inference_align.py replaces vLLM-internal paged-attention
kernels; those live outside the row-split GEMM / reduction path this package accelerates.  What is
kept here is the part of that patch that touches this package's own code: rotary inverse frequencies
are computed on the CPU in fp32 (reference :35-44) so every process derives identical tables.
"""
import torch

_align_enabled = False


def compute_inv_freq(rotary_dim: int, base: float, device=None) -> torch.Tensor:
    arange = torch.arange(0, rotary_dim, 2, dtype=torch.float, device="cpu")
    inv_freq = 1.0 / (base ** (arange / rotary_dim))
    return inv_freq if device is None else inv_freq.to(device)


def align_is_enabled() -> bool:
    return _align_enabled


def patch_training_inference_align():
    global _align_enabled
    _align_enabled = True
    print("Train/inference alignment: rotary tables computed on the CPU; attention kernels are not patched by this package")


def patch_training_baseline():
    global _align_enabled
    _align_enabled = False
