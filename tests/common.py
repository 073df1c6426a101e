"""Shared synthetic inputs for the tests (the counterpart of /root/reference/tests/common.py:4-22).

Inputs are made with numpy / CPU torch generators so the CPU oracle and the GPU path see the same bits on any box."""
import numpy as np
import torch

from oracle import gaac_oracle as O


def kv_like16(H, S, seed=0, outliers=1e-3, scale_seed=None):
    """uint16 [H,S,128] BF16 bit patterns: Gaussian x per-channel scale 2^(U*8-4) shared across heads, each ELEMENT
    x1e4 with probability `outliers` (exercises all three tiers)."""
    rng = np.random.default_rng(seed)
    srng = rng if scale_seed is None else np.random.default_rng(scale_seed)
    scale = np.exp2(srng.random((1, 1, 128)) * 8 - 4)
    x = rng.standard_normal((H, S, 128)) * scale
    x = np.where(rng.random((H, S, 128)) < outliers, x * 1e4, x)
    return O.f32_to_bf16_rne(x.astype(np.float32))


def to_bf16(x16: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(x16).view(np.int16)).view(torch.bfloat16).to(device)


def to_u16(x: torch.Tensor) -> np.ndarray:
    return x.detach().contiguous().cpu().view(torch.int16).numpy().view(np.uint16)


def randn_bf16(shape, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    return O.f32_to_bf16_rne((rng.standard_normal(shape) * scale).astype(np.float32))
