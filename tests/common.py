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


def attention_error_bound(q16: np.ndarray, k16: np.ndarray, v16: np.ndarray, scale: float):
    """(ref, tol): the oracle's fp32 attention and an elementwise bound on a kernel that, like the reference's
    (/root/reference/gaac/kernel.py:178-182), rounds the softmax weights to BF16 before the second product:
    tol[j, d] = 2^-8 * sum_t p[j, t] * |v[t, d]|  (each weight is off by at most 2^-9 relative: half a unit of BF16's 8 significant bits;
    the factor 2 is slack for the fp32 summation orders)  +  the reference's own 2e-2 * max|ref| + 1e-3 (tests/test_kernel.py:19).
    The weights and the first term are computed in float64.  Unlike a bound on |ref| alone, the first term does not vanish when large
    values of opposite sign cancel in the result."""
    ref = O.ref_attention(q16, k16, v16, scale)
    n_q, n_kv = q16.shape[0], k16.shape[1]
    G = n_q // n_kv
    q = O.bf16_to_f32(q16).astype(np.float64)
    rnd = np.zeros((n_q, 128), np.float64)
    for h in range(n_kv):
        k = O.bf16_to_f32(k16[:, h]).astype(np.float64); v = O.bf16_to_f32(v16[:, h]).astype(np.float64)
        s = (q[h * G:(h + 1) * G] @ k.T) * scale
        p = np.exp(s - s.max(-1, keepdims=True)); p /= p.sum(-1, keepdims=True)
        rnd[h * G:(h + 1) * G] = p @ np.abs(v)
    return ref, 2.0 ** -8 * rnd + 2e-2 * np.abs(ref).max() + 1e-3
