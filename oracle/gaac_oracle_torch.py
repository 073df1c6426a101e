"""The reference's CPU path in PyTorch ops, for bench.py's cpu_baseline leg.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this file.  The reference's CPU-runnable path is its pure-PyTorch codec
(/root/reference/gaac/codec.py:186-218, Codec.decode) followed by fp32 scaled-dot-product attention over the decoded rows
(/root/reference/tests/common.py:15-22, /root/reference/examples/attention.py:32); this file restates both with torch tensor ops on
host tensors, so that the timed baseline runs on the library the reference's own CPU path runs on (torch's intra-op thread pool)
instead of numpy.  It works on the reference-layout page of oracle/gaac_oracle.py (OPage), a chunk of token rows at a time: the
reference's one-shot decode materialises [H, S, 128, 3]-shaped int64 temporaries, gigabytes at 64K tokens.

Pinned by tests/test_oracle.py: decode_torch equals the numpy oracle's decode (itself pinned by the reference-written golden pages)
bit for bit on the golden pages and on random pages with all three tiers; sdpa_torch equals the oracle's ref_attention.
"""
from __future__ import annotations
import numpy as np
import torch

from .gaac_oracle import D, T, GS, NG, CB, OPage, perm, storage_index


def decode_torch(page: OPage, rows_per_chunk: int = 8192) -> torch.Tensor:
    """Reference-layout page -> int16 tensor [H, S, D] holding the BF16 bit patterns (view as torch.bfloat16 for the values)."""
    H, S = page.H, page.S
    S_pad = page.sm.shape[1] // D
    si, ci = (torch.from_numpy(x) for x in storage_index(page.kind))
    p = torch.from_numpy(perm(page.kind))
    hidx = torch.arange(H) % page.n_kv
    b3 = torch.from_numpy(page.base3.astype(np.int32))[hidx][:, p].reshape(H, 1, NG, GS)
    b4 = torch.from_numpy(page.base4.astype(np.int32))[hidx][:, p].reshape(H, 1, NG, GS)
    sm_st = torch.from_numpy(page.sm).reshape(H, S_pad // T, T * D)
    cd_st = torch.from_numpy(page.codes).reshape(H, S_pad // T, T * CB)
    flags = torch.from_numpy(page.flags)
    ovf_off = torch.from_numpy(page.ovf_off).to(torch.int64)
    head0 = torch.from_numpy(page.ovf_head_start[:-1].astype(np.int64)).reshape(H, 1, 1)
    ovf = torch.from_numpy(page.ovf).to(torch.int64)
    last = ovf.numel() - 1
    sh3 = 3 * torch.arange(GS, dtype=torch.int32)
    sh5 = 5 * torch.arange(GS, dtype=torch.int64)
    sh1 = torch.arange(GS, dtype=torch.int64)
    g2 = 2 * torch.arange(NG, dtype=torch.int64)
    out = torch.empty(H, S, D, dtype=torch.int16)
    step = max(T, rows_per_chunk // T * T)
    for s0 in range(0, S, step):
        s1 = min(S, s0 + step); n = s1 - s0
        t0, t1 = s0 // T, -(-s1 // T)
        # tile storage order -> token-major rows
        sm_tm = torch.empty(H, t1 - t0, T * D, dtype=torch.uint8); sm_tm[:, :, si] = sm_st[:, t0:t1]
        cd_tm = torch.empty(H, t1 - t0, T * CB, dtype=torch.uint8); cd_tm[:, :, ci] = cd_st[:, t0:t1]
        sm = sm_tm.reshape(H, -1, NG, GS)[:, :n].to(torch.int32)
        cd = cd_tm.reshape(H, -1, NG, 3)[:, :n].to(torch.int32)
        w24 = cd[..., 0] | (cd[..., 1] << 8) | (cd[..., 2] << 16)
        code = (w24.unsqueeze(-1) >> sh3) & 7                                          # [H, n, NG, GS]
        f = flags[:, s0:s1].to(torch.int64) & 0xFFFFFFFF
        tag = (f.unsqueeze(-1) >> g2) & 3                                              # 0, 1, 3
        gsize = torch.where(tag == 1, 1, torch.where(tag == 3, 5, 0))
        gstart = head0 + ovf_off[:, s0:s1].unsqueeze(-1) + (gsize.cumsum(-1) - gsize)
        b0 = ovf[gstart.clamp(max=last)]
        bit4 = ((b0.unsqueeze(-1) >> sh1) & 1).to(torch.int32)
        w40 = torch.zeros_like(gstart)
        for k in range(5):
            w40 |= ovf[(gstart + k).clamp(max=last)] << (8 * k)
        hi5 = ((w40.unsqueeze(-1) >> sh5) & 31).to(torch.int32)
        tg = tag.unsqueeze(-1)
        exp = torch.where(tg == 0, b3 + code, torch.where(tg == 1, b4 + (code | (bit4 << 3)), code | (hi5 << 3)))
        raw = ((sm & 0x80) << 8) | (exp << 7) | (sm & 0x7F)
        raw = torch.where(raw >= 0x8000, raw - 0x10000, raw).to(torch.int16).reshape(H, n, D)
        out[:, s0:s1][..., p] = raw
    return out


def sdpa_torch(q16: np.ndarray, kdec: torch.Tensor, vdec: torch.Tensor, scale: float) -> torch.Tensor:
    """q16: uint16 [n_q, D] BF16 bits; kdec / vdec: int16 [n_kv, S, D] BF16 bits (decode_torch) -> float32 [n_q, D]: fp32 softmax
    attention, query head j over kv head j // G, through torch's scaled_dot_product_attention."""
    n_q, n_kv = q16.shape[0], kdec.shape[0]
    q = torch.from_numpy(q16.astype(np.int16)).view(torch.bfloat16).float().view(1, n_q, 1, D)
    k = kdec.view(torch.bfloat16).float().unsqueeze(0); v = vdec.view(torch.bfloat16).float().unsqueeze(0)
    o = torch.nn.functional.scaled_dot_product_attention(q, k, v, scale=scale, enable_gqa=n_q != n_kv)
    return o.view(n_q, D)
