"""CPU oracle for the GAAC compressed-KV decode path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this file: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg may use it, and only as the checker.  It restates, in numpy on raw BF16 bit patterns (uint16), what the
reference's pure-PyTorch codec computes, in the REFERENCE byte layout, so its pages can be compared field by
field with pages the reference itself would produce:

  perm_k / perm_v / storage_index      /root/reference/gaac/codec.py:29-67
  exponent_hist / bases_from_hist      /root/reference/gaac/codec.py:70-84
  encode                               /root/reference/gaac/codec.py:133-184
  decode                               /root/reference/gaac/codec.py:186-218
  row_offsets                          /root/reference/gaac/codec.py:221-225
  page_nbytes                          /root/reference/gaac/codec.py:104-112
  ref_attention                        /root/reference/tests/common.py:15-22
  cache_stats / bytes_per_slot         /root/reference/gaac/kv_cache.py:142-146, 228-234

How each function is pinned (tests/test_oracle.py):
  * encode / storage_index / perms: golden pages written once by the reference's own codec
    (tests/golden/codec_*.npz, made by tests/golden/make_codec_golden.py) compared field by field;
    plus an independent scalar encoder (pure Python loops over the format rules) on small inputs.
  * decode: decode(encode(x)) == x for every bit pattern class (NaN, Inf, denormal, -0), decode of the golden pages
    equals the golden input.
  * bases_from_hist: brute-force sliding-window argmax with first-max tie break.  exponent_hist: np.bincount.
  * row_offsets / tile_off: exclusive cumsum of per-row escape bytes recomputed from tiers.
  * ref_attention: float64 softmax attention written with explicit loops on small inputs.
  * byte accounting: closed forms 11.25 / 12.25 / 16.25 bits per element.
"""
from __future__ import annotations
from dataclasses import dataclass
import numpy as np

D = 128          # head dim
T = 16           # tokens per tile
GS = 8           # elements per group
NG = D // GS     # groups per token row
CB = D * 3 // 8  # code bytes per token row
TAIL = 16
TILE_MAX_ESC = T * NG * 5


def perm_k() -> np.ndarray:
    """stored position -> channel for K: position 32j+4s+q holds channel 16s+2j+(0,1,8,9)[q]."""
    p = np.empty(D, dtype=np.int64)
    for pos in range(D):
        j, s, q = pos >> 5, (pos >> 2) & 7, pos & 3
        p[pos] = 16 * s + 2 * j + (0, 1, 8, 9)[q]
    return p


def perm_v() -> np.ndarray:
    """stored position -> channel for V: position 16r+n holds channel 8n+r."""
    pos = np.arange(D)
    return 8 * (pos & 15) + (pos >> 4)


def perm(kind: str) -> np.ndarray:
    return perm_k() if kind == "k" else perm_v()


def storage_index(kind: str) -> tuple[np.ndarray, np.ndarray]:
    """Reference tile byte order: (sm_idx[2048], cd_idx[768]) = storage byte -> token-major byte (tok*D+pos / tok*CB+b)."""
    sm, cd = [], []
    if kind == "k":
        for octet in range(2):
            for lane in range(32):
                tok, j = 8 * octet + lane // 4, lane % 4
                sm.extend(tok * D + 32 * j + np.arange(32))
                cd.extend(tok * CB + 12 * j + np.arange(12))
    else:
        for lane in range(32):
            j, r = lane % 4, lane // 4
            for tok in (2 * j, 2 * j + 1, 2 * j + 8, 2 * j + 9):
                sm.extend(tok * D + 16 * r + np.arange(16))
                cd.extend(tok * CB + 6 * r + np.arange(6))
    return np.asarray(sm, dtype=np.int64), np.asarray(cd, dtype=np.int64)


def exponent_of(x16: np.ndarray) -> np.ndarray:
    return (x16.astype(np.int32) >> 7) & 0xFF


def exponent_hist(x16: np.ndarray, n_kv: int) -> np.ndarray:
    """x16: uint16 [..., n_kv, D] token-major -> int64 [n_kv*D, 256]."""
    e = exponent_of(x16).reshape(-1, n_kv * D)
    hist = np.zeros((n_kv * D, 256), dtype=np.int64)
    for c in range(n_kv * D):
        hist[c] = np.bincount(e[:, c], minlength=256)
    return hist


def bases_from_hist(hist: np.ndarray, n_kv: int) -> tuple[np.ndarray, np.ndarray]:
    """Start of the densest 8-wide and 16-wide exponent window per row; the lowest start wins ties."""
    cs = np.concatenate([np.zeros((hist.shape[0], 1), dtype=np.float64), np.cumsum(hist.astype(np.float64), 1)], 1)
    out = []
    for w in (8, 16):
        out.append(np.argmax(cs[:, w:] - cs[:, :-w], 1).astype(np.uint8).reshape(n_kv, D))
    return out[0], out[1]


def calibrate(sample16: np.ndarray, n_kv: int) -> tuple[np.ndarray, np.ndarray]:
    """sample16: uint16 [H, T, D]; head h pools into kv head h % n_kv (codec.py:121-126)."""
    H = sample16.shape[0]
    x = sample16.reshape(H // n_kv, n_kv, -1, D).transpose(0, 2, 1, 3)
    return bases_from_hist(exponent_hist(x, n_kv), n_kv)


@dataclass
class OPage:
    """Reference-layout page (same fields as the reference's Page dataclass, numpy arrays)."""
    sm: np.ndarray              # uint8 [H, S_pad*D]
    codes: np.ndarray           # uint8 [H, S_pad*CB]
    flags: np.ndarray           # int32 [H, S_pad]
    ovf_off: np.ndarray         # int32 [H, S]
    ovf: np.ndarray             # uint8 [total+8]
    ovf_head_start: np.ndarray  # int32 [H+1]
    tile_off: np.ndarray        # int32 [H, S_pad/16]
    base3: np.ndarray           # uint8 [n_kv, D]
    base4: np.ndarray           # uint8 [n_kv, D]
    H: int
    S: int
    n_kv: int
    kind: str


def page_nbytes(H: int, S: int, esc: int) -> int:
    return H * S * (D + CB + 4) + esc + H * ((S + T - 1) // T) * 4


def tiers_of(e_st: np.ndarray, b3_st: np.ndarray, b4_st: np.ndarray):
    """e_st: int32 [H,S,D] exponents in stored order, b*_st: [H,1,D] -> (tier [H,S,NG], d3, d4)."""
    d3, d4 = e_st - b3_st, e_st - b4_st
    H, S, _ = e_st.shape
    fit3 = ((d3 >= 0) & (d3 <= 7)).reshape(H, S, NG, GS).all(-1)
    fit4 = ((d4 >= 0) & (d4 <= 15)).reshape(H, S, NG, GS).all(-1)
    tier = np.where(fit3, 0, np.where(fit4, 1, 2)).astype(np.int32)
    return tier, d3, d4


def encode_token_major(x16: np.ndarray, kind: str, base3: np.ndarray, base4: np.ndarray, n_kv: int, bidx=None):
    """Everything up to (not including) the tile storage permutation.  Returns a dict of token-major arrays:
    sm [H,S,D] u8, codes [H,S,CB] u8, flags [H,S] u32, tier [H,S,NG], row_bytes [H,S], esc = list of per-head uint8 arrays."""
    H, S, _ = x16.shape
    p = perm(kind)
    xs = x16.astype(np.int32)[..., p]
    e = (xs >> 7) & 0xFF
    sm = (((xs >> 8) & 0x80) | (xs & 0x7F)).astype(np.uint8)
    hidx = (np.arange(H) % n_kv) if bidx is None else np.asarray(bidx)
    b3 = base3.astype(np.int32)[hidx][:, p][:, None, :]
    b4 = base4.astype(np.int32)[hidx][:, p][:, None, :]
    tier, d3, d4 = tiers_of(e, b3, b4)
    tier_e = np.repeat(tier, GS, axis=-1)
    code = np.where(tier_e == 0, d3 & 7, np.where(tier_e == 1, d4 & 7, e & 7)).astype(np.uint32)
    # 24-bit little-endian word per group: code i at bits 3i..3i+2
    w24 = (code.reshape(H, S, NG, GS) << (3 * np.arange(GS, dtype=np.uint32))).sum(-1).astype(np.uint32)
    codes = np.stack([(w24 >> 0) & 0xFF, (w24 >> 8) & 0xFF, (w24 >> 16) & 0xFF], -1).astype(np.uint8).reshape(H, S, CB)
    g = np.arange(NG, dtype=np.uint64)
    flags = (((tier >= 1).astype(np.uint64) << (2 * g)) | ((tier == 2).astype(np.uint64) << (2 * g + 1))).sum(-1).astype(np.uint32)
    gsize = np.where(tier == 1, 1, np.where(tier == 2, 5, 0)).astype(np.int64)
    row_bytes = gsize.sum(-1)
    bit4 = (((d4 >> 3) & 1).reshape(H, S, NG, GS) << np.arange(GS)).sum(-1).astype(np.uint8)
    hi5 = ((e >> 3).astype(np.uint64).reshape(H, S, NG, GS) << (5 * np.arange(GS, dtype=np.uint64))).sum(-1)
    esc = []
    for h in range(H):
        t, gs = tier[h].reshape(-1), gsize[h].reshape(-1)
        start = np.cumsum(gs) - gs
        buf = np.zeros(int(gs.sum()), dtype=np.uint8)
        m1 = t == 1
        buf[start[m1]] = bit4[h].reshape(-1)[m1]
        m2 = t == 2
        if m2.any():
            w = hi5[h].reshape(-1)[m2]
            for k in range(5):
                buf[start[m2] + k] = ((w >> np.uint64(8 * k)) & np.uint64(0xFF)).astype(np.uint8)
        esc.append(buf)
    return dict(sm=sm, codes=codes, flags=flags, tier=tier, row_bytes=row_bytes, esc=esc)


def encode(x16: np.ndarray, kind: str, base3: np.ndarray, base4: np.ndarray, n_kv: int, bidx=None) -> OPage:
    """x16: uint16 [H,S,D] -> reference-layout page."""
    H, S, _ = x16.shape
    tm = encode_token_major(x16, kind, base3, base4, n_kv, bidx)
    S_pad = (S + T - 1) // T * T
    sm = np.zeros((H, S_pad, D), dtype=np.uint8); sm[:, :S] = tm["sm"]
    cd = np.zeros((H, S_pad, CB), dtype=np.uint8); cd[:, :S] = tm["codes"]
    si, ci = storage_index(kind)
    sm_st = sm.reshape(H, S_pad // T, T * D)[:, :, si].reshape(H, S_pad * D)
    cd_st = cd.reshape(H, S_pad // T, T * CB)[:, :, ci].reshape(H, S_pad * CB)
    rb = tm["row_bytes"]
    head_start = np.concatenate([[0], np.cumsum(rb.sum(1))]).astype(np.int64)
    ovf_off = (np.cumsum(rb, 1) - rb).astype(np.int32)
    ovf = np.zeros(int(head_start[-1]) + 8, dtype=np.uint8)
    for h in range(H):
        ovf[head_start[h]:head_start[h + 1]] = tm["esc"][h]
    flags = np.zeros((H, S_pad), dtype=np.int32)
    flags[:, :S] = tm["flags"].view(np.int32) if tm["flags"].dtype == np.uint32 else tm["flags"]
    return OPage(np.ascontiguousarray(sm_st), np.ascontiguousarray(cd_st), flags, ovf_off, ovf, head_start.astype(np.int32),
                 np.ascontiguousarray(ovf_off[:, ::T]), base3, base4, H, S, n_kv, kind)


def row_offsets(flags: np.ndarray, S: int) -> np.ndarray:
    f = flags[:, :S].astype(np.int64) & 0xFFFFFFFF
    rb = np.zeros_like(f)
    for g in range(NG):
        rb += ((f >> (2 * g)) & 1) + 4 * ((f >> (2 * g + 1)) & 1)
    return (np.cumsum(rb, 1) - rb).astype(np.int32)


def decode(page: OPage, bidx=None) -> np.ndarray:
    """Reference-layout page -> uint16 [H,S,D], bit-exact."""
    H, S = page.H, page.S
    S_pad = page.sm.shape[1] // D
    si, ci = storage_index(page.kind)
    sm_tm = np.empty((H, S_pad // T, T * D), dtype=np.uint8)
    sm_tm[:, :, si] = page.sm.reshape(H, S_pad // T, T * D)
    cd_tm = np.empty((H, S_pad // T, T * CB), dtype=np.uint8)
    cd_tm[:, :, ci] = page.codes.reshape(H, S_pad // T, T * CB)
    sm = sm_tm.reshape(H, S_pad, D)[:, :S].astype(np.int32)
    cd = cd_tm.reshape(H, S_pad, NG, 3)[:, :S].astype(np.uint32)
    w24 = cd[..., 0] | (cd[..., 1] << 8) | (cd[..., 2] << 16)
    code = ((w24[..., None] >> (3 * np.arange(GS, dtype=np.uint32))) & 7).astype(np.int32)          # [H,S,NG,GS]
    p = perm(page.kind)
    hidx = (np.arange(H) % page.n_kv) if bidx is None else np.asarray(bidx)
    b3 = page.base3.astype(np.int32)[hidx][:, p].reshape(H, 1, NG, GS)
    b4 = page.base4.astype(np.int32)[hidx][:, p].reshape(H, 1, NG, GS)
    f = page.flags[:, :S].astype(np.int64) & 0xFFFFFFFF
    tag = np.stack([(f >> (2 * g)) & 3 for g in range(NG)], -1)                                      # 0, 1, 3
    gsize = np.where(tag == 1, 1, np.where(tag == 3, 5, 0)).astype(np.int64)
    gstart = page.ovf_head_start[:-1].astype(np.int64).reshape(H, 1, 1) + page.ovf_off.astype(np.int64)[..., None] + (np.cumsum(gsize, -1) - gsize)
    ovf = page.ovf.astype(np.int64)
    last = ovf.size - 1
    b0 = ovf[np.minimum(gstart, last)]
    bit4 = ((b0[..., None] >> np.arange(GS)) & 1).astype(np.int32)
    w40 = np.zeros_like(gstart)
    for k in range(5):
        w40 |= ovf[np.minimum(gstart + k, last)] << (8 * k)
    hi5 = ((w40[..., None] >> (5 * np.arange(GS))) & 31).astype(np.int32)
    tg = tag[..., None]
    exp = np.where(tg == 0, b3 + code, np.where(tg == 1, b4 + (code | (bit4 << 3)), code | (hi5 << 3)))
    raw = ((sm.reshape(H, S, NG, GS) & 0x80) << 8) | (exp << 7) | (sm.reshape(H, S, NG, GS) & 0x7F)
    out = np.empty((H, S, D), dtype=np.uint16)
    out[..., p] = raw.reshape(H, S, D).astype(np.uint16)
    return out


def bf16_to_f32(x16: np.ndarray) -> np.ndarray:
    return (x16.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_rne(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + np.uint32(0x7FFF)
    return ((u + r) >> 16).astype(np.uint16)


def ref_attention(q16: np.ndarray, k16: np.ndarray, v16: np.ndarray, scale: float) -> np.ndarray:
    """q16 [n_q,D], k16/v16 [L,n_kv,D] (uint16 bf16 bits) -> float32 [n_q,D]; q head j reads kv head j // G."""
    n_q, n_kv = q16.shape[0], k16.shape[1]
    G = n_q // n_kv
    q = bf16_to_f32(q16)
    out = np.zeros((n_q, D), dtype=np.float32)
    for h in range(n_kv):
        k = bf16_to_f32(k16[:, h]); v = bf16_to_f32(v16[:, h])
        s = (q[h * G:(h + 1) * G] @ k.T) * np.float32(scale)
        s = s - s.max(-1, keepdims=True)
        p = np.exp(s); p /= p.sum(-1, keepdims=True)
        out[h * G:(h + 1) * G] = p @ v
    return out


def bytes_per_slot(n_kv: int, capacity: int, ovf_bytes_per_tile: int = 128, per_sequence_bases: bool = True) -> int:
    cap = (capacity + T - 1) // T * T
    per_head = cap * (D + CB + 4) + (cap // T) * 4 + (cap // T) * ovf_bytes_per_tile + 8 + 8 + TAIL * D * 2 + (2 * D if per_sequence_bases else 0)
    return 2 * n_kv * per_head + 8 * n_kv


def cache_stats(S_sum: int, tail_sum: int, esc: int, n_kv: int) -> dict:
    used = 2 * (S_sum * (D + CB + 4) + (S_sum // T) * 4 + tail_sum * D * 2) + esc
    bf16 = 2 * (S_sum + tail_sum) * D * 2
    return dict(tokens=(S_sum + tail_sum) // max(1, n_kv), bytes_used=used, bf16_bytes=bf16, ratio=bf16 / max(1, used))


# ---- paged slot geometry (/root/reference/gaac/vllm/store.py:17-19, 62-64) -------------------------------------------
SM_OFF, CD_OFF, FL_OFF, OVF_OFF = 0, 2048, 2816, 2880


def slot_fits(tile_escape_bytes: int, ovf_slot: int = 128) -> bool:
    return tile_escape_bytes <= ovf_slot
