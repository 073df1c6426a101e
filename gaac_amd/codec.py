"""Lossless BF16 KV format: calibration, encoder and bit-exact decoder on MI355X.

Same public surface as /root/reference/gaac/codec.py (constants, perm_k/perm_v/perm, storage_index, bases_from_hist,
exponent_hist, Page, Codec, row_offsets) with the same tensor shapes and dtypes; the arithmetic runs in the HIP
kernels of libgaac_hip.so.  The format is the reference's (element split, channel permutation, 8-element groups, tier
rule, 3-bit codes, tag words, escape stream, tile offsets); only the order of the sign/mantissa and code bytes INSIDE a
16-token tile differs: it is the gfx950 MFMA operand order (storage_index returns it), see csrc/gaac_core.h.
"""
from __future__ import annotations
from dataclasses import dataclass
import torch
from . import _lib

D = 128     # head dim
T = 16      # tokens per tile
GS = 8      # elements per group
CB = D * 3 // 8   # code bytes per token row
TILE_MAX_ESC = T * (D // GS) * 5


def perm_k(D: int = D) -> torch.Tensor:
    """K stored position -> channel: position 32j+4s+q holds channel 16s+2j+(0,1,8,9)[q] (codec.py:29-36)."""
    pos = torch.arange(D)
    return 16 * ((pos >> 2) & 7) + 2 * (pos >> 5) + (pos & 1) + 8 * ((pos >> 1) & 1)


def perm_v(D: int = D) -> torch.Tensor:
    """V stored position -> channel: position 16r+n holds channel 8n+r (codec.py:39-45)."""
    pos = torch.arange(D)
    return 8 * (pos & 15) + (pos >> 4)


def perm(kind: str) -> torch.Tensor:
    return perm_k() if kind == "k" else perm_v()


def storage_index(kind: str, dev) -> tuple[torch.Tensor, torch.Tensor]:
    """(sm_idx [T*D], code_idx [T*CB]): native storage byte -> token-major byte (tok*D + pos / tok*CB + b) within one tile.

    Lane l = a + 16q of the wave that owns the tile holds four units (8-element groups); K: unit u = (token a, group 4q+u),
    V: unit u = (token 4q+u, group a).  sm byte 1024j + 16l + 8v + i = element i of unit 2j+v; code byte 256k + 4l + b =
    byte 4k+b of the lane's 12 code bytes (unit u owns bytes 3u..3u+2)."""
    l = torch.arange(64)
    a, q = l & 15, l >> 4
    sm = torch.empty(T * D, dtype=torch.long)
    cd = torch.empty(T * CB, dtype=torch.long)
    for u in range(4):
        tok, grp = (a, 4 * q + u) if kind == "k" else (4 * q + u, a)
        j, v = u >> 1, u & 1
        for i in range(8):
            sm[1024 * j + 16 * l + 8 * v + i] = tok * D + 8 * grp + i
        for b in range(3):
            c = 3 * u + b
            cd[256 * (c >> 2) + 4 * l + (c & 3)] = tok * CB + 3 * grp + b
    return sm.to(dev), cd.to(dev)


def exponent_hist(x: torch.Tensor, n_kv: int) -> torch.Tensor:
    """x: [..., n_kv, D] bf16 (token-major) -> int64 [n_kv*D, 256] exponent histogram (codec.py:80-84)."""
    x = x.contiguous()
    hist = torch.zeros(n_kv * D, 256, dtype=torch.int64, device=x.device)
    _lib.call("gaac_exponent_hist", _lib.ptr(x), x.numel() // (n_kv * D), n_kv, _lib.ptr(hist), _lib.stream())
    return hist


def bases_from_hist(hist: torch.Tensor, n_kv: int) -> tuple[torch.Tensor, torch.Tensor]:
    """hist: [n_kv*D, 256] counts -> (base3, base4) uint8 [n_kv, D]: start of the densest 8- / 16-wide window (codec.py:70-77)."""
    hist = hist.to(torch.int64).contiguous()
    b3 = torch.empty(n_kv, D, dtype=torch.uint8, device=hist.device)
    b4 = torch.empty(n_kv, D, dtype=torch.uint8, device=hist.device)
    _lib.call("gaac_bases_from_hist", _lib.ptr(hist), n_kv * D, _lib.ptr(b3), _lib.ptr(b4), _lib.stream())
    return b3, b4


@dataclass
class Page:
    """Compressed K or V of H heads x S tokens (all heads the same length).  Fields as codec.py:87-102."""
    sm: torch.Tensor              # uint8 [H, S_pad*D]   sign+mantissa bytes, native tile order
    codes: torch.Tensor           # uint8 [H, S_pad*CB]  3-bit codes, native tile order
    flags: torch.Tensor           # int32 [H, S_pad]     per-row tag words (0 for padded rows)
    ovf_off: torch.Tensor         # int32 [H, S]         row offset within the head's escape stream
    ovf: torch.Tensor             # uint8 [total + 8]    escape bytes of all heads
    ovf_head_start: torch.Tensor  # int32 [H+1]
    tile_off: torch.Tensor        # int32 [H, S_pad/16]  tile offset within the head's escape stream
    base3: torch.Tensor           # uint8 [n_kv, D]
    base4: torch.Tensor           # uint8 [n_kv, D]
    H: int
    S: int
    n_kv: int
    kind: str                     # 'k' | 'v'

    @property
    def nbytes(self) -> int:
        """Stored bytes: sign/mantissa + codes + escapes + tags + tile offsets (bases excluded: 4 KiB per layer)."""
        esc = int(self.ovf_head_start[-1] - self.ovf_head_start[0])
        return self.H * self.S * (D + CB + 4) + esc + self.H * ((self.S + T - 1) // T) * 4

    @property
    def ratio(self) -> float:
        return self.H * self.S * D * 2 / self.nbytes


def row_offsets(flags: torch.Tensor, S: int) -> torch.Tensor:
    """Row offsets within each head's escape stream from the tag words (codec.py:221-225)."""
    flags = flags.contiguous()
    H, S_pad = flags.shape
    out = torch.empty(H, S, dtype=torch.int32, device=flags.device)
    if S:
        sums = torch.empty(H * ((S + 2047) // 2048), dtype=torch.int32, device=flags.device)
        _lib.call("gaac_row_offsets", _lib.ptr(flags), H, S, S_pad, _lib.ptr(sums), _lib.ptr(out), _lib.stream())
    return out


def encode_page(x: torch.Tensor, kind: str, base3: torch.Tensor, base4: torch.Tensor, n_kv: int, scratch=None) -> Page:
    """x: [H, S, D] bf16 on the GPU -> Page.  Host-side steps mirror TileEncoder.encode (encoder.py:111-123)."""
    H, S, _ = x.shape
    dev = x.device
    x = x.contiguous()
    S_pad = (S + T - 1) // T * T
    ntiles = S_pad // T
    sm = torch.empty(H, S_pad * D, dtype=torch.uint8, device=dev)
    cd = torch.empty(H, S_pad * CB, dtype=torch.uint8, device=dev)
    flags = torch.empty(H, S_pad, dtype=torch.int32, device=dev)
    slots = scratch(H * ntiles * TILE_MAX_ESC, dev) if scratch else torch.empty(H * ntiles * TILE_MAX_ESC, dtype=torch.uint8, device=dev)
    tile_bytes = torch.empty(H, ntiles, dtype=torch.int32, device=dev)
    k = 0 if kind == "k" else 1
    _lib.call("gaac_encode_tiles", k, _lib.ptr(x), S * D, D, H, S, S_pad, _lib.ptr(base3), _lib.ptr(base4), n_kv, None,
              _lib.ptr(sm), _lib.ptr(cd), _lib.ptr(flags), _lib.ptr(slots), _lib.ptr(tile_bytes), _lib.stream())
    head_bytes = tile_bytes.sum(1)
    head_start = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev), torch.cumsum(head_bytes, 0)]).to(torch.int32).contiguous()
    ovf = torch.zeros(int(head_start[-1]) + 8, dtype=torch.uint8, device=dev)
    tile_off = torch.empty_like(tile_bytes)
    _lib.call("gaac_compact", _lib.ptr(slots), _lib.ptr(tile_bytes), _lib.ptr(tile_off), _lib.ptr(head_start), _lib.ptr(ovf),
              H, ntiles, _lib.stream())
    return Page(sm, cd, flags, row_offsets(flags, S), ovf, head_start, tile_off, base3, base4, H, S, n_kv, kind)


class Codec:
    """Per-(kv head, channel) exponent bases + encoder/decoder (codec.py:115-218)."""
    def __init__(self, n_kv: int, device: str = "cuda"):
        self.n_kv, self.device = n_kv, device
        self.base3 = self.base4 = None

    def calibrate(self, sample: torch.Tensor) -> "Codec":
        """sample: [H, T, D] bf16 with head h using bases of h % n_kv."""
        H = sample.shape[0]
        x = sample.to(self.device).reshape(H // self.n_kv, self.n_kv, -1, D).permute(0, 2, 1, 3)   # [., T, n_kv, D]
        self.base3, self.base4 = bases_from_hist(exponent_hist(x, self.n_kv), self.n_kv)
        return self

    def set_bases(self, base3: torch.Tensor, base4: torch.Tensor) -> "Codec":
        self.base3 = base3.to(self.device, torch.uint8).reshape(self.n_kv, D).contiguous()
        self.base4 = base4.to(self.device, torch.uint8).reshape(self.n_kv, D).contiguous()
        return self

    def encode(self, x: torch.Tensor, kind: str) -> Page:
        """x: [H, S, D] bf16 -> Page."""
        return encode_page(x.to(self.device), kind, self.base3, self.base4, self.n_kv)

    @staticmethod
    def decode(page: Page) -> torch.Tensor:
        """Bit-exact reconstruction: Page -> [H, S, D] bf16."""
        H, S = page.H, page.S
        S_pad = page.sm.shape[1] // D
        out = torch.empty(H, S, D, dtype=torch.bfloat16, device=page.sm.device)
        if S:
            _lib.call("gaac_decode_tiles", 0 if page.kind == "k" else 1, _lib.ptr(page.sm), _lib.ptr(page.codes), _lib.ptr(page.flags),
                      _lib.ptr(page.tile_off), _lib.ptr(page.ovf), _lib.ptr(page.ovf_head_start), _lib.ptr(page.base3), _lib.ptr(page.base4),
                      page.n_kv, None, H, S, S_pad, _lib.ptr(out), S * D, D, _lib.stream())
        return out
