"""Host side of the tile format: exponent-base calibration, page encoding and decoding, all computed by the HIP kernels of
libgaac_hip.so.

The names exported here (constants, perm_k / perm_v / perm, storage_index, exponent_hist, bases_from_hist, Page, Codec,
row_offsets) and their tensor shapes and dtypes are those of /root/reference/gaac/codec.py.  What a tile MEANS is the
reference's too: a BF16 element is a sign/mantissa byte plus an exponent; channels are permuted; 8 consecutive stored
elements form a group; a group's tier (3-bit codes / 4-bit codes / raw exponents) is recorded in a 2-bit tag; bytes that do
not fit the 3-bit codes go to a per-head escape stream, addressed through one offset per tile.  What differs is where the
bytes of a tile lie, because the attention kernel loads a tile straight into gfx950 MFMA operand registers:
  * sign/mantissa and code bytes are in the order storage_index returns, for K and for V;
  * K tag words and K escape bytes are in the reference's order (one tag word per token, escapes by token, then group);
  * V tag words and V escape bytes are TRANSPOSED within the tile: tag word a of a tile belongs to group a and holds the tags
    of its 16 tokens (token j at bits 2j), and the tile's escape bytes run by group, then token.
Per-tile escape byte counts, tile offsets and head starts are the same numbers as the reference's.  csrc/gaac_core.h states
the byte order in full."""
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
    """Channel held at each stored position of a K row (the permutation of codec.py:29-36): with pos = 32j + 4s + q, q < 4, s < 8,
    the channel is 16s + 2j + (0, 1, 8, 9)[q]."""
    pos = torch.arange(D)
    return 16 * ((pos >> 2) & 7) + 2 * (pos >> 5) + (pos & 1) + 8 * ((pos >> 1) & 1)


def perm_v(D: int = D) -> torch.Tensor:
    """Channel held at each stored position of a V row (the permutation of codec.py:39-45): pos = 16r + n, n < 16, holds channel 8n + r."""
    pos = torch.arange(D)
    return 8 * (pos & 15) + (pos >> 4)


def perm(kind: str) -> torch.Tensor:
    return perm_k() if kind == "k" else perm_v()


def storage_index(kind: str, dev) -> tuple[torch.Tensor, torch.Tensor]:
    """Byte order inside a tile, as two index tensors (sm_idx [T*D], code_idx [T*CB]): entry i names the byte of a token-major tile
    (tok*D + pos, resp. tok*CB + b) that this library stores at byte i.

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
    """Counts of the 8-bit exponent per (kv head, channel): x bf16 [..., n_kv, D] -> int64 [n_kv*D, 256] (the quantity of codec.py:80-84)."""
    x = x.contiguous()
    hist = torch.zeros(n_kv * D, 256, dtype=torch.int64, device=x.device)
    _lib.call("gaac_exponent_hist", _lib.ptr(x), x.numel() // (n_kv * D), n_kv, _lib.ptr(hist), _lib.stream())
    return hist


def bases_from_hist(hist: torch.Tensor, n_kv: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Exponent bases from a histogram [n_kv*D, 256]: per row the lowest exponent of the 8 (base3) and of the 16 (base4) consecutive
    exponents that cover the most samples, first such window on ties (codec.py:70-77).  Returns two uint8 [n_kv, D] tables."""
    hist = hist.to(torch.int64).contiguous()
    b3 = torch.empty(n_kv, D, dtype=torch.uint8, device=hist.device)
    b4 = torch.empty(n_kv, D, dtype=torch.uint8, device=hist.device)
    _lib.call("gaac_bases_from_hist", _lib.ptr(hist), n_kv * D, _lib.ptr(b3), _lib.ptr(b4), _lib.stream())
    return b3, b4


@dataclass
class Page:
    """H heads of encoded K or V, S tokens in every head; S_pad = S rounded up to whole tiles.  Field names and shapes are those of
    codec.py:87-102; the comments say what the bytes are HERE (see the module text for the order inside a tile)."""
    sm: torch.Tensor              # uint8 [H, S_pad*D]   sign+mantissa bytes, native tile order
    codes: torch.Tensor           # uint8 [H, S_pad*CB]  3-bit codes, native tile order
    flags: torch.Tensor           # int32 [H, S_pad]     16 tag words per tile: K one per token; V one per GROUP (token j at bits 2j)
    ovf_off: torch.Tensor         # int32 [H, S]         where the escapes of tag word i start in the head's stream (K: a token's, V: a group's)
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
        """Bytes the page occupies for S tokens per head: token rows (sign/mantissa, codes, tag word), escape bytes and one offset per tile.
        The base tables are left out (two [n_kv, D] byte tables per kind, shared by every page of a layer)."""
        esc = int(self.ovf_head_start[-1] - self.ovf_head_start[0])
        return self.H * self.S * (D + CB + 4) + esc + self.H * ((self.S + T - 1) // T) * 4

    @property
    def ratio(self) -> float:
        return self.H * self.S * D * 2 / self.nbytes


def row_offsets(flags: torch.Tensor, S: int) -> torch.Tensor:
    """Prefix sums of the escape bytes that the tag words announce: out[h, i] = start of tag word i's escapes within head h's stream
    (int32 [H, S]; the role of codec.py:221-225).  For K word i is token i.  For V word 16t + a is group a of tile t, and with
    S % 16 != 0 the last tile's words beyond S are cut off although they are valid: decode V through tile_off, as the kernels do."""
    flags = flags.contiguous()
    H, S_pad = flags.shape
    out = torch.empty(H, S, dtype=torch.int32, device=flags.device)
    if S:
        sums = torch.empty(H * ((S + 2047) // 2048), dtype=torch.int32, device=flags.device)
        _lib.call("gaac_row_offsets", _lib.ptr(flags), H, S, S_pad, _lib.ptr(sums), _lib.ptr(out), _lib.stream())
    return out


def encode_page(x: torch.Tensor, kind: str, base3: torch.Tensor, base4: torch.Tensor, n_kv: int, scratch=None) -> Page:
    """Encode x (bf16 [H, S, D], on the GPU) with the given bases.  Two launches: every tile is encoded with its escapes in a worst-case
    slot, then the slots are packed head by head into one stream (the steps of encoder.py:111-123)."""
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
    """Holds the two exponent-base tables of a layer (uint8 [n_kv, D] each) and encodes / decodes pages with them; the interface of
    codec.py:115-218."""
    def __init__(self, n_kv: int, device: str = "cuda"):
        self.n_kv, self.device = n_kv, device
        self.base3 = self.base4 = None

    def calibrate(self, sample: torch.Tensor) -> "Codec":
        """Derive the bases from sample, bf16 [H, tokens, D]; H may be a multiple of n_kv, head h then counts towards kv head h % n_kv."""
        H = sample.shape[0]
        x = sample.to(self.device).reshape(H // self.n_kv, self.n_kv, -1, D).permute(0, 2, 1, 3)   # [., T, n_kv, D]
        self.base3, self.base4 = bases_from_hist(exponent_hist(x, self.n_kv), self.n_kv)
        return self

    def set_bases(self, base3: torch.Tensor, base4: torch.Tensor) -> "Codec":
        self.base3 = base3.to(self.device, torch.uint8).reshape(self.n_kv, D).contiguous()
        self.base4 = base4.to(self.device, torch.uint8).reshape(self.n_kv, D).contiguous()
        return self

    def encode(self, x: torch.Tensor, kind: str) -> Page:
        """Page of x, bf16 [H, S, D]; head h is encoded with the bases of kv head h % n_kv."""
        return encode_page(x.to(self.device), kind, self.base3, self.base4, self.n_kv)

    @staticmethod
    def decode(page: Page) -> torch.Tensor:
        """The bf16 [H, S, D] tensor the page was made from, bit for bit."""
        H, S = page.H, page.S
        S_pad = page.sm.shape[1] // D
        out = torch.empty(H, S, D, dtype=torch.bfloat16, device=page.sm.device)
        if S:
            _lib.call("gaac_decode_tiles", 0 if page.kind == "k" else 1, _lib.ptr(page.sm), _lib.ptr(page.codes), _lib.ptr(page.flags),
                      _lib.ptr(page.tile_off), _lib.ptr(page.ovf), _lib.ptr(page.ovf_head_start), _lib.ptr(page.base3), _lib.ptr(page.base4),
                      page.n_kv, None, H, S, S_pad, _lib.ptr(out), S * D, D, _lib.stream())
        return out
