"""Tile encoder on MI355X: one wave64 per (head, 16-token tile).  Public surface of /root/reference/gaac/encoder.py:79-123.

Tiers, tag words and 3-bit codes are computed in registers, sign/mantissa and code bytes are written in the native tile
order, and each tile's escape bytes go to a bounded per-tile slot (1280 B worst case); compact() packs the slots into
each head's escape stream."""
from __future__ import annotations
import torch
from . import _lib
from .codec import Codec, Page, D, T, CB, TILE_MAX_ESC, perm, storage_index, row_offsets

SLOT = TILE_MAX_ESC


class TileEncoder:
    def __init__(self, kind: str, device="cuda"):
        self.kind = kind
        self.device = device
        self._slots = None
        self._tables = None

    def _layout(self):
        if self._tables is None:
            p = perm(self.kind).to(self.device).to(torch.int32)
            si, ci = storage_index(self.kind, self.device)
            inv_s = torch.empty_like(si); inv_s[si] = torch.arange(si.numel(), device=self.device)
            inv_c = torch.empty_like(ci); inv_c[ci] = torch.arange(ci.numel(), device=self.device)
            self._tables = (p, inv_s.to(torch.int32).contiguous(), inv_c.to(torch.int32).contiguous())
        return self._tables

    # layout tables of the reference object (the kernels do not read them: the order is compiled in)
    perm = property(lambda self: self._layout()[0])
    inv_sm = property(lambda self: self._layout()[1])
    inv_cd = property(lambda self: self._layout()[2])

    def _scratch(self, n: int, dev):
        if self._slots is None or self._slots.numel() < n:
            self._slots = torch.empty(n, dtype=torch.uint8, device=dev)
        return self._slots

    def encode_tiles(self, x, base3, base4, sm, cd, flags, S, S_pad, n_kv, bidx=None) -> torch.Tensor:
        """Encode x [H, S_in, D] (any head / token strides, e.g. a transposed view of a token-major prompt; tiles 0..ceil(S/16)-1) into sm/cd/flags with token stride S_pad; escape bytes stay in the
        scratch slots.  Returns tile_bytes int32 [H, ntiles]; finish with compact()."""
        H = x.shape[0]; ntiles = (S + T - 1) // T; dev = x.device
        if x.stride(2) != 1 or x.stride(0) % 8 or x.stride(1) % 8 or x.data_ptr() % 16:      # any head / row strides with 16-byte aligned rows
            x = x.contiguous()
        slots = self._scratch(H * ntiles * SLOT, dev)
        tile_bytes = torch.empty(H, ntiles, dtype=torch.int32, device=dev)
        _lib.call("gaac_encode_tiles", 0 if self.kind == "k" else 1, _lib.ptr(x), x.stride(0), x.stride(1), H, S, S_pad, _lib.ptr(base3), _lib.ptr(base4),
                  n_kv, _lib.ptr(bidx), _lib.ptr(sm), _lib.ptr(cd), _lib.ptr(flags), _lib.ptr(slots), _lib.ptr(tile_bytes), _lib.stream())
        return tile_bytes

    def compact(self, tile_bytes, head_start, ovf) -> torch.Tensor:
        """Pack the scratch slots into ovf at head_start[h] + tile_off[h, t]; returns tile_off int32 [H, ntiles]."""
        H, ntiles = tile_bytes.shape
        tile_off = torch.empty_like(tile_bytes)
        _lib.call("gaac_compact", _lib.ptr(self._slots), _lib.ptr(tile_bytes), _lib.ptr(tile_off), _lib.ptr(head_start), _lib.ptr(ovf),
                  H, ntiles, _lib.stream())
        return tile_off

    def encode(self, codec: Codec, x: torch.Tensor) -> Page:
        """x: [H, S, D] bf16 -> Page."""
        H, S, _ = x.shape; dev = x.device
        S_pad = (S + T - 1) // T * T
        sm = torch.empty(H, S_pad * D, dtype=torch.uint8, device=dev)
        cd = torch.empty(H, S_pad * CB, dtype=torch.uint8, device=dev)
        flags = torch.zeros(H, S_pad, dtype=torch.int32, device=dev)
        tile_bytes = self.encode_tiles(x, codec.base3, codec.base4, sm, cd, flags, S, S_pad, codec.n_kv)
        head_bytes = tile_bytes.sum(1)
        head_start = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev), torch.cumsum(head_bytes, 0)]).to(torch.int32).contiguous()
        ovf = torch.zeros(int(head_start[-1]) + 8, dtype=torch.uint8, device=dev)
        tile_off = self.compact(tile_bytes, head_start, ovf)
        return Page(sm, cd, flags, row_offsets(flags, S), ovf, head_start, tile_off, codec.base3, codec.base4, H, S, codec.n_kv, self.kind)
