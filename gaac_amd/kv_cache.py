"""Slot-based compressed KV cache of one attention layer, resident in HBM, behind the interface of
/root/reference/gaac/kv_cache.py:122-234 (constructor arguments, method names, attribute names and tensor shapes are that
class's, so an engine written against it runs unchanged).

Layout: slot s owns cache heads [s*n_kv, (s+1)*n_kv).  Per head and kind there are `cap` token rows of compressed tiles
(16 tokens each), a fixed window of `ovf_cap` bytes in the escape buffer, and a 16-row BF16 staging tail that collects
tokens until a tile is complete.  A decode step costs two launches on the current stream and never returns to the host:
`append` writes one token per batch row (and encodes the tile in place on the step that completes it), `attention` reads
tiles + tail.  Both take the batch's slot map from device memory, so the step can be captured in a HIP graph; a row whose
slot is -1 is left alone (its attention output is exactly 0).  Exponent bases come either from the caller ([n_kv, D],
shared by all sequences) or from each prompt at prefill ([n_slots*n_kv, D]).

The escape buffers carry 8 bytes of padding behind the last head's window, because the kernels fetch escape bytes with
unaligned 8-byte loads that may reach past a head's last escape byte; bytes_per_slot counts that padding per head."""
from __future__ import annotations
import torch
from . import _lib
from .codec import Codec, Page, D, T, CB, TILE_MAX_ESC, row_offsets
from .encoder import TileEncoder
from .kernel import _ext, choose_nsplit, attn_launch, AttnWorkspace

TAIL = 16
ROW_BYTES = D + CB + 4          # sign/mantissa + codes + tag word of one token row
HEADROOM = TILE_MAX_ESC + 8     # one worst-case tile + the stream's read padding


def _round_up_tokens(n: int) -> int:
    return -(-n // T) * T


class _Store:
    """The K half or the V half of the cache.  Attribute names are those of kv_cache.py:99-111, which the attention launch reads by name."""
    def __init__(self, kind: str, H: int, cap: int, ovf_cap: int, base3: torch.Tensor, base4: torch.Tensor, dev):
        z = lambda *shape, dtype=torch.uint8: torch.zeros(*shape, dtype=dtype, device=dev)
        self.kind, self.H, self.cap = kind, H, cap
        self.sm, self.codes = z(H, cap * D), z(H, cap * CB)
        self.flags, self.tile_off = z(H, cap, dtype=torch.int32), z(H, cap // T, dtype=torch.int32)
        self.ovf_used = z(H, dtype=torch.int32)
        self.tail = z(H, TAIL, D, dtype=torch.bfloat16)
        self.base3, self.base4 = base3, base4
        self.enc = TileEncoder(kind, dev)
        self.ovf = None
        self._set_stream(z(H * ovf_cap), ovf_cap)

    def _set_stream(self, buf: torch.Tensor, ovf_cap: int):
        self.ovf, self.ovf_cap = buf, ovf_cap
        self.head_start = (torch.arange(self.H + 1, device=buf.device, dtype=torch.int32) * ovf_cap).contiguous()

    def grow(self, ovf_cap: int):
        """Move to an escape buffer with ovf_cap bytes per head, keeping every head's bytes at the start of its new window."""
        wider = torch.zeros(self.H * ovf_cap, dtype=torch.uint8, device=self.ovf.device)
        wider.view(self.H, ovf_cap)[:, :self.ovf_cap].copy_(self.ovf.view(self.H, self.ovf_cap))
        self._set_stream(wider, ovf_cap)

    def heads(self, h0: int, h1: int, S: int, n_kv: int) -> Page:
        """Page over the tiles of heads [h0, h1), S tokens each; shares the cache's memory."""
        own_rows = self.base3.shape[0] != n_kv
        b3, b4 = (self.base3[h0:h1], self.base4[h0:h1]) if own_rows else (self.base3, self.base4)
        return Page(self.sm[h0:h1], self.codes[h0:h1], self.flags[h0:h1], row_offsets(self.flags[h0:h1], S), self.ovf,
                    self.head_start[h0:h1 + 1], self.tile_off[h0:h1], b3, b4, h1 - h0, S, n_kv, self.kind)

    def load_prompt(self, h0: int, h1: int, xh: torch.Tensor, n_kv: int, calibrate: bool, grow) -> None:
        """xh: [n_kv, L, D], any strides.  The first L - L % 16 tokens are encoded into the heads' tile rows; the remaining L % 16 go to the tail raw."""
        L = xh.shape[1]; full = L // T * T
        if calibrate:
            c = Codec(n_kv, xh.device).calibrate(xh)
            self.base3[h0:h1] = c.base3; self.base4[h0:h1] = c.base4
        self.ovf_used[h0:h1] = 0
        if full:
            rows = (torch.arange(h0, h1, device=xh.device, dtype=torch.int32) % self.base3.shape[0]).contiguous()
            tile_bytes = self.enc.encode_tiles(xh, self.base3, self.base4, self.sm[h0:h1], self.codes[h0:h1], self.flags[h0:h1],
                                               full, self.cap, n_kv, bidx=rows)
            per_head = tile_bytes.sum(1)
            need = int(per_head.max()) + HEADROOM      # the next decode tile must fit before check_capacity runs again
            if need > self.ovf_cap: grow(need)
            self.tile_off[h0:h1, :full // T] = self.enc.compact(tile_bytes, self.head_start[h0:h1 + 1], self.ovf)
            self.ovf_used[h0:h1] = per_head.to(torch.int32)
        if L > full: self.tail[h0:h1, :L - full] = xh[:, full:]

    def kernel_args(self):
        return tuple(_lib.ptr(t) for t in (self.tail, self.base3, self.base4, self.sm, self.codes, self.flags, self.ovf, self.tile_off, self.ovf_used))


class CompressedKVCache:
    def __init__(self, n_slots: int, n_kv: int, capacity: int, bases: dict | None = None,
                 ovf_bytes_per_tile: int = 128, device="cuda"):
        """n_slots sequences of up to `capacity` tokens (rounded up to whole tiles), n_kv cache heads each.  bases: dict with uint8
        [n_kv, D] tables under 'k3', 'k4', 'v3', 'v4', or None to calibrate on every prompt.  ovf_bytes_per_tile sizes each head's
        escape window: that many bytes for every tile the head can hold (the window grows on demand until a graph is captured)."""
        _ext()      # fail here, not at the first decode step, if the native library is missing
        self.n_slots, self.n_kv = n_slots, n_kv
        self.cap = _round_up_tokens(capacity)
        self.H = n_slots * n_kv
        self.per_sequence_bases = bases is None
        def table(key):
            if bases is None: return torch.zeros(self.H, D, dtype=torch.uint8, device=device)
            return bases[key].to(device, torch.uint8).reshape(n_kv, D).contiguous()
        ovf_cap = (self.cap // T) * ovf_bytes_per_tile + 8
        self.k = _Store("k", self.H, self.cap, ovf_cap, table("k3"), table("k4"), device)
        self.v = _Store("v", self.H, self.cap, ovf_cap, table("v3"), table("v4"), device)
        self.S = torch.zeros(self.H, dtype=torch.int32, device=device)          # compressed tokens per head
        self.tail_len = torch.zeros(self.H, dtype=torch.int32, device=device)
        # set by the append kernel instead of writing out of bounds: bit 0 = a head was full, bit 1 = an escape stream was full
        self.overflow = torch.zeros(1, dtype=torch.int32, device=device)
        self.growable = True       # set False once graphs captured the buffer addresses
        self._partials = {}        # split partials + merge epochs per launch shape (stable addresses for graph replays)

    @staticmethod
    def bytes_per_slot(n_kv: int, capacity: int, ovf_bytes_per_tile: int = 128, per_sequence_bases: bool = True) -> int:
        """Device bytes one slot occupies, the quantity an engine divides its memory budget by (kv_cache.py:142-146).  Per head,
        for K and for V: token rows (sign/mantissa + codes + tag word), one offset per tile, the escape window and its 8 bytes of
        read padding, the escape counter (8 bytes with alignment), the staging tail, and with per-sequence bases the two base
        rows; per head once more: the S and tail_len counters."""
        cap = _round_up_tokens(capacity); tiles = cap // T
        head = cap * ROW_BYTES + tiles * 4 + (tiles * ovf_bytes_per_tile + 8) + 8 + TAIL * D * 2
        if per_sequence_bases: head += 2 * D
        return n_kv * (2 * head + 8)

    # ------------------------------------------------------------------ prefill
    def prefill(self, slot: int, k: torch.Tensor, v: torch.Tensor):
        """Put a whole prompt into `slot`, replacing what the slot held: k, v bf16 [L, n_kv, D] in the model's token-major layout."""
        L = k.shape[0]
        assert L <= self.cap, f"prompt has {L} tokens, a slot holds {self.cap}"
        h0, h1 = slot * self.n_kv, (slot + 1) * self.n_kv
        for st, x in ((self.k, k), (self.v, v)):
            st.load_prompt(h0, h1, x.contiguous().transpose(0, 1), self.n_kv, self.per_sequence_bases, self._grow)      # a view: no transposing copy
        self.S[h0:h1] = L // T * T
        self.tail_len[h0:h1] = L % T

    # ------------------------------------------------------------------ decode step
    def append(self, slots: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
        """Decode-step write: batch row b adds the token k[b], v[b] (bf16 [B, n_kv, D]) to slot slots[b] (int32 [B]; -1 leaves the row out).
        A single launch with no host synchronization."""
        k, v = k.contiguous(), v.contiguous()
        if k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16 or k.shape != v.shape or tuple(k.shape[1:]) != (self.n_kv, D):
            raise RuntimeError(f"append expects k, v bf16 [B, {self.n_kv}, {D}]")
        if slots.dtype != torch.int32 or slots.numel() != k.shape[0]:
            raise RuntimeError("append expects slots int32 [B]")
        p = _lib.ptr
        _lib.call("gaac_cache_append", p(slots), slots.numel(), self.n_kv, p(k), p(v), p(self.tail_len), p(self.S), self.cap, self.k.ovf_cap,
                  self.k.base3.shape[0], *self.k.kernel_args(), *self.v.kernel_args(), p(self.overflow), _lib.stream())

    def attention(self, q: torch.Tensor, slots: torch.Tensor, scale: float, max_len: int | None = None, nsplit: int | None = None):
        """Decode-step read: bf16 [B, n_q, D] queries, row b over everything slot slots[b] holds (tiles and tail); returns bf16 [B, n_q, D].
        max_len only picks the split count when nsplit is not given."""
        B, n_q, _ = q.shape
        if nsplit is None: nsplit = choose_nsplit(B, self.n_kv, max_len or self.cap)
        ws = self._partials.get((B, n_q, nsplit))
        if ws is None:
            ws = self._partials[(B, n_q, nsplit)] = AttnWorkspace(B * n_q, nsplit, q.dtype, q.device, with_out=False)
        out = attn_launch(self.k, self.v, q.reshape(B * n_q, D).contiguous(), slots, n_q, self.n_kv, self.S, self.cap, scale, nsplit,
                          self.k.tail, self.v.tail, self.tail_len, TAIL, ws=ws)
        return out.view(B, n_q, D)

    # ------------------------------------------------------------------ housekeeping
    def max_escape_bytes(self) -> torch.Tensor:
        return torch.maximum(self.k.ovf_used.max(), self.v.ovf_used.max())

    def check_capacity(self, used: int | None = None):
        """Host-side guard of the escape windows (kv_cache.py:198-203); the engine calls it every 16 decode steps at the latest.  In
        16 steps a head completes one tile at most, and a tile has at most TILE_MAX_ESC escape bytes, so a window that has that
        much room left after a check cannot fill up before the next one.  Grows the windows when the room is gone; raises if the
        append kernel already had to drop data or a fused attention launch gave up waiting for a partial.  used: max_escape_bytes() if the caller fetched it already."""
        for ws in self._partials.values(): ws.check()      # a fused attention launch that gave up a wait (rows NaN): re-arm with ws.reset()
        hit = int(self.overflow)
        if hit:
            raise RuntimeError("compressed KV cache lost data:" + (" a sequence grew past the slot's token capacity;" if hit & 1 else "") +
                               (" an escape window filled up between two check_capacity calls (call it every 16 decode steps)" if hit & 2 else ""))
        used = int(self.max_escape_bytes()) if used is None else used
        if used + HEADROOM > self.k.ovf_cap: self._grow(used + HEADROOM)

    def _grow(self, need: int):
        if not self.growable:
            raise RuntimeError(f"every head's escape window must grow from {self.k.ovf_cap} to {need} bytes, but a captured graph holds the "
                               "buffer's address: construct the cache with a larger ovf_bytes_per_tile, or pass bases calibrated on typical prompts")
        cap = max(2 * self.k.ovf_cap, need + 4096 + 7) // 8 * 8
        self.k.grow(cap); self.v.grow(cap)

    def decompress(self, slot: int) -> tuple[torch.Tensor, torch.Tensor]:
        """The K and V that `slot` holds, bf16 [L, n_kv, D] each, equal bit for bit to what was stored: tiles through the decoder kernel, then the tail rows."""
        h0, h1 = slot * self.n_kv, (slot + 1) * self.n_kv
        S, n_tail = int(self.S[h0]), int(self.tail_len[h0])
        def one(st):
            raw = st.tail[h0:h1, :n_tail]
            xh = torch.cat([Codec.decode(st.heads(h0, h1, S, self.n_kv)), raw], 1) if S else raw
            return xh.transpose(0, 1).contiguous()
        return one(self.k), one(self.v)

    def stats(self) -> dict:
        """Occupancy (same keys as kv_cache.py:228-234): bytes_used counts encoded rows, tile offsets, escape bytes and the BF16 tail rows of
        all slots; bf16_bytes is what the same tokens take uncompressed."""
        rows, raw_rows = int(self.S.sum()), int(self.tail_len.sum())
        escapes = int(self.k.ovf_used.sum()) + int(self.v.ovf_used.sum())
        used = 2 * (rows * ROW_BYTES + rows // T * 4 + raw_rows * D * 2) + escapes
        bf16 = 2 * (rows + raw_rows) * D * 2
        return dict(tokens=(rows + raw_rows) // max(1, self.n_kv), bytes_used=used, bf16_bytes=bf16, ratio=bf16 / max(1, used))
