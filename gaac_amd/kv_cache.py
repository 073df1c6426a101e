"""Compressed KV cache of one attention layer for serving on MI355X.

Drop-in for the cache of /root/reference/gaac/kv_cache.py:122-234 (same constructor, methods, attributes and tensor
shapes).  A sequence owns a slot of n_kv cache heads; a head stores compressed 16-token tiles (token stride `cap`), one
escape stream of `ovf_cap` bytes and a raw BF16 tail of 0..15 tokens.  A decode step is two launches on the current
stream, append (the step that fills a tail compresses the tile in place) and attention, without host synchronization,
so it can be captured in a HIP graph; batch rows find their slot through a device slot map and rows with slot -1 are
skipped (attention output exactly 0).  Bases are per model ([n_kv, D] tables) or per sequence, calibrated on the
prompt at prefill ([n_slots*n_kv, D] tables)."""
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
    """One kind ('k' | 'v') of the cache: the tensors the kernels read, named as in kv_cache.py:99-111."""
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
        """Re-home every head's escape bytes in a stream of ovf_cap bytes per head."""
        wider = torch.zeros(self.H * ovf_cap, dtype=torch.uint8, device=self.ovf.device)
        wider.view(self.H, ovf_cap)[:, :self.ovf_cap].copy_(self.ovf.view(self.H, self.ovf_cap))
        self._set_stream(wider, ovf_cap)

    def heads(self, h0: int, h1: int, S: int, n_kv: int) -> Page:
        """The compressed part of heads [h0, h1) as a Page view (no copies)."""
        own_rows = self.base3.shape[0] != n_kv
        b3, b4 = (self.base3[h0:h1], self.base4[h0:h1]) if own_rows else (self.base3, self.base4)
        return Page(self.sm[h0:h1], self.codes[h0:h1], self.flags[h0:h1], row_offsets(self.flags[h0:h1], S), self.ovf,
                    self.head_start[h0:h1 + 1], self.tile_off[h0:h1], b3, b4, h1 - h0, S, n_kv, self.kind)

    def load_prompt(self, h0: int, h1: int, xh: torch.Tensor, n_kv: int, calibrate: bool, grow) -> None:
        """xh: [n_kv, L, D] (any strides).  Full tiles are compressed into rows [0, L//16*16) of the heads, the rest becomes the tail."""
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
        """capacity: max tokens per sequence; bases: {'k3','k4','v3','v4'} uint8 [n_kv, D] (None = per-sequence calibration);
        ovf_bytes_per_tile: escape-stream reservation per 16-token tile."""
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
        """Resident bytes of one slot (kv_cache.py:142-146): per head and kind the tile rows, tile offsets, escape stream
        (+8 padding), two counters, the raw tail and, for per-sequence bases, two base rows; plus S and tail_len per head."""
        cap = _round_up_tokens(capacity); tiles = cap // T
        head = cap * ROW_BYTES + tiles * 4 + (tiles * ovf_bytes_per_tile + 8) + 8 + TAIL * D * 2
        if per_sequence_bases: head += 2 * D
        return n_kv * (2 * head + 8)

    # ------------------------------------------------------------------ prefill
    def prefill(self, slot: int, k: torch.Tensor, v: torch.Tensor):
        """Store a sequence's prompt K/V ([L, n_kv, D] bf16, token-major as produced by the model) in `slot` (a reused slot is reset)."""
        L = k.shape[0]
        assert L <= self.cap, f"sequence of {L} tokens exceeds the cache capacity {self.cap}"
        h0, h1 = slot * self.n_kv, (slot + 1) * self.n_kv
        for st, x in ((self.k, k), (self.v, v)):
            st.load_prompt(h0, h1, x.contiguous().transpose(0, 1), self.n_kv, self.per_sequence_bases, self._grow)      # a view: no transposing copy
        self.S[h0:h1] = L // T * T
        self.tail_len[h0:h1] = L % T

    # ------------------------------------------------------------------ decode step
    def append(self, slots: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
        """One new token per batch row: slots int32 [B] (-1 = skip), k/v [B, n_kv, D] bf16.  One launch, graph-safe."""
        k, v = k.contiguous(), v.contiguous()
        if k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16 or k.shape != v.shape or tuple(k.shape[1:]) != (self.n_kv, D):
            raise RuntimeError(f"append expects k, v bf16 [B, {self.n_kv}, {D}]")
        if slots.dtype != torch.int32 or slots.numel() != k.shape[0]:
            raise RuntimeError("append expects slots int32 [B]")
        p = _lib.ptr
        _lib.call("gaac_cache_append", p(slots), slots.numel(), self.n_kv, p(k), p(v), p(self.tail_len), p(self.S), self.cap, self.k.ovf_cap,
                  self.k.base3.shape[0], *self.k.kernel_args(), *self.v.kernel_args(), p(self.overflow), _lib.stream())

    def attention(self, q: torch.Tensor, slots: torch.Tensor, scale: float, max_len: int | None = None, nsplit: int | None = None):
        """q: [B, n_q, D] bf16 (row b attends over slot slots[b]) -> [B, n_q, D] bf16."""
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
        """Call at least once every 16 decode steps: a head finalizes at most one tile in 16 steps, so one worst-case tile of
        headroom per head keeps the escape streams overflow-proof between checks (kv_cache.py:198-203)."""
        hit = int(self.overflow)
        if hit:
            raise RuntimeError("compressed KV cache overflow:" + (" a head exceeded its token capacity;" if hit & 1 else "") +
                               (" an escape stream was full (check_capacity must run at least every 16 decode steps)" if hit & 2 else ""))
        used = int(self.max_escape_bytes()) if used is None else used
        if used + HEADROOM > self.k.ovf_cap: self._grow(used + HEADROOM)

    def _grow(self, need: int):
        if not self.growable:
            raise RuntimeError(f"escape stream needs {need} B per head but holds {self.k.ovf_cap} B and graphs are captured; "
                               "raise ovf_bytes_per_tile or calibrate the exponent bases on representative prompts")
        cap = max(2 * self.k.ovf_cap, need + 4096 + 7) // 8 * 8
        self.k.grow(cap); self.v.grow(cap)

    def decompress(self, slot: int) -> tuple[torch.Tensor, torch.Tensor]:
        """Bit-exact BF16 K/V of `slot` ([L, n_kv, D] each): decoded tiles followed by the raw tail."""
        h0, h1 = slot * self.n_kv, (slot + 1) * self.n_kv
        S, n_tail = int(self.S[h0]), int(self.tail_len[h0])
        def one(st):
            raw = st.tail[h0:h1, :n_tail]
            xh = torch.cat([Codec.decode(st.heads(h0, h1, S, self.n_kv)), raw], 1) if S else raw
            return xh.transpose(0, 1).contiguous()
        return one(self.k), one(self.v)

    def stats(self) -> dict:
        """Bytes in use (compressed tiles + escapes + metadata + raw tails) vs the BF16 bytes of the same tokens (kv_cache.py:228-234)."""
        rows, raw_rows = int(self.S.sum()), int(self.tail_len.sum())
        escapes = int(self.k.ovf_used.sum()) + int(self.v.ovf_used.sum())
        used = 2 * (rows * ROW_BYTES + rows // T * 4 + raw_rows * D * 2) + escapes
        bf16 = 2 * (rows + raw_rows) * D * 2
        return dict(tokens=(rows + raw_rows) // max(1, self.n_kv), bytes_used=used, bf16_bytes=bf16, ratio=bf16 / max(1, used))
