"""Paged slot pool on MI355X: per-layer state, store path and decode attention through a block table.

Mirrors the interfaces of /root/reference/gaac/vllm/store.py:177-227 (LayerState) and paged_kernel.py:288-301 (choose_nsplit,
paged_attention).  A block of 16 tokens (all kv heads, K and V) is 2*n_kv tile slots of TS = 2880 + ovf_slot bytes in a flat
uint8 pool; the mode table says per slot whether it is compressed in place (MT[p] == p) or lives as a raw BF16 tile in the side
pool (MT[p] == ~r): the block a sequence is still filling, or a finished tile whose escape bytes exceed the slot.  A sequence's
"tail" is simply its raw filling tile.  Everything is enqueued on the current stream without host synchronization."""
from __future__ import annotations
import numpy as np
import torch
from . import _lib
from .kernel import AttnWorkspace, shared_workspace

D = 128
BLOCK = 16
SM_OFF, CD_OFF, FL_OFF, OVF_OFF = 0, 2048, 2816, 2880   # byte layout of a tile slot; TS = OVF_OFF + ovf_slot


def choose_nsplit(B: int, n_kv: int, S: int, target_ctas: int = 2048, min_tok: int = 256, cap: int = 256) -> int:
    """Splits per (row, kv head) for the longest sequence S of the batch: sequences of a serving batch differ in length, so the
    launch is cut into several times more blocks than the 512 that are resident (they balance out as they are scheduled), at
    least min_tok tokens each.  (Any split count works; a split of more than 1024 tiles leaves the prefetch pipeline after its
    first 1024 and is slower from there on.)"""
    return max(min(max(1, target_ctas // (B * n_kv)), max(1, S // min_tok), cap), 1)


def build_store_entries(num_computed, query_len, block_table) -> np.ndarray:
    """Host side of the store path (the entry list of backend.py:207-226): request i has num_computed[i] tokens in the pool and
    brings query_len[i] new rows, laid out back to back in the step's K/V tensors.  Returns int32 [E, 4] = (block, first row in
    K/V, offset in the block, rows), one entry per touched (request, block)."""
    ent, row = [], 0
    for i, (c, n) in enumerate(zip(num_computed, query_len)):
        c, n = int(c), int(n)
        pos = c
        while pos < c + n:
            lb, off = divmod(pos, BLOCK)
            take = min(BLOCK - off, c + n - pos)
            ent.append((int(block_table[i][lb]), row + (pos - c), off, take))
            pos += take
        row += n
    return np.asarray(ent, dtype=np.int32).reshape(-1, 4)


class LayerState:
    """Per-layer device state outside the block pool: raw side pool, mode table, free stack, error counter and bases.  The block pool
    itself is the caller's allocation of num_blocks * 2 * n_kv slots of TS bytes (pool_bytes()); no kernel touches a byte outside
    the slots, so an engine's own block buffer of exactly that size can be handed over."""
    def __init__(self, num_blocks: int, n_kv: int, raw_tiles: int, bases: dict, ovf_slot: int = 128, device="cuda"):
        _lib.load()
        self.n_kv, self.ovf_slot, self.TS = n_kv, ovf_slot, OVF_OFF + ovf_slot
        assert ovf_slot >= 16 and self.TS % 16 == 0, "ovf_slot must be a positive multiple of 16"
        self.num_blocks = num_blocks
        i32 = dict(dtype=torch.int32, device=device)
        self.mt = torch.arange(num_blocks * 2 * n_kv, **i32)                 # every tile starts 'compressed at itself'
        self.raw = torch.zeros(raw_tiles, BLOCK, D, dtype=torch.bfloat16, device=device)
        self.stack = torch.arange(raw_tiles, **i32)
        self.top = torch.tensor([raw_tiles], **i32)
        self.err = torch.zeros(1, **i32)
        self.b3k, self.b4k, self.b3v, self.b4v = (bases[k].to(device).to(torch.uint8).reshape(n_kv, D).contiguous() for k in ("k3", "k4", "v3", "v4"))
        self._ws = {}
        self._pending_free = None      # (freeq, n): raw tiles a store queued and no launch has pushed back yet

    @staticmethod
    def pool_bytes(num_blocks: int, n_kv: int, ovf_slot: int = 128) -> int:
        """Bytes of the block pool: num_blocks * 2 * n_kv slots of 2880 + ovf_slot bytes, nothing more."""
        return num_blocks * 2 * n_kv * (OVF_OFF + ovf_slot)

    @property
    def bases(self):
        return (self.b3k, self.b4k, self.b3v, self.b4v)

    def _base_ptrs(self):
        return tuple(_lib.ptr(t) for t in self.bases)

    def _flush_free(self):
        if self._pending_free is not None:
            freeq, n = self._pending_free
            self._pending_free = None
            _lib.call("gaac_paged_free", _lib.ptr(freeq), n, _lib.ptr(self.stack), _lib.ptr(self.top), _lib.stream())

    def store(self, key: torch.Tensor, value: torch.Tensor, buf: torch.Tensor, ent: torch.Tensor, freeq: torch.Tensor | None = None,
              defer_free: bool = False):
        """key/value: [num_tokens, n_kv, D] bf16 (or int16 views); buf: uint8 flat block pool; ent: int32 [E,4] = (blk, tok0, off0, n);
        freeq: int32 [E*2*n_kv] scratch (allocated when omitted).  defer_free: the raw tiles this store gives back are pushed onto
        the free stack by the next attention() launch of this layer instead of a launch of their own (a decode step is then two
        launches); any other call that needs the stack first (another store, release_blocks, check) pushes them itself."""
        self._flush_free()
        E = ent.shape[0]
        if E == 0: return
        if key.stride(-1) != 1 or key.stride(1) != D or value.stride(-1) != 1 or value.stride(1) != D:
            raise RuntimeError("store expects K/V rows of n_kv*128 contiguous elements")
        n = E * 2 * self.n_kv
        if freeq is None: freeq = torch.empty(n, dtype=torch.int32, device=buf.device)
        p = _lib.ptr
        _lib.call("gaac_paged_store", p(key), p(value), key.stride(0), value.stride(0), p(ent), E, p(buf), self.TS, p(self.raw), p(self.mt),
                  p(self.stack), p(self.top), p(self.err), p(freeq), *self._base_ptrs(), self.n_kv, _lib.stream())
        self._pending_free = (freeq, n)
        if not defer_free: self._flush_free()

    def decode_blocks(self, buf: torch.Tensor, pairs: torch.Tensor, sk: torch.Tensor, sv: torch.Tensor):
        """pairs: int32 [P,3] (block, first scratch row, valid rows); sk/sv: flat K/V [rows, n_kv, D] bf16 (written)."""
        P = pairs.shape[0]
        if P == 0: return
        if sk.stride(0) != sv.stride(0) or sk.stride(0) < self.n_kv * D:
            raise RuntimeError("decode_blocks expects K/V scratch rows of at least n_kv*128 elements and equal strides")
        p = _lib.ptr
        _lib.call("gaac_paged_decode", p(buf), self.TS, p(self.raw), p(self.mt), p(pairs), P, p(sk), p(sv), sk.stride(0),
                  *self._base_ptrs(), self.n_kv, _lib.stream())

    def release_blocks(self, blocks: torch.Tensor):
        """blocks: int32 [F] block ids whose content is dead."""
        F = blocks.shape[0]
        if F == 0: return
        self._flush_free()
        p = _lib.ptr
        _lib.call("gaac_paged_release", p(blocks), F, p(self.mt), p(self.stack), p(self.top), self.n_kv, _lib.stream())

    def check(self):
        """Host poll (every 16 steps in the reference, backend.py:233-236): raises when the raw side pool ran dry."""
        self._flush_free()
        for ws in self._ws.values(): ws.check()      # a fused attention launch that gave up a wait: re-arm with ws.reset()
        failed = int(self.err)
        if failed:
            raise RuntimeError(f"raw side pool exhausted ({failed} failed allocations); raise raw_tiles or ovf_slot")

    def attention(self, q: torch.Tensor, buf: torch.Tensor, bt: torch.Tensor, seq_lens: torch.Tensor, nsplit: int, max_seq_len: int | None = None,
                  out: torch.Tensor | None = None) -> torch.Tensor:
        B, n_q, _ = q.shape
        if out is None: out = torch.empty(B, n_q * D, dtype=q.dtype, device=q.device)
        ws = self._ws.get((B, n_q, nsplit))
        if ws is None: ws = self._ws[(B, n_q, nsplit)] = AttnWorkspace(B * n_q, nsplit, q.dtype, q.device, with_out=False)
        free, self._pending_free = self._pending_free, None
        return paged_attention(q, out, buf, self.raw, self.mt, bt, seq_lens, self.bases, self.TS, n_q, self.n_kv, nsplit, max_seq_len, ws,
                               free=None if free is None else (free[0], free[1], self.stack, self.top))


def paged_attention(q, out, buf, raw, mt, bt, seq_lens, bases, TS, n_q, n_kv, nsplit, max_seq_len=None, ws=None, free=None):
    """q: [B, n_q, 128] bf16 contiguous; out: [B, n_q*128] bf16 (written); buf: uint8 flat block pool; raw: [tiles,16,128] bf16;
    mt: int32 [num_blocks*2*n_kv]; bt: int32 [B, max_blocks]; seq_lens: int32 [B]; bases: (b3k,b4k,b3v,b4v) uint8 [n_kv,128].
    max_seq_len: host-side bound of seq_lens (default: what the block table can address).  ws: the launch's
    AttnWorkspace (default: one cached per device, stream and launch shape, so repeated calls allocate nothing).  free: (freeq, n, stack,
    top) of a preceding store whose raw tiles this launch pushes back (LayerState.store(defer_free=True))."""
    B = q.shape[0]
    if q.shape[-1] != D: raise RuntimeError("head_dim must be 128")
    if max_seq_len is None: max_seq_len = bt.shape[1] * BLOCK
    if ws is None: ws = shared_workspace(B * n_q, nsplit, q.dtype, q.device)
    elif ws.rows != B * n_q or ws.nslot != nsplit: raise RuntimeError("attention workspace does not match the launch shape")
    p = _lib.ptr
    q = q.contiguous()
    _lib.call("gaac_paged_attn", p(buf), TS, p(raw), p(mt), p(bt), bt.stride(0), p(seq_lens), int(max_seq_len), p(q), B, n_q, n_kv,
              float(1.0 / (D ** 0.5)), nsplit, p(bases[0]), p(bases[1]), p(bases[2]), p(bases[3]), bases[0].shape[0],
              p(ws.pm), p(ws.pl), p(ws.pa), p(ws.epoch), p(out),
              *((p(free[0]), int(free[1]), p(free[2]), p(free[3])) if free is not None else (None, 0, None, None)), _lib.stream())
    return out
