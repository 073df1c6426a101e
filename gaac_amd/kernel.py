"""Fused decode attention over the compressed KV on MI355X.  Public surface of /root/reference/gaac/kernel.py:332-359.

attention() launches the split-K kernel (one block per (batch row, kv head, split), MFMA score and output products on
K/V decoded in registers, optional raw-BF16 tail as one more block row; the last block of a kv head to finish merges
the partials) on the current stream, with no host synchronization.  Cache heads are addressed through a slot map exactly as in the reference: batch row b
reads cache head SLOT[b]*n_kv + kvh, SLOT[b] < 0 = padded row (output 0)."""
from __future__ import annotations
import torch
from . import _lib

D = 128
GMAX = 16
MAX_SPLITS = 1024


class _Ext:
    """What the reference's `_ext()` returns (/root/reference/gaac/kernel.py:332-337): an object whose
    `gaac_attn_launch(<16 store tensors>, q, slot, n_q, n_kv, SL, S_pad, scale, nsplit, kt, vt, TL, TCAP) -> Tensor` has the tensor
    signature and behaviour of the reference's pybind entry (kernel.py:296-326): it checks the GQA group and the head dim, allocates the
    output ([B*n_q, 128], dtype of q), takes the raw tail when `kt.numel() > 0`, launches on the current stream without synchronizing
    and returns the output.  The calls of /root/reference/gaac/kernel.py:355 and kv_cache.py:188 work on it unchanged.
    `lib` is the loaded C library (ctypes.CDLL) for callers that want the raw entry points."""
    def __init__(self, lib):
        self.lib = lib

    def gaac_attn_launch(self, smk, ck, fk, tok, ovk, ohsk, b3k, b4k, smv, cv, fv, tov, ovv, ohsv, b3v, b4v,
                         q, slot, n_q, n_kv, SL, S_pad, scale, nsplit, kt, vt, TL, TCAP):
        G = n_q // max(1, n_kv)
        if not (1 <= G <= GMAX and G * n_kv == n_q):
            raise RuntimeError(f"GQA group size must be 1..{GMAX}")
        if q.shape[-1] != D:
            raise RuntimeError("head_dim must be 128")
        B = slot.shape[0]
        has_tail = kt.numel() > 0
        out = torch.empty(B * n_q, D, dtype=q.dtype, device=q.device)
        ws = shared_workspace(B * n_q, nsplit, q.dtype, q.device)
        p = _lib.ptr
        _lib.call("gaac_attn_fused", p(smk), p(ck), p(fk), p(tok), p(ovk), p(ohsk), p(b3k), p(b4k),
                  p(smv), p(cv), p(fv), p(tov), p(ovv), p(ohsv), p(b3v), p(b4v),
                  p(q), p(slot), B, n_q, n_kv, p(SL), int(S_pad), float(scale), int(nsplit), b3k.shape[0],
                  p(kt) if has_tail else None, p(vt) if has_tail else None, p(TL) if has_tail else None, int(TCAP) if has_tail else 0,
                  -1, p(ws.pm), p(ws.pl), p(ws.pa), p(ws.epoch), p(out), _lib.stream())
        return out


_ext_obj = None


def _ext():
    """The native extension in the shape of the reference's (raises if the library is not built)."""
    global _ext_obj
    if _ext_obj is None: _ext_obj = _Ext(_lib.load())
    return _ext_obj


def choose_nsplit(B: int, n_kv: int, S: int, target_ctas: int = 256, min_tok: int = 256, cap: int = 256) -> int:
    """Splits per (row, kv head): one eight-wave block per CU of the 256-CU MI355X (the reference targets 96 CTAs for a 48-SM
    part, kernel.py:340-342), at least min_tok tokens per split.  Launches of up to 256 blocks use eight-wave blocks, larger
    ones four-wave blocks (two per CU)."""
    return min(max(1, target_ctas // (B * n_kv)), max(1, S // min_tok), cap)


class AttnWorkspace:
    """Output + split partials of one launch shape (rows = B*n_q).  The one-kernel launch stores every partial value as a 64-bit
    record (fp32 bits | launch epoch << 32): pm, pl [rows*NSLOT], pa [rows*NSLOT*D] int64.  epoch: [0] the epoch of the last merged
    one-kernel launch on this workspace, [1] failure bits that a launch sets instead of hanging (bit 0: a merging block gave up
    waiting for a partial and wrote its rows as NaN; bit 1: the epoch could not be advanced), [2 + i] the arrival mark of block i of
    the launch (rows*NSLOT words: a launch has B*n_kv*NSLOT <= rows*NSLOT blocks).  The two-kernel launch
    (phase "split" / "combine" / "both") keeps plain fp32 partials in buffers of its own, made on first use, so that its values can
    never be taken for records."""
    def __init__(self, rows: int, nslot: int, dtype, dev, with_out: bool = True):
        self.rows, self.nslot, self.dev = rows, nslot, dev
        self.out = torch.empty(rows, D, dtype=dtype, device=dev) if with_out else None      # None: a fresh output per launch
        self.pm = torch.zeros(rows * nslot, dtype=torch.int64, device=dev)
        self.pl = torch.zeros(rows * nslot, dtype=torch.int64, device=dev)
        self.pa = torch.zeros(rows * nslot * D, dtype=torch.int64, device=dev)
        self.epoch = torch.zeros(2 + rows * nslot, dtype=torch.int32, device=dev)
        self._f32 = None

    def f32_partials(self):
        """fp32 pm, pl, pa of the two-kernel launch (allocated on first use)."""
        if self._f32 is None:
            n = self.rows * self.nslot
            self._f32 = tuple(torch.empty(k, dtype=torch.float32, device=self.dev) for k in (n, n, n * D))
        return self._f32

    def failure_bits(self) -> int:
        """Host read of the failure word (synchronizes with the device)."""
        return int(self.epoch[1])

    def check(self):
        """Raises if a one-kernel launch on this workspace gave up a wait since the last reset() (its output rows are NaN, or the
        epoch stands still); poll it where the engine polls its other device-side error words."""
        bits = self.failure_bits()
        if bits:
            raise RuntimeError("fused decode attention gave up waiting for" + (" a split's partial (rows written as NaN)" if bits & 1 else "") +
                               (" the other blocks of the launch (epoch not advanced)" if bits & 2 else "") +
                               "; the workspace may hold records of a wrong epoch: re-arm with reset()")

    def reset(self):
        """Re-arm after a failed launch: the epochs, the failure bits and the records start from zero again."""
        for t in (self.pm, self.pl, self.pa, self.epoch): t.zero_()


_SHARED_WS_MAX = 8            # launch shapes whose workspace is kept per process; the least recently used one goes first
_shared_ws: dict = {}


def shared_workspace(rows: int, nslot: int, dtype, dev) -> AttnWorkspace:
    """The workspace that callers who pass none share: one per (device, launch shape, stream), zeroed once when it is made (a fresh
    buffer per call would have to be cleared per call: recycled memory may hold records whose epoch matches a new counter), at most
    _SHARED_WS_MAX of them (least recently used first out).  It has no output buffer of its own, so every launch returns a fresh
    tensor.  A workspace is never made while the stream is capturing (its memory and its zeroing would end up inside the graph):
    callers that capture pass their own, as CompressedKVCache and LayerState do."""
    dev = torch.device(dev)
    key = (dev.type, dev.index if dev.index is not None else torch.cuda.current_device(), rows, nslot, dtype, torch.cuda.current_stream(dev).cuda_stream)
    ws = _shared_ws.pop(key, None)
    if ws is None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("no attention workspace for this launch shape yet and the stream is capturing: run the launch once before "
                               "the capture, or pass a workspace (AttnWorkspace) of your own")
        ws = AttnWorkspace(rows, nslot, dtype, dev, with_out=False)
        while len(_shared_ws) >= _SHARED_WS_MAX: _shared_ws.pop(next(iter(_shared_ws)))
    _shared_ws[key] = ws      # most recently used last
    return ws


def _store_args(st):
    p = _lib.ptr
    hs = st.head_start if hasattr(st, "head_start") else st.ovf_head_start
    return (p(st.sm), p(st.codes), p(st.flags), p(st.tile_off), p(st.ovf), p(hs), p(st.base3), p(st.base4))


def attn_launch(K, V, q2d, slots, n_q, n_kv, SL, S_pad, scale, nsplit, kt=None, vt=None, TL=None, TCAP=0, ws=None, phase="fused", S_all=-1):
    """K, V: objects with sm, codes, flags, tile_off, ovf, head_start|ovf_head_start, base3, base4 (a Page or a cache store).
    q2d: [B*n_q, D] bf16 contiguous.  Returns [B*n_q, D] bf16.  phase: "fused" (one kernel, one block of each
    kv head merges) | "both" (split kernel then merge kernel) | "split" | "combine" (the halves of "both").
    S_all >= 0: every addressed head holds exactly S_all compressed tokens (SL is not read by the one-kernel launch)."""
    G = n_q // max(1, n_kv)
    if not (1 <= G <= GMAX and G * n_kv == n_q):
        raise RuntimeError(f"GQA group size must be 1..{GMAX}")
    if q2d.shape[-1] != D:
        raise RuntimeError("head_dim must be 128")
    B = slots.shape[0] if slots is not None else q2d.shape[0] // n_q      # slots=None: row b attends over cache heads b*n_kv ..
    has_tail = kt is not None and kt.numel() > 0
    nslot = nsplit        # the raw tail is folded into the last split's partial
    if ws is None:
        ws = shared_workspace(B * n_q, nslot, q2d.dtype, q2d.device)
    elif ws.rows != B * n_q or ws.nslot != nslot:
        raise RuntimeError("attention workspace does not match the launch shape")
    p = _lib.ptr
    out = ws.out if ws.out is not None else torch.empty(B * n_q, D, dtype=q2d.dtype, device=q2d.device)
    if phase == "combine":
        pm, pl, pa = ws.f32_partials()
        _lib.call("gaac_attn_combine", p(pm), p(pl), p(pa), p(out), B * n_q, nslot, _lib.stream())
        return out
    args = (*_store_args(K), *_store_args(V), p(q2d), p(slots), B, n_q, n_kv, p(SL), S_pad, float(scale), nsplit, K.base3.shape[0],
            p(kt) if has_tail else None, p(vt) if has_tail else None, p(TL) if has_tail else None, TCAP if has_tail else 0)
    if phase == "fused":
        _lib.call("gaac_attn_fused", *args, int(S_all), p(ws.pm), p(ws.pl), p(ws.pa), p(ws.epoch), p(out), _lib.stream())
        return out
    args = (*args, *(p(t) for t in ws.f32_partials()))
    if phase == "split":
        _lib.call("gaac_attn_split", *args, _lib.stream())
    else:
        _lib.call("gaac_attn_launch", *args, p(out), _lib.stream())
    return out


def attention(q, kp, vp, scale=None, nsplit=None, phase="fused"):
    """Decode attention over two Pages (kinds 'k' / 'v', H = B*n_kv heads of equal length).
    q: [B, n_q, D] bf16 (one query token per sequence) -> [B, n_q, D] bf16."""
    B, n_q, Dq = q.shape
    n_kv = kp.H // B
    dev = q.device
    if nsplit is None: nsplit = choose_nsplit(B, n_kv, kp.S)
    SL = torch.full((kp.H,), kp.S, dtype=torch.int32, device=dev)
    out = attn_launch(kp, vp, q.reshape(B * n_q, Dq).contiguous(), None, n_q, n_kv, SL, kp.sm.shape[1] // D,
                      scale if scale is not None else Dq ** -0.5, nsplit, phase=phase, S_all=kp.S)
    return out.view(B, n_q, Dq)


def bf16_attention(q, k, v, scale=None, nsplit=None, ws=None, seq_lens=None, out=None):
    """Baseline: decode attention over UNCOMPRESSED K/V (k, v: [B*n_kv, S, D] bf16, rows contiguous; q: [B, n_q, D]) with the kernel
    structure of the compressed path minus the decoder.  seq_lens: optional int32 [B] device tensor of valid tokens per batch row
    (<= S).  Returns [B, n_q, D] bf16."""
    B, n_q, Dq = q.shape
    H, S, _ = k.shape
    n_kv = H // B
    if k.stride(1) != D or v.stride(1) != D or k.stride(0) != v.stride(0): raise RuntimeError("bf16_attention expects token rows of 128 contiguous elements")
    if nsplit is None: nsplit = choose_nsplit(B, n_kv, S)
    if ws is None: ws = shared_workspace(B * n_q, nsplit, q.dtype, q.device)
    elif ws.rows != B * n_q or ws.nslot != nsplit: raise RuntimeError("attention workspace does not match the launch shape")
    if out is None: out = ws.out if ws.out is not None else torch.empty(B * n_q, D, dtype=q.dtype, device=q.device)
    p = _lib.ptr
    _lib.call("gaac_bf16_attn", p(k), p(v), S, p(seq_lens), k.stride(0) // D, p(q.contiguous()), B, n_q, n_kv,
              float(scale if scale is not None else Dq ** -0.5), nsplit, p(ws.pm), p(ws.pl), p(ws.pa), p(ws.epoch), p(out), _lib.stream())
    return out.view(B, n_q, Dq)
