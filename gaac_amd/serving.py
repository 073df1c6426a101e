"""The call site of the compressed cache in a serving engine, with the surface of the reference's bundled engine, and a decode loop
built on it.

  Context, get_context / set_context / reset_context     /root/reference/nanovllm/utils/context.py:5-31 (same fields, incl. kv_slots and
                                                         prefill_spans of the GAAC mode)
  Attention (forward, forward_gaac)                      /root/reference/nanovllm/layers/attention.py:43-96: prefill attends over the
                                                         prompt's own K/V and then compresses every span into its slot; decode appends
                                                         the new token and runs the fused attention over the compressed cache
  allocate_gaac_cache, gaac_stats                        /root/reference/nanovllm/engine/model_runner.py:130-153: slots sized from a byte
                                                         budget with CompressedKVCache.bytes_per_slot, one cache per attention layer
  DecodeRunner                                           model_runner.py:209-215, 249-253, 268-273, 295-318: decode inputs, the step
                                                         captured as a graph with padded rows at slot -1, the escape-capacity check
                                                         every 16 steps

The model is a Llama-architecture stack (RMSNorm, rotary embedding, GQA, SwiGLU) on plain torch ops with random weights.  Where the
reference calls flash-attn (prefill, and the uncompressed decode path) this module uses torch's scaled_dot_product_attention and the
library's own BF16 decode kernel; the KV backend of a layer is either CompressedKVCache (`Attention.gaac`) or an uncompressed BF16
cache (`Attention.bf16`), the baseline."""
from __future__ import annotations
from dataclasses import dataclass
import torch
import torch.nn.functional as F
from .kv_cache import CompressedKVCache
from .kernel import bf16_attention, choose_nsplit, AttnWorkspace

D = 128


@dataclass
class Context:
    """Per-step state the attention layers read (nanovllm/utils/context.py:5-17)."""
    is_prefill: bool = False
    cu_seqlens_q: torch.Tensor | None = None
    cu_seqlens_k: torch.Tensor | None = None
    max_seqlen_q: int = 0
    max_seqlen_k: int = 0
    slot_mapping: torch.Tensor | None = None
    context_lens: torch.Tensor | None = None
    block_tables: torch.Tensor | None = None
    kv_slots: torch.Tensor | None = None        # decode: int32 [bs] cache slot per batch row (-1 = padding)
    prefill_spans: list | None = None           # prefill: [(slot, start, end)] token ranges of the batch


_CONTEXT = Context()


def get_context() -> Context:
    return _CONTEXT


def set_context(is_prefill, cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q=0, max_seqlen_k=0, slot_mapping=None, context_lens=None,
                block_tables=None, kv_slots=None, prefill_spans=None):
    global _CONTEXT
    _CONTEXT = Context(is_prefill, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, slot_mapping, context_lens, block_tables, kv_slots, prefill_spans)


def reset_context():
    global _CONTEXT
    _CONTEXT = Context()


def _causal_varlen_attention(q, k, v, spans, scale):
    """Causal attention of every sequence over its own K/V (what flash_attn_varlen_func does at attention.py:87-90), one SDPA call per
    span.  q [N, n_heads, D], k / v [N, n_kv, D]; spans: [(start, end)]."""
    o = torch.empty_like(q)
    G = q.shape[1] // k.shape[1]
    for start, end in spans:
        o[start:end] = F.scaled_dot_product_attention(q[start:end].transpose(0, 1)[None], k[start:end].transpose(0, 1)[None], v[start:end].transpose(0, 1)[None],
                                                      is_causal=True, scale=scale, enable_gqa=G > 1)[0].transpose(0, 1)
    return o


class Attention(torch.nn.Module):
    """The attention layer of the engine (attention.py:43-96).  `gaac`: the layer's CompressedKVCache; `bf16`: an uncompressed cache
    (the baseline); `observer`: callable(k, v) on every prefill step (exponent-base calibration).  `nsplit`: split count of the decode
    launch (None: chosen per call from context.max_seqlen_k, fixed by the runner when the step is captured as a graph)."""
    def __init__(self, num_heads, head_dim, scale, num_kv_heads):
        super().__init__()
        assert head_dim == D, "head_dim must be 128"
        self.num_heads, self.head_dim, self.scale, self.num_kv_heads = num_heads, head_dim, scale, num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])
        self.gaac = None
        self.bf16 = None
        self.observer = None
        self.nsplit = None

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
        context = get_context()
        if self.observer is not None and context.is_prefill:
            self.observer(k, v)
        if self.gaac is not None:
            return self.forward_gaac(q, k, v, context)
        if self.bf16 is None:
            raise RuntimeError("Attention: no KV cache attached (set .gaac to a CompressedKVCache or .bf16 to an uncompressed cache)")
        if context.is_prefill:
            o = _causal_varlen_attention(q, k, v, [(s, e) for _slot, s, e in context.prefill_spans or ()], self.scale)
            for slot, start, end in context.prefill_spans or ():
                self.bf16.prefill(slot, k[start:end], v[start:end])
            return o
        self.bf16.append(context.context_lens.to(torch.int64), k, v)
        return self.bf16.attention(q, context.context_lens + 1, self.scale, self.nsplit or choose_nsplit(q.shape[0], self.num_kv_heads, context.max_seqlen_k))

    def forward_gaac(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, context: Context):
        if context.is_prefill:
            # the whole prompt is in this step: attend over its own K/V, then compress it into the sequence's slot
            assert context.block_tables is None, "GAAC mode: chunked prefill / prefix caching are not supported"
            o = _causal_varlen_attention(q, k, v, [(s, e) for _slot, s, e in context.prefill_spans or ()], self.scale)
            for slot, start, end in context.prefill_spans or ():
                self.gaac.prefill(slot, k[start:end], v[start:end])
            return o
        # decode: append the new token (compressing a tile when the tail fills), then fused attention over the compressed cache
        self.gaac.append(context.kv_slots, k, v)
        return self.gaac.attention(q, context.kv_slots, self.scale, max_len=context.max_seqlen_k, nsplit=self.nsplit)


def allocate_gaac_cache(layers, budget: int, num_kv_heads: int, max_model_len: int, max_num_seqs: int, gaac_bases=None,
                        ovf_bytes_per_tile: int = 128, device="cuda"):
    """One compressed cache per attention layer with a fixed slot (max_model_len tokens) per running sequence, as many slots as
    `budget` bytes hold (model_runner.py:130-148).  layers: the Attention modules; gaac_bases: {layer: {k3, k4, v3, v4}} or None
    (per-sequence calibration).  Returns (num_slots, caches) and attaches each cache as `layer.gaac`."""
    layers = list(layers)
    per_slot = len(layers) * CompressedKVCache.bytes_per_slot(num_kv_heads, max_model_len, ovf_bytes_per_tile, per_sequence_bases=gaac_bases is None)
    num_slots = min(max_num_seqs, budget // per_slot)
    assert num_slots > 0, f"GAAC cache: {per_slot / 2**30:.2f} GiB per sequence does not fit in {budget / 2**30:.2f} GiB"
    caches = []
    for i, layer in enumerate(layers):
        layer.gaac = CompressedKVCache(num_slots, num_kv_heads, max_model_len, gaac_bases[i] if gaac_bases is not None else None,
                                       ovf_bytes_per_tile, device=device)
        caches.append(layer.gaac)
    return num_slots, caches


def gaac_stats(caches, num_kv_slots: int) -> dict:
    """model_runner.py:150-153."""
    s = [c.stats() for c in caches]
    used, bf16 = sum(x["bytes_used"] for x in s), sum(x["bf16_bytes"] for x in s)
    return dict(num_kv_slots=num_kv_slots, bytes_used=used, bf16_bytes=bf16, ratio=bf16 / max(1, used))


@dataclass
class ModelConfig:
    hidden: int = 4096
    n_layers: int = 32
    n_heads: int = 32
    n_kv_heads: int = 8
    ffn: int = 14336
    vocab: int = 128256
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    max_len: int = 32768 + 256


class Weights:
    """Random-init BF16 weights of the stack (no checkpoint is read)."""
    def __init__(self, cfg: ModelConfig, device="cuda", seed: int = 0):
        g = torch.Generator(device=device).manual_seed(seed)
        w = lambda *shape, std=0.02: (torch.randn(*shape, generator=g, device=device, dtype=torch.float32) * std).to(torch.bfloat16)
        self.cfg = cfg
        self.embed = w(cfg.vocab, cfg.hidden)
        self.lm_head = w(cfg.vocab, cfg.hidden)
        self.final_norm = torch.ones(cfg.hidden, dtype=torch.bfloat16, device=device)
        qkv_out = (cfg.n_heads + 2 * cfg.n_kv_heads) * D
        self.layers = [dict(norm1=torch.ones(cfg.hidden, dtype=torch.bfloat16, device=device), qkv=w(qkv_out, cfg.hidden),
                            o=w(cfg.hidden, cfg.n_heads * D), norm2=torch.ones(cfg.hidden, dtype=torch.bfloat16, device=device),
                            gate_up=w(2 * cfg.ffn, cfg.hidden), down=w(cfg.hidden, cfg.ffn)) for _ in range(cfg.n_layers)]
        half = torch.arange(0, D, 2, device=device, dtype=torch.float32) / D
        ang = torch.arange(cfg.max_len, device=device, dtype=torch.float32)[:, None] * (cfg.rope_theta ** -half)[None, :]
        self.cos, self.sin = ang.cos(), ang.sin()          # [max_len, 64]

    def nbytes(self) -> int:
        n = self.embed.numel() + self.lm_head.numel() + self.final_norm.numel()
        return 2 * (n + sum(t.numel() for l in self.layers for t in l.values()))


def _rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x: [N, heads, D]; cos/sin: [N, D/2] (rotate-half convention)."""
    x1, x2 = x[..., :D // 2].float(), x[..., D // 2:].float()
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1).to(x.dtype)


class _Bf16Cache:
    """Uncompressed cache of one layer: K/V [n_slots*n_kv, cap, D] bf16; batch row b of a decode step uses slot b."""
    def __init__(self, n_slots: int, n_kv: int, cap: int, device):
        self.n_kv, self.cap = n_kv, cap
        self.k = torch.zeros(n_slots * n_kv, cap, D, dtype=torch.bfloat16, device=device)
        self.v = torch.zeros_like(self.k)
        self._ws = {}

    def prefill(self, slot: int, k: torch.Tensor, v: torch.Tensor):
        L = k.shape[0]; h0 = slot * self.n_kv
        self.k[h0:h0 + self.n_kv, :L] = k.transpose(0, 1); self.v[h0:h0 + self.n_kv, :L] = v.transpose(0, 1)

    def append(self, pos: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
        """pos int64 [B]: position of the new token of slot b; k/v [B, n_kv, D].  Index writes only: graph-safe."""
        B = k.shape[0]
        heads = torch.arange(B * self.n_kv, device=k.device)
        rows = pos.repeat_interleave(self.n_kv)
        self.k[heads, rows] = k.reshape(B * self.n_kv, D); self.v[heads, rows] = v.reshape(B * self.n_kv, D)

    def attention(self, q: torch.Tensor, seq_lens: torch.Tensor, scale: float, nsplit: int):
        B, n_q, _ = q.shape
        ws = self._ws.get((B, n_q, nsplit))
        if ws is None: ws = self._ws[(B, n_q, nsplit)] = AttnWorkspace(B * n_q, nsplit, q.dtype, q.device, with_out=False)
        H = B * self.n_kv
        return bf16_attention(q, self.k[:H], self.v[:H], scale, nsplit, ws, seq_lens=seq_lens, out=torch.empty(B * n_q, D, dtype=q.dtype, device=q.device))

    def nbytes_used(self, tokens: int) -> int:
        return tokens * self.n_kv * 2 * D * 2


class DecodeRunner:
    """Prefill sequences into slots, then run greedy decode steps for slots 0..B-1, optionally as one captured HIP graph."""
    def __init__(self, weights: Weights, n_slots: int, kv: str = "gaac", bases: dict | None = None, ovf_bytes_per_tile: int = 128,
                 kv_budget: int | None = None):
        """kv_budget: bytes for the compressed caches (None: exactly n_slots slots); with a budget the slot count is what fits, at most n_slots."""
        assert kv in ("gaac", "bf16")
        self.w, self.cfg, self.kv = weights, weights.cfg, kv
        cfg, dev = self.cfg, weights.embed.device
        self.scale = D ** -0.5
        self.attn = [Attention(cfg.n_heads, D, self.scale, cfg.n_kv_heads) for _ in range(cfg.n_layers)]
        if kv == "gaac":
            if kv_budget is None:
                kv_budget = n_slots * cfg.n_layers * CompressedKVCache.bytes_per_slot(cfg.n_kv_heads, cfg.max_len, ovf_bytes_per_tile, per_sequence_bases=bases is None)
            n_slots, self.caches = allocate_gaac_cache(self.attn, kv_budget, cfg.n_kv_heads, cfg.max_len, n_slots, bases, ovf_bytes_per_tile, dev)
        else:
            self.caches = [_Bf16Cache(n_slots, cfg.n_kv_heads, cfg.max_len, dev) for _ in range(cfg.n_layers)]
            for a, c in zip(self.attn, self.caches): a.bf16 = c
        self.n_slots = n_slots
        self.lens = torch.zeros(n_slots, dtype=torch.int32, device=dev)      # tokens held per slot
        self.steps = 0
        self.graph = None

    # ---------------------------------------------------------------- layers
    def _qkv(self, layer, x, pos):
        cfg = self.cfg
        h = F.rms_norm(x, (cfg.hidden,), layer["norm1"], cfg.rms_eps)
        qkv = F.linear(h, layer["qkv"]).view(x.shape[0], cfg.n_heads + 2 * cfg.n_kv_heads, D)
        q, k, v = qkv[:, :cfg.n_heads], qkv[:, cfg.n_heads:cfg.n_heads + cfg.n_kv_heads], qkv[:, cfg.n_heads + cfg.n_kv_heads:]
        cos, sin = self.w.cos.index_select(0, pos), self.w.sin.index_select(0, pos)
        return _rope(q, cos, sin), _rope(k, cos, sin).contiguous(), v.contiguous()

    def _mlp(self, layer, x):
        cfg = self.cfg
        h = F.rms_norm(x, (cfg.hidden,), layer["norm2"], cfg.rms_eps)
        gu = F.linear(h, layer["gate_up"])
        return x + F.linear(F.silu(gu[:, :cfg.ffn]) * gu[:, cfg.ffn:], layer["down"])

    # ---------------------------------------------------------------- prefill
    @torch.no_grad()
    def prefill(self, slot: int, tokens: torch.Tensor) -> torch.Tensor:
        """tokens int64 [L] on the device: causal attention over the prompt's own K/V per layer, then the K/V go into `slot`.
        Returns the logits of the last position [vocab] (fp32)."""
        cfg, L = self.cfg, tokens.shape[0]
        pos = torch.arange(L, device=tokens.device)
        x = self.w.embed.index_select(0, tokens)
        cu = torch.tensor([0, L], dtype=torch.int32, device=tokens.device)
        set_context(True, cu, cu, L, L, prefill_spans=[(slot, 0, L)])
        for layer, attn in zip(self.w.layers, self.attn):
            q, k, v = self._qkv(layer, x, pos)
            o = attn(q, k, v)
            x = self._mlp(layer, x + F.linear(o.reshape(L, cfg.n_heads * D), layer["o"]))
        reset_context()
        self.lens[slot] = L
        x = F.rms_norm(x[-1:], (cfg.hidden,), self.w.final_norm, cfg.rms_eps)
        return F.linear(x, self.w.lm_head)[0].float()

    # ---------------------------------------------------------------- decode
    def _step(self, tokens: torch.Tensor, slots: torch.Tensor, lens: torch.Tensor, nsplit: int) -> torch.Tensor:
        """One token per batch row (row b = slot b, slots[b] = -1 for a padded row).  lens: tokens already held (int32 [B], advanced
        here).  Returns logits [B, vocab] bf16."""
        cfg = self.cfg
        pos = lens.to(torch.int64)
        x = self.w.embed.index_select(0, tokens)
        # decode inputs of the step (model_runner.py:209-215): the slot map of the batch rows; lengths stay on the device
        set_context(False, max_seqlen_k=cfg.max_len, context_lens=lens, kv_slots=slots)
        for layer, attn in zip(self.w.layers, self.attn):
            attn.nsplit = nsplit
            q, k, v = self._qkv(layer, x, pos)
            o = attn(q, k, v)
            x = self._mlp(layer, x + F.linear(o.reshape(x.shape[0], cfg.n_heads * D), layer["o"]))
        reset_context()
        lens += (slots >= 0).to(lens.dtype)
        x = F.rms_norm(x, (cfg.hidden,), self.w.final_norm, cfg.rms_eps)
        return F.linear(x, self.w.lm_head)

    @torch.no_grad()
    def start_decode(self, first_tokens: torch.Tensor, use_graph: bool = True, nsplit: int | None = None):
        """first_tokens int64 [B]: the token each of slots 0..B-1 decodes next.  With use_graph the step (all layers, cache appends,
        attention, greedy sampling, feeding the token back) is captured once and replayed."""
        B, dev = first_tokens.shape[0], first_tokens.device
        self.B = B
        self.tok = first_tokens.clone()
        self.slots = torch.arange(B, dtype=torch.int32, device=dev)
        self.dlens = self.lens[:B].clone()
        self.nsplit = nsplit or choose_nsplit(B, self.cfg.n_kv_heads, self.cfg.max_len)
        self.logits = None
        self.graph = None
        if not use_graph: return
        side = torch.cuda.Stream(); side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):      # warm up with every row padded: nothing is appended, lengths do not move
            self.slots.fill_(-1)
            keep = self.dlens.clone()
            self._one()
            self.dlens.copy_(keep); self.tok.copy_(first_tokens)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                self._one()
            self.dlens.copy_(keep); self.tok.copy_(first_tokens)
        torch.cuda.current_stream().wait_stream(side)
        self.slots.copy_(torch.arange(B, dtype=torch.int32, device=dev))
        for c in self.caches:
            if self.kv == "gaac": c.growable = False
        self.graph = g

    def _one(self):
        self.logits = self._step(self.tok, self.slots, self.dlens, self.nsplit)
        self.tok.copy_(self.logits.argmax(-1))

    @torch.no_grad()
    def decode(self, n_steps: int, forced: torch.Tensor | None = None, keep_logits: bool = False):
        """Runs n_steps greedy steps; returns the generated tokens [n_steps, B] (device).  forced int64 [n_steps, B]: teacher forcing: the
        token every row consumes at step i+1 is forced[i] instead of the one it generated (the returned tokens are still the model's
        own choices).  keep_logits: also returns the logits of every step [n_steps, B, vocab] (fp32)."""
        out, logits = [], []
        for i in range(n_steps):
            if self.graph is not None: self.graph.replay()
            else: self._one()
            out.append(self.tok.clone())
            if keep_logits: logits.append(self.logits.float().clone())
            if forced is not None: self.tok.copy_(forced[i])
            self.steps += 1
            if self.kv == "gaac" and self.steps % 16 == 0:      # every 16 steps a head finalizes at most one tile (model_runner.py:268-273)
                used = torch.stack([c.max_escape_bytes() for c in self.caches]).tolist()
                for c, u in zip(self.caches, used): c.check_capacity(u)
        self.lens[:self.B] = self.dlens
        return (torch.stack(out), torch.stack(logits)) if keep_logits else torch.stack(out)

    # ---------------------------------------------------------------- accounting
    def kv_stats(self) -> dict:
        """Bytes of KV in use (and reserved) vs the BF16 bytes of the same tokens, summed over layers (model_runner.py:150-153)."""
        cfg = self.cfg
        tokens = int(self.lens.sum())
        bf16 = tokens * cfg.n_kv_heads * 2 * D * 2 * cfg.n_layers
        if self.kv == "gaac":
            s = [c.stats() for c in self.caches]
            used = sum(x["bytes_used"] for x in s)
            reserved = cfg.n_layers * self.n_slots * CompressedKVCache.bytes_per_slot(cfg.n_kv_heads, cfg.max_len, per_sequence_bases=self.caches[0].per_sequence_bases)
        else:
            used = bf16
            reserved = cfg.n_layers * self.n_slots * cfg.n_kv_heads * cfg.max_len * 2 * D * 2
        return dict(tokens=tokens, bytes_used=used, bf16_bytes=bf16, ratio=bf16 / max(1, used), bytes_reserved=reserved)
