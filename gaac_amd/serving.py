"""A decoder-only transformer decode loop over the compressed KV cache: the call site of the cache in a serving engine.

Counterpart of the GAAC branch of the reference's engine: the attention layer (/root/reference/nanovllm/layers/attention.py:83-96:
prefill attends over the prompt's own K/V and then compresses it into the sequence's slot; decode appends the new token and runs
the fused attention over the compressed cache), and the runner's cache handling (/root/reference/nanovllm/engine/model_runner.py:
130-153 allocation per layer, 268-273 escape-capacity check every 16 steps, 295-318 decode step captured as a graph with padded rows
at slot -1, gaac_stats).  The model is a Llama-architecture stack (RMSNorm, rotary embedding, GQA, SwiGLU) on plain torch ops; the
KV backend is either CompressedKVCache ("gaac") or an uncompressed BF16 cache read by the baseline kernel ("bf16")."""
from __future__ import annotations
from dataclasses import dataclass
import torch
import torch.nn.functional as F
from .kv_cache import CompressedKVCache
from .kernel import bf16_attention, choose_nsplit, AttnWorkspace

D = 128


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
    def __init__(self, weights: Weights, n_slots: int, kv: str = "gaac", bases: dict | None = None, ovf_bytes_per_tile: int = 128):
        assert kv in ("gaac", "bf16")
        self.w, self.cfg, self.kv, self.n_slots = weights, weights.cfg, kv, n_slots
        cfg, dev = self.cfg, weights.embed.device
        self.scale = D ** -0.5
        if kv == "gaac":
            self.caches = [CompressedKVCache(n_slots, cfg.n_kv_heads, cfg.max_len, None if bases is None else bases[i], ovf_bytes_per_tile, dev)
                           for i in range(cfg.n_layers)]
        else:
            self.caches = [_Bf16Cache(n_slots, cfg.n_kv_heads, cfg.max_len, dev) for _ in range(cfg.n_layers)]
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
        G = cfg.n_heads // cfg.n_kv_heads
        for layer, cache in zip(self.w.layers, self.caches):
            q, k, v = self._qkv(layer, x, pos)
            o = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                               is_causal=True, scale=self.scale, enable_gqa=G > 1)[0].transpose(0, 1)
            cache.prefill(slot, k, v)
            x = self._mlp(layer, x + F.linear(o.reshape(L, cfg.n_heads * D), layer["o"]))
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
        for layer, cache in zip(self.w.layers, self.caches):
            q, k, v = self._qkv(layer, x, pos)
            if self.kv == "gaac":
                cache.append(slots, k, v)
                o = cache.attention(q, slots, self.scale, nsplit=nsplit)
            else:
                cache.append(pos, k, v)
                o = cache.attention(q, lens + 1, self.scale, nsplit)
            x = self._mlp(layer, x + F.linear(o.reshape(x.shape[0], cfg.n_heads * D), layer["o"]))
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
    def decode(self, n_steps: int) -> torch.Tensor:
        """Runs n_steps greedy steps; returns the generated tokens [n_steps, B] (device)."""
        out = []
        for _ in range(n_steps):
            if self.graph is not None: self.graph.replay()
            else: self._one()
            out.append(self.tok.clone())
            self.steps += 1
            if self.kv == "gaac" and self.steps % 16 == 0:      # every 16 steps a head finalizes at most one tile (model_runner.py:268-273)
                used = torch.stack([c.max_escape_bytes() for c in self.caches]).tolist()
                for c, u in zip(self.caches, used): c.check_capacity(u)
        self.lens[:self.B] = self.dlens
        return torch.stack(out)

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
