"""GPU tests of the decode loop over the cache (the engine call site): a small Llama-architecture stack with random weights.
Pinned properties: the compressed cache is lossless (decompressed K/V of every layer bit-equal what the layer was handed, and the
uncompressed cache where both runs see the same inputs), under teacher forcing the compressed and uncompressed runs agree on the logits
of every step within attention rounding, a captured decode step replays to the same tokens as eager steps, the engine-shaped surface
(context, spans, budgeted allocation, stats) behaves as the reference's runner expects, and the byte accounting is the closed form."""
import numpy as np
import pytest
import torch

from gpu_util import require_gpu

pytestmark = pytest.mark.gpu


def _setup(dev, kv, weights=None, prompts=None):
    from gaac_amd.serving import ModelConfig, Weights, DecodeRunner
    cfg = ModelConfig(hidden=256, n_layers=2, n_heads=8, n_kv_heads=2, ffn=512, vocab=512, rope_theta=10000.0, max_len=512)
    weights = weights or Weights(cfg, dev, seed=1)
    run = DecodeRunner(weights, n_slots=3, kv=kv)
    g = torch.Generator(device=dev).manual_seed(2)
    prompts = prompts or [torch.randint(0, cfg.vocab, (L,), generator=g, device=dev) for L in (200, 37, 64)]
    first = torch.stack([run.prefill(i, p).argmax() for i, p in enumerate(prompts)])
    return cfg, weights, run, prompts, first


def _cached_bf16(run, layer, slot, L):
    c, n_kv = run.caches[layer], run.cfg.n_kv_heads
    h0 = slot * n_kv
    return c.k[h0:h0 + n_kv, :L].transpose(0, 1).contiguous(), c.v[h0:h0 + n_kv, :L].transpose(0, 1).contiguous()


def _bits(t):
    return t.contiguous().view(torch.int16)


def test_teacher_forced_decode_matches_the_uncompressed_cache():
    """Both runs consume the same 40 tokens per sequence (teacher forcing), so they can be compared step by step: the logits of every
    step agree within attention rounding (the reference's bound, /root/reference/tests/test_kernel.py:19), every layer's cache holds
    bit for bit the K/V rows its attention layer was handed, layer 0 (whose inputs do not depend on attention) holds the same bits in
    both runs, and the first decode step's attention output is the oracle's attention over the decompressed cache."""
    from common import attention_error_bound, to_u16
    dev = require_gpu()
    cfg, w, gaac, prompts, first_g = _setup(dev, "gaac")
    _, _, bf16, _, first_b = _setup(dev, "bf16", w, prompts)
    assert torch.equal(first_g, first_b)
    for layer in range(cfg.n_layers):        # prefill: the same K/V went into both caches
        for slot, p in enumerate(prompts):
            dk, dv = gaac.caches[layer].decompress(slot)
            bk, bv = _cached_bf16(bf16, layer, slot, p.shape[0])
            assert torch.equal(_bits(dk), _bits(bk)) and torch.equal(_bits(dv), _bits(bv))
    seen = [[] for _ in range(cfg.n_layers)]       # (q, k, v, o) of every decode step, per layer
    for layer, attn in enumerate(gaac.attn):
        attn.register_forward_hook(lambda m, args, out, layer=layer: seen[layer].append(tuple(t.clone() for t in (*args, out))))
    n = 40
    forced = torch.randint(0, cfg.vocab, (n, 3), generator=torch.Generator(device=dev).manual_seed(5), device=dev)
    gaac.start_decode(first_g, use_graph=False); bf16.start_decode(first_b, use_graph=False)
    tg, lg = gaac.decode(n, forced=forced, keep_logits=True)
    tb, lb = bf16.decode(n, forced=forced, keep_logits=True)
    for i in range(n):
        err, bar = (lg[i] - lb[i]).abs().max().item(), 2e-2 * lb[i].abs().max().item() + 1e-3
        assert err <= bar, f"step {i}: logits differ by {err:.4g} > {bar:.4g}"
    assert (tg == tb).float().mean().item() >= 0.9
    # cache contents: prompt rows, then exactly the rows each layer appended
    for layer in range(cfg.n_layers):
        new_k = torch.stack([s[1] for s in seen[layer]]); new_v = torch.stack([s[2] for s in seen[layer]])      # [n, B, n_kv, D]
        for slot, p in enumerate(prompts):
            L = p.shape[0]
            dk, dv = gaac.caches[layer].decompress(slot)
            assert dk.shape[0] == L + n
            assert torch.equal(_bits(dk[L:]), _bits(new_k[:, slot])) and torch.equal(_bits(dv[L:]), _bits(new_v[:, slot]))
            if layer == 0:
                bk, bv = _cached_bf16(bf16, 0, slot, L + n)
                assert torch.equal(_bits(dk), _bits(bk)) and torch.equal(_bits(dv), _bits(bv))
    # first decode step, every layer: what the layer returned vs the oracle over what the cache held at that time
    for layer in range(cfg.n_layers):
        q, _, _, o = seen[layer][0]
        for slot, p in enumerate(prompts):
            L = p.shape[0] + 1
            dk, dv = gaac.caches[layer].decompress(slot)
            ref, tol = attention_error_bound(to_u16(q[slot]), to_u16(dk[:L]), to_u16(dv[:L]), gaac.scale)
            assert (np.abs(o[slot].float().cpu().numpy() - ref) <= tol).all()
    st = gaac.kv_stats()
    assert st["tokens"] == sum(p.shape[0] for p in prompts) + 3 * n and st["bf16_bytes"] == st["tokens"] * cfg.n_kv_heads * 512 * cfg.n_layers
    assert 1.2 < st["ratio"] < 1.5


def test_engine_surface_context_spans_and_a_cache_sized_from_a_budget():
    """The attention layer called the way the reference's runner calls it (/root/reference/nanovllm/engine/model_runner.py:130-153,
    195-215): caches allocated from a byte budget, a prefill step holding two sequences as spans of one token batch, a decode step with
    a padded row (slot -1), stats summed over layers."""
    from common import attention_error_bound, to_u16
    from gaac_amd.serving import Attention, allocate_gaac_cache, gaac_stats, set_context, reset_context, get_context
    from gaac_amd.kv_cache import CompressedKVCache
    dev = require_gpu()
    n_heads, n_kv, cap, scale = 8, 2, 256, 128 ** -0.5
    layers = [Attention(n_heads, 128, scale, n_kv) for _ in range(3)]
    per_slot = 3 * CompressedKVCache.bytes_per_slot(n_kv, cap)
    with pytest.raises(AssertionError, match="does not fit"):
        allocate_gaac_cache(layers, per_slot - 1, n_kv, cap, max_num_seqs=8, device=dev)
    num_slots, caches = allocate_gaac_cache(layers, 2 * per_slot + per_slot // 2, n_kv, cap, max_num_seqs=8, device=dev)
    assert num_slots == 2 and all(l.gaac is c and c.n_slots == 2 for l, c in zip(layers, caches))
    assert allocate_gaac_cache([Attention(n_heads, 128, scale, n_kv)], 100 * per_slot, n_kv, cap, max_num_seqs=4, device=dev)[0] == 4
    g = torch.Generator(device=dev).manual_seed(11)
    rnd = lambda *shape: torch.randn(*shape, generator=g, device=dev).to(torch.bfloat16)
    La, Lb = 50, 33
    q, k, v = rnd(La + Lb, n_heads, 128), rnd(La + Lb, n_kv, 128), rnd(La + Lb, n_kv, 128)
    cu = torch.tensor([0, La, La + Lb], dtype=torch.int32, device=dev)
    set_context(True, cu, cu, La, La, prefill_spans=[(1, 0, La), (0, La, La + Lb)])
    assert get_context().is_prefill and get_context().prefill_spans[0] == (1, 0, La)
    o = layers[0](q, k, v)
    reset_context()
    assert get_context().prefill_spans is None and not get_context().is_prefill
    dk, dv = caches[0].decompress(1)
    assert torch.equal(_bits(dk), _bits(k[:La])) and torch.equal(_bits(dv), _bits(v[:La]))
    dk, dv = caches[0].decompress(0)
    assert torch.equal(_bits(dk), _bits(k[La:])) and torch.equal(_bits(dv), _bits(v[La:]))
    # the last prompt position of a span attends over the whole span
    ref, tol = attention_error_bound(to_u16(q[La - 1]), to_u16(k[:La]), to_u16(v[:La]), scale)
    assert (np.abs(o[La - 1].float().cpu().numpy() - ref) <= tol).all()
    # decode: rows 0 and 2 are sequences (slots 1 and 0), row 1 is padding
    q1, k1, v1 = rnd(3, n_heads, 128), rnd(3, n_kv, 128), rnd(3, n_kv, 128)
    set_context(False, max_seqlen_k=cap, kv_slots=torch.tensor([1, -1, 0], dtype=torch.int32, device=dev))
    o1 = layers[0](q1, k1, v1)
    reset_context()
    for row, slot, L in ((0, 1, La), (2, 0, Lb)):
        dk, dv = caches[0].decompress(slot)
        assert dk.shape[0] == L + 1 and torch.equal(_bits(dk[-1]), _bits(k1[row])) and torch.equal(_bits(dv[-1]), _bits(v1[row]))
        ref, tol = attention_error_bound(to_u16(q1[row]), to_u16(dk), to_u16(dv), scale)
        assert (np.abs(o1[row].float().cpu().numpy() - ref) <= tol).all()
    st = gaac_stats(caches, num_slots)
    assert st["num_kv_slots"] == 2 and st["bf16_bytes"] == (La + Lb + 2) * n_kv * 512 and st["bytes_used"] == sum(c.stats()["bytes_used"] for c in caches)
    with pytest.raises(RuntimeError, match="no KV cache attached"):
        Attention(n_heads, 128, scale, n_kv)(q1, k1, v1)


@pytest.mark.parametrize("kv", ["gaac", "bf16"])
def test_captured_decode_step_replays_like_eager_steps(kv):
    """One graph of the whole step (all layers, append, attention, sampling) replayed 40 times vs 40 eager steps: same tokens, same
    lengths (two tails fill up on the way in the compressed cache)."""
    dev = require_gpu()
    cfg, w, a, prompts, first = _setup(dev, kv)
    _, _, b, _, _ = _setup(dev, kv, w, prompts)
    a.start_decode(first, use_graph=True); b.start_decode(first, use_graph=False)
    ta, tb = a.decode(40), b.decode(40)
    assert torch.equal(ta, tb)
    assert torch.equal(a.lens, b.lens) and a.lens.tolist() == [p.shape[0] + 40 for p in prompts]
    if kv == "gaac":
        for layer in range(cfg.n_layers):
            ka, va = a.caches[layer].decompress(0); kb, vb = b.caches[layer].decompress(0)
            assert torch.equal(ka.view(torch.int16), kb.view(torch.int16)) and torch.equal(va.view(torch.int16), vb.view(torch.int16))
