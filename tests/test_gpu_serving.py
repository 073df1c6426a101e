"""GPU tests of the decode loop over the cache (the engine call site): a small Llama-architecture stack with random weights.
Pinned properties: the compressed cache is lossless (decompressed K/V of every layer bit-equal the uncompressed cache after
prefill), a captured decode step replays to the same tokens as eager steps, compressed and uncompressed runs agree on the logits
within attention rounding and on (almost) every greedy token, and the byte accounting is the closed form."""
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


def test_prefill_is_lossless_and_decode_matches_the_uncompressed_cache():
    dev = require_gpu()
    cfg, w, gaac, prompts, first_g = _setup(dev, "gaac")
    _, _, bf16, _, first_b = _setup(dev, "bf16", w, prompts)
    assert torch.equal(first_g, first_b)
    for layer in range(cfg.n_layers):
        for slot, p in enumerate(prompts):
            dk, dv = gaac.caches[layer].decompress(slot)
            L, h0 = p.shape[0], slot * cfg.n_kv_heads
            assert torch.equal(dk.view(torch.int16), bf16.caches[layer].k[h0:h0 + cfg.n_kv_heads, :L].transpose(0, 1).contiguous().view(torch.int16))
            assert torch.equal(dv.view(torch.int16), bf16.caches[layer].v[h0:h0 + cfg.n_kv_heads, :L].transpose(0, 1).contiguous().view(torch.int16))
    gaac.start_decode(first_g, use_graph=False); bf16.start_decode(first_b, use_graph=False)
    tg, tb = gaac.decode(1), bf16.decode(1)
    lg, lb = gaac.logits.float(), bf16.logits.float()
    assert (lg - lb).abs().max().item() <= 2e-2 * lb.abs().max().item() + 1e-3
    tg = torch.cat([tg, gaac.decode(39)]); tb = torch.cat([tb, bf16.decode(39)])
    assert (tg == tb).float().mean().item() >= 0.9
    st = gaac.kv_stats()
    assert st["tokens"] == sum(p.shape[0] for p in prompts) + 3 * 40 and st["bf16_bytes"] == st["tokens"] * cfg.n_kv_heads * 512 * cfg.n_layers
    assert 1.2 < st["ratio"] < 1.5
    # tokens that both runs generated identically give bit-identical layer-0 K/V rows in both caches
    same = (tg == tb).all(0)
    for slot in range(3):
        if not bool(same[slot]): continue
        dk, _ = gaac.caches[0].decompress(slot)
        L, h0 = dk.shape[0], slot * cfg.n_kv_heads
        assert L == prompts[slot].shape[0] + 40
        assert torch.equal(dk.view(torch.int16), bf16.caches[0].k[h0:h0 + cfg.n_kv_heads, :L].transpose(0, 1).contiguous().view(torch.int16))


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
