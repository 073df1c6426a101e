"""Properties that hold at any size, checked at the full size of the headline configuration (batch 1, 32 q / 8 kv heads, d = 128,
65536 compressed tokens + a 7-token tail), where the CPU oracle would take minutes: the round trip is the identity, the result does
not depend on how the sequence is split, equal value rows come back unchanged, a zero query averages the values, and dropping the
tail rows gives the attention over the compressed rows alone."""
import numpy as np
import pytest
import torch

from gpu_util import require_gpu

pytestmark = pytest.mark.gpu
N_KV, G, D, S, TAIL = 8, 4, 128, 65536, 7
SCALE = D ** -0.5


def _kv(seed, dev, spread):
    """bf16 [N_KV, S + TAIL, D] made on the device: per-channel scales over `spread` octaves, sparse large values (all three tiers)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    sig = torch.exp2(torch.rand(N_KV, 1, D, generator=g, device=dev) * spread - spread / 2)
    x = torch.randn(N_KV, S + TAIL, D, generator=g, device=dev) * sig
    hit = torch.rand(N_KV, S + TAIL, D, generator=g, device=dev) < 0.0003
    return torch.where(hit, x * 4096.0, x).to(torch.bfloat16)


def _encode(x, kind):
    from gaac_amd import Codec, TileEncoder
    c = Codec(N_KV).calibrate(x[:, :1024])
    return TileEncoder(kind).encode(c, x[:, :S].contiguous())


def _attend(q, kp, vp, k, v, nsplit, with_tail=True):
    """the fused launch over the compressed pages (+ the raw tail rows S .. S+TAIL)"""
    from gaac_amd.kernel import attn_launch
    dev = q.device
    kt = torch.zeros(N_KV, 16, D, dtype=torch.bfloat16, device=dev); vt = torch.zeros_like(kt)
    kt[:, :TAIL] = k[:, S:]; vt[:, :TAIL] = v[:, S:]
    TL = torch.full((N_KV,), TAIL if with_tail else 0, dtype=torch.int32, device=dev)
    SL = torch.full((N_KV,), S, dtype=torch.int32, device=dev)
    slots = torch.zeros(1, dtype=torch.int32, device=dev)
    return attn_launch(kp, vp, q.reshape(N_KV * G, D), slots, N_KV * G, N_KV, SL, S, SCALE, nsplit, kt, vt, TL, 16).float()


def _fp32_attention(q, k, v):
    """textbook softmax attention in fp32 on the device over the given rows, GQA by repetition"""
    qf = q.float().view(N_KV, G, D)
    s = torch.einsum("hgd,hsd->hgs", qf, k.float()) * SCALE
    return torch.einsum("hgs,hsd->hgd", torch.softmax(s, -1), v.float()).reshape(N_KV * G, D)


def test_round_trip_is_the_identity_at_full_size():
    dev = require_gpu()
    from gaac_amd import Codec
    for kind, seed in (("k", 1), ("v", 2)):
        x = _kv(seed, dev, 8.0)[:, :S].contiguous()
        page = _encode(x, kind)
        assert torch.equal(Codec.decode(page).view(torch.int16), x.view(torch.int16))
        assert 1.3 < page.ratio < 1.5
        tags = page.flags.view(N_KV, S, 1) >> (2 * torch.arange(16, device=dev, dtype=torch.int32)) & 3
        assert int((tags == 2).sum()) == 0 and int((tags == 1).sum()) > 0 and int((tags == 3).sum()) > 0      # tags are 0, 1 or 3


def test_full_size_attention_properties():
    dev = require_gpu()
    k, v = _kv(11, dev, 2.0), _kv(12, dev, 2.0)
    kp, vp = _encode(k, "k"), _encode(v, "v")
    g = torch.Generator(device=dev).manual_seed(3)
    q = (torch.randn(N_KV * G, D, generator=g, device=dev) * 0.3).to(torch.bfloat16)
    ref = _fp32_attention(q, k, v)
    mag = float(ref.abs().max())
    outs = {n: _attend(q, kp, vp, k, v, n) for n in (1, 32, 61, 256)}
    for n, o in outs.items():      # the reference's tolerance (tests/test_kernel.py:19) against fp32 attention over the same bf16 rows
        assert float((o - ref).abs().max()) <= 2e-2 * mag + 1e-3, n
    for n in (1, 61, 256):         # split-count independence up to fp32 summation order + the bf16 output rounding
        assert float((outs[n] - outs[32]).abs().max()) <= 2.0 ** -7 * mag + 1e-6, n
    # a zero query weighs every row alike: the output is the mean of the value rows
    mean_v = v.float().mean(1, keepdim=True).expand(N_KV, G, D).reshape(N_KV * G, D)
    o = _attend(torch.zeros_like(q), kp, vp, k, v, 32)
    assert float((o - mean_v).abs().max()) <= 2e-2 * float(mean_v.abs().max()) + 1e-3
    # without the tail rows the result is the attention over the compressed rows alone
    o = _attend(q, kp, vp, k, v, 32, with_tail=False)
    ref_c = _fp32_attention(q, k[:, :S], v[:, :S])
    assert float((o - ref_c).abs().max()) <= 2e-2 * float(ref_c.abs().max()) + 1e-3


def test_equal_value_rows_come_back_unchanged_at_full_size():
    dev = require_gpu()
    k = _kv(21, dev, 2.0)
    row = (torch.randn(N_KV, 1, D, generator=torch.Generator(device=dev).manual_seed(5), device=dev) * 2).to(torch.bfloat16)
    v = row.expand(N_KV, S + TAIL, D).contiguous()
    kp, vp = _encode(k, "k"), _encode(v, "v")
    q = torch.randn(N_KV * G, D, generator=torch.Generator(device=dev).manual_seed(6), device=dev).to(torch.bfloat16)
    o = _attend(q, kp, vp, k, v, 32)
    want = row.float().expand(N_KV, G, D).reshape(N_KV * G, D)
    # softmax weights sum to one: every output row is the value row, up to the fp32 normalisation and the bf16 rounding of the output
    assert float((o - want).abs().max()) <= 2.0 ** -7 * float(want.abs().max())


def test_doubled_values_double_the_output_at_full_size():
    """V -> 2 V is exact in bf16 and moves every exponent, and with them the calibrated bases, by one: the page has the same tiers
    under the shifted bases, and the output doubles (up to the order of the fp32 sums, which the dynamic tile hand-out changes from launch to launch,
    and the bf16 rounding of the output)."""
    dev = require_gpu()
    k, v = _kv(31, dev, 2.0), _kv(32, dev, 2.0)
    v2 = (v.float() * 2).to(torch.bfloat16)
    assert torch.equal(v2.float(), v.float() * 2)
    kp, vp, vp2 = _encode(k, "k"), _encode(v, "v"), _encode(v2, "v")
    assert torch.equal(vp2.base3.int(), vp.base3.int() + 1) and torch.equal(vp2.flags, vp.flags)      # (raw groups keep the exponent's own low bits as their codes)
    q = (torch.randn(N_KV * G, D, generator=torch.Generator(device=dev).manual_seed(7), device=dev) * 0.3).to(torch.bfloat16)
    o, o2 = _attend(q, kp, vp, k, v, 32), _attend(q, kp, vp2, k, v2, 32)
    assert float((o2 - 2 * o).abs().max()) <= 2.0 ** -7 * float(o2.abs().max())


def test_byte_offsets_beyond_4_gib():
    """Five batch rows of 2^20 tokens: the sign/mantissa array of a page is 5 GiB, so the last row's tiles sit beyond 32-bit byte
    offsets in every kernel (encoder, decoder, attention).  Checked on the first and the last row."""
    dev = require_gpu()
    from gaac_amd import Codec, TileEncoder, attention
    B, n_kv, g_, S_ = 5, 8, 2, 1 << 20
    gen = torch.Generator(device=dev).manual_seed(31)
    def make(seed_shift):
        sig = torch.exp2(torch.rand(B * n_kv, 1, D, generator=gen, device=dev) * 2 - 1)
        x = torch.empty(B * n_kv, S_, D, dtype=torch.bfloat16, device=dev)
        for h in range(B * n_kv):      # head by head: no fp32 copy of the whole tensor
            x[h] = (torch.randn(S_, D, generator=gen, device=dev) * sig[h]).to(torch.bfloat16)
        return x
    k, v = make(0), make(1)
    ck, cv = Codec(n_kv).calibrate(k[:n_kv, :2048]), Codec(n_kv).calibrate(v[:n_kv, :2048])
    kp, vp = TileEncoder("k").encode(ck, k), TileEncoder("v").encode(cv, v)
    assert kp.sm.numel() > (1 << 32) and kp.sm.shape == (B * n_kv, S_ * D)
    for page, x in ((kp, k), (vp, v)):
        back = Codec.decode(page)
        for h in (0, B * n_kv - 1):
            assert torch.equal(back[h].view(torch.int16), x[h].view(torch.int16)), h
        del back
    q = (torch.randn(B, n_kv * g_, D, generator=gen, device=dev) * 0.3).to(torch.bfloat16)
    out = attention(q, kp, vp, SCALE).float()
    for b in (0, B - 1):
        kb, vb = k[b * n_kv:(b + 1) * n_kv].float(), v[b * n_kv:(b + 1) * n_kv].float()
        s = torch.einsum("hgd,hsd->hgs", q[b].float().view(n_kv, g_, D), kb) * SCALE
        ref = torch.einsum("hgs,hsd->hgd", torch.softmax(s, -1), vb).reshape(n_kv * g_, D)
        assert float((out[b] - ref).abs().max()) <= 2e-2 * float(ref.abs().max()) + 1e-3, b
        del kb, vb, s


def test_config_2_at_full_size():
    """24 query heads over 4 kv heads (group 6), 65536 compressed tokens + 7 tail tokens, V's channel scales over 4 octaves, at the
    launcher's own split count (64 splits of eight-wave blocks) and at others, against fp32 attention on the device over the same rows."""
    dev = require_gpu()
    from gaac_amd import Codec, TileEncoder
    from gaac_amd.kernel import attn_launch, choose_nsplit
    n_kv, g_ = 4, 6
    gen = torch.Generator(device=dev).manual_seed(41)
    def make(spread):
        sig = torch.exp2(torch.rand(n_kv, 1, D, generator=gen, device=dev) * spread - spread / 2)
        x = torch.randn(n_kv, S + TAIL, D, generator=gen, device=dev) * sig
        hit = torch.rand(n_kv, S + TAIL, D, generator=gen, device=dev) < 0.0003
        return torch.where(hit, x * 4096.0, x).to(torch.bfloat16)
    k, v = make(2.0), make(4.0)
    kp = TileEncoder("k").encode(Codec(n_kv).calibrate(k[:, :1024]), k[:, :S].contiguous())
    vp = TileEncoder("v").encode(Codec(n_kv).calibrate(v[:, :1024]), v[:, :S].contiguous())
    assert torch.equal(Codec.decode(vp).view(torch.int16), v[:, :S].contiguous().view(torch.int16))
    q = (torch.randn(n_kv * g_, D, generator=gen, device=dev) * 0.3).to(torch.bfloat16)
    kt = torch.zeros(n_kv, 16, D, dtype=torch.bfloat16, device=dev); vt = torch.zeros_like(kt)
    kt[:, :TAIL] = k[:, S:]; vt[:, :TAIL] = v[:, S:]
    TL = torch.full((n_kv,), TAIL, dtype=torch.int32, device=dev); SL = torch.full((n_kv,), S, dtype=torch.int32, device=dev)
    s = torch.einsum("hgd,hsd->hgs", q.float().view(n_kv, g_, D), k.float()) * SCALE
    ref = torch.einsum("hgs,hsd->hgd", torch.softmax(s, -1), v.float()).reshape(n_kv * g_, D)
    mag = float(ref.abs().max())
    assert choose_nsplit(1, n_kv, S) == 64
    for ns, s_all in ((64, S), (64, -1), (32, S), (200, -1)):
        o = attn_launch(kp, vp, q, None, n_kv * g_, n_kv, SL, S, SCALE, ns, kt, vt, TL, 16, S_all=s_all).float()
        assert float((o - ref).abs().max()) <= 2e-2 * mag + 1e-3, (ns, s_all)
        assert float((o - ref).abs().mean()) <= 1e-3 * max(mag, 1.0), (ns, s_all)


def test_config_3_paged_pool_at_full_size():
    """16 sequences of U[4096, 65536] tokens (seed 4) in a pool addressed through a permuted block table (seed 5), 32 query / 8 kv heads:
    prompts stored, a few decode steps appended (blocks fill up and are compressed), then decode attention at the launcher's split count,
    at one where the longest sequence puts exactly 1024 tiles into a split (what a block's tile table holds at a time), and at 3, 2 and
    1 splits, where a split runs on for several rounds of its table (the reference resolves block-table entries tile by tile and has no
    such bound, /root/reference/gaac/vllm/paged_kernel.py:137-165), against fp32 attention on the device over the rows that went in;
    decode_blocks returns those rows bit for bit."""
    dev = require_gpu()
    from gaac_amd.codec import exponent_hist, bases_from_hist
    from gaac_amd.paged import LayerState, build_store_entries, choose_nsplit, BLOCK
    n_seq, n_kv, g_, steps = 16, 8, 4, 5
    n_q = n_kv * g_
    lens = np.random.default_rng(4).integers(4096, 65537, n_seq).tolist()
    lens[3] = 65536 - steps                       # one sequence ends exactly on the edge of the tile table (1024 tiles per split) at 4 splits
    nblk = [-(-(L + steps) // BLOCK) for L in lens]
    perm = np.random.default_rng(5).permutation(sum(nblk))
    bt_cpu = np.zeros((n_seq, max(nblk)), np.int32); o = 0
    for i, nb in enumerate(nblk):
        bt_cpu[i, :nb] = perm[o:o + nb]; o += nb
    gen = torch.Generator(device=dev).manual_seed(6)
    sig_k = torch.exp2(torch.rand(1, n_kv, D, generator=gen, device=dev) * 2 - 1); sig_v = torch.exp2(torch.rand(1, n_kv, D, generator=gen, device=dev) * 2 - 1)
    def rows(n, sig):
        x = torch.randn(n, n_kv, D, generator=gen, device=dev) * sig
        hit = torch.rand(n, n_kv, D, generator=gen, device=dev) < 0.0003
        return torch.where(hit, x * 4096.0, x).to(torch.bfloat16)
    k3, k4 = bases_from_hist(exponent_hist(rows(1024, sig_k), n_kv), n_kv); v3, v4 = bases_from_hist(exponent_hist(rows(1024, sig_v), n_kv), n_kv)
    st = LayerState(sum(nblk), n_kv, 2 * n_kv * 4 * n_seq + sum(nblk) * 2 * n_kv // 100 + 64, dict(k3=k3, k4=k4, v3=v3, v4=v4), 128, dev)
    buf = torch.zeros(LayerState.pool_bytes(sum(nblk), n_kv, 128), dtype=torch.uint8, device=dev)
    hist_k, hist_v = [], []
    for i, L in enumerate(lens):
        kk, vv = rows(L, sig_k), rows(L, sig_v)
        st.store(kk, vv, buf, torch.from_numpy(build_store_entries([0], [L], [bt_cpu[i]])).to(dev))
        hist_k.append(kk); hist_v.append(vv)
    cur = list(lens)
    for _ in range(steps):
        kn, vn = rows(n_seq, sig_k), rows(n_seq, sig_v)
        st.store(kn, vn, buf, torch.from_numpy(build_store_entries(cur, [1] * n_seq, bt_cpu)).to(dev))
        for i in range(n_seq):
            hist_k[i] = torch.cat([hist_k[i], kn[i:i + 1]]); hist_v[i] = torch.cat([hist_v[i], vn[i:i + 1]])
        cur = [c + 1 for c in cur]
    st.check()
    bt = torch.from_numpy(bt_cpu).to(dev)
    seq_lens = torch.tensor(cur, dtype=torch.int32, device=dev)
    q = (torch.randn(n_seq, n_q, D, generator=gen, device=dev) * 0.3).to(torch.bfloat16)
    refs = []
    for i in range(n_seq):
        s = torch.einsum("hgd,shd->hgs", q[i].float().view(n_kv, g_, D), hist_k[i].float()) * SCALE
        refs.append(torch.einsum("hgs,shd->hgd", torch.softmax(s, -1), hist_v[i].float()).reshape(n_q, D))
    assert max(cur) == 65536
    for ns in (choose_nsplit(n_seq, n_kv, max(cur)), 4, 7, 3, 2, 1):
        out = st.attention(q, buf, bt, seq_lens, ns, max_seq_len=max(cur)).float().view(n_seq, n_q, D)
        for i in range(n_seq):
            assert float((out[i] - refs[i]).abs().max()) <= 2e-2 * float(refs[i].abs().max()) + 1e-3, (ns, i, cur[i])
    st.check()
    for i in (int(np.argmax(cur)), int(np.argmin(cur))):
        nb_l = -(-cur[i] // BLOCK)
        pairs = torch.tensor([(int(bt_cpu[i][j]), 16 * j, min(16, cur[i] - 16 * j)) for j in range(nb_l)], dtype=torch.int32, device=dev)
        sk = torch.empty(cur[i], n_kv, D, dtype=torch.bfloat16, device=dev); sv = torch.empty_like(sk)
        st.decode_blocks(buf, pairs, sk, sv)
        assert torch.equal(sk.view(torch.int16), hist_k[i].view(torch.int16)) and torch.equal(sv.view(torch.int16), hist_v[i].view(torch.int16))


def test_config_4_call_site_at_full_size():
    """Config 4: the Llama-3-8B architecture (32 layers, hidden 4096, 32 q / 8 kv heads, FFN 14336, vocab 128256; random bf16 weights),
    batch 4 at 32768-token contexts, through the engine-shaped call site.  Teacher forcing makes the compressed and the uncompressed
    run comparable step by step: after the prefill and after 6 forced decode steps every layer's cache holds the same K/V bits in
    both runs where their inputs are the same (all layers during prefill, layer 0 throughout; position-weighted checksums), the
    rows a layer appended are bit for bit what it was handed, and the logits of every step differ by no more than a small multiple
    of what the uncompressed run itself changes by when only its split count (summation order) changes."""
    dev = require_gpu()
    from gaac_amd.serving import ModelConfig, Weights, DecodeRunner
    B, ctx, steps = 4, 32768, 6
    cfg = ModelConfig(max_len=ctx + 64)
    w = Weights(cfg, dev, seed=0)
    g = torch.Generator(device=dev).manual_seed(1)
    prompts = [torch.randint(0, cfg.vocab, (ctx,), generator=g, device=dev) for _ in range(B)]
    forced = torch.randint(0, cfg.vocab, (steps, B), generator=g, device=dev)

    def checksum(x, L):
        bits = x[:L].contiguous().view(torch.int16).to(torch.int64).flatten()
        return int((bits * (torch.arange(bits.numel(), device=dev) % 65521 + 1)).sum().item())

    def run(kv, nsplit=None, sums=True):
        r = DecodeRunner(w, n_slots=B, kv=kv)
        first = torch.stack([r.prefill(i, p).argmax() for i, p in enumerate(prompts)])
        fed = [[] for _ in range(cfg.n_layers)]
        hooks = [at.register_forward_hook(lambda m, args, out, l=l: fed[l].append((args[1].clone(), args[2].clone()))) for l, at in enumerate(r.attn)]
        r.start_decode(first, use_graph=False, nsplit=nsplit)
        _, lg = r.decode(steps, forced=forced, keep_logits=True)
        for h in hooks: h.remove()
        cs = []
        for l in range(cfg.n_layers if sums else 0):
            for slot in range(B):
                L = ctx + steps if l == 0 else ctx
                if kv == "gaac":
                    dk, dv = r.caches[l].decompress(slot)
                    assert dk.shape[0] == ctx + steps
                    nk = torch.stack([f[0][slot] for f in fed[l]]); nv = torch.stack([f[1][slot] for f in fed[l]])
                    assert torch.equal(dk[ctx:].view(torch.int16), nk.view(torch.int16)) and torch.equal(dv[ctx:].view(torch.int16), nv.view(torch.int16)), (l, slot)
                else:
                    c, h0 = r.caches[l], slot * cfg.n_kv_heads
                    dk, dv = c.k[h0:h0 + cfg.n_kv_heads, :L].transpose(0, 1), c.v[h0:h0 + cfg.n_kv_heads, :L].transpose(0, 1)
                cs.append((checksum(dk, L), checksum(dv, L)))
                del dk, dv
        st = r.kv_stats()
        del r
        torch.cuda.empty_cache()
        return first, lg, cs, st

    first_g, lg, cs_g, st_g = run("gaac")
    first_b, lb, cs_b, _ = run("bf16")
    assert torch.equal(first_g, first_b)
    assert cs_g == cs_b
    _, ln, _, _ = run("bf16", nsplit=5, sums=False)
    d = (lg - lb).abs().flatten(1); dn = (ln - lb).abs().flatten(1)
    for i in range(steps):
        assert d[i].max().item() <= 4 * dn.max().item() and d[i].mean().item() <= 2 * dn.mean().item(), (i, d[i].max().item(), dn.max().item())
    assert st_g["tokens"] == B * (ctx + steps) and 1.3 < st_g["ratio"] < 1.5
