"""GPU tests of the slot cache: prefill / append / attention / decompress over a changing batch and one decode step replayed
as a HIP graph.  Same scenarios and tolerances as /root/reference/tests/test_kv_cache.py:15-86; the expected values come
from the history kept on the host (bit-exact decompress) and the oracle's fp32 attention."""
import numpy as np
import pytest
import torch

from oracle import gaac_oracle as O
from common import kv_like16, to_bf16, to_u16, randn_bf16
from gpu_util import require_gpu

pytestmark = pytest.mark.gpu
N_KV, G, SCALE = 4, 4, 128 ** -0.5


def _tok16(x16):          # [n_kv, L, D] -> token-major [L, n_kv, D]
    return np.ascontiguousarray(x16.transpose(1, 0, 2))


def _bases(seed, dev):
    from gaac_amd.codec import exponent_hist, bases_from_hist
    out = {}
    for name, sd in (("k", seed), ("v", seed + 1)):
        x = to_bf16(_tok16(kv_like16(N_KV, 4096, seed=sd, scale_seed=1000 + (name == "v"))), dev)
        out[name + "3"], out[name + "4"] = bases_from_hist(exponent_hist(x, N_KV), N_KV)
    return out


def _prompt(L, seed):
    return _tok16(kv_like16(N_KV, L, seed=seed, scale_seed=1000)), _tok16(kv_like16(N_KV, L, seed=seed + 500, scale_seed=1001))


def _check(cache, hist, slots_l, q16, dev):
    slots = torch.tensor(slots_l, dtype=torch.int32, device=dev)
    out = O.bf16_to_f32(to_u16(cache.attention(to_bf16(q16, dev), slots, SCALE)))
    for b, s in enumerate(slots_l):
        if s < 0:
            assert np.abs(out[b]).max() == 0
            continue
        k16, v16 = hist[s]
        ref = O.ref_attention(q16[b], k16, v16, SCALE)
        assert np.abs(out[b] - ref).max() <= 2e-2 * np.abs(ref).max() + 1e-3
        dk, dv = cache.decompress(s)
        assert np.array_equal(to_u16(dk), k16) and np.array_equal(to_u16(dv), v16)


@pytest.mark.parametrize("static_bases", [True, False])
def test_slots_prefill_append(static_bases):
    dev = require_gpu()
    from gaac_amd import CompressedKVCache
    cache = CompressedKVCache(n_slots=4, n_kv=N_KV, capacity=1024, bases=_bases(10, dev) if static_bases else None)
    hist = {}
    for s, L in {0: 37, 2: 500, 3: 16}.items():
        k16, v16 = _prompt(L, 20 + s)
        cache.prefill(s, to_bf16(k16, dev), to_bf16(v16, dev)); hist[s] = (k16, v16)
    for step in range(40):      # decode steps over a changing batch (slot order != batch order, plus a padded row)
        slots_l = [3, 0, 2, -1] if step % 3 else [2, 3, -1, 0]
        k16 = randn_bf16((4, N_KV, 128), seed=100 + step, scale=0.5); v16 = randn_bf16((4, N_KV, 128), seed=200 + step, scale=0.5)
        cache.append(torch.tensor(slots_l, dtype=torch.int32, device=dev), to_bf16(k16, dev), to_bf16(v16, dev))
        for b, s in enumerate(slots_l):
            if s >= 0: hist[s] = (np.concatenate([hist[s][0], k16[b:b + 1]]), np.concatenate([hist[s][1], v16[b:b + 1]]))
        if step % 16 == 15: cache.check_capacity()
        if step % 13 == 0 or step == 39:
            _check(cache, hist, slots_l, randn_bf16((4, N_KV * G, 128), seed=300 + step, scale=0.1), dev)
    st = cache.stats()
    assert st["tokens"] == sum(len(h[0]) for h in hist.values())
    S = sum(len(h[0]) // 16 * 16 for h in hist.values()) * N_KV; tl = sum(len(h[0]) % 16 for h in hist.values()) * N_KV
    esc = int(cache.k.ovf_used.sum()) + int(cache.v.ovf_used.sum())
    assert st["bytes_used"] == 2 * (S * 180 + S // 16 * 4 + tl * 256) + esc and st["bf16_bytes"] == 2 * (S + tl) * 256
    # slot reuse: a new sequence replaces slot 0
    k16, v16 = _prompt(64, 99)
    cache.prefill(0, to_bf16(k16, dev), to_bf16(v16, dev)); hist[0] = (k16, v16)
    _check(cache, hist, [0], randn_bf16((1, N_KV * G, 128), seed=400, scale=0.1), dev)


def test_graph_decode_step():
    """append + attention captured once and replayed 40 times (two tails fill up on the way), every replay checked."""
    dev = require_gpu()
    from gaac_amd import CompressedKVCache
    cache = CompressedKVCache(n_slots=2, n_kv=N_KV, capacity=512, bases=_bases(11, dev))
    k0, v0 = _prompt(200, 5)
    cache.prefill(1, to_bf16(k0, dev), to_bf16(v0, dev))
    slots = torch.tensor([1, -1], dtype=torch.int32, device=dev)
    q = torch.zeros(2, N_KV * G, 128, dtype=torch.bfloat16, device=dev)
    kn = torch.zeros(2, N_KV, 128, dtype=torch.bfloat16, device=dev); vn = torch.zeros_like(kn)
    def step():
        cache.append(slots, kn, vn); return cache.attention(q, slots, SCALE, max_len=512)
    s = torch.cuda.Stream(); s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):          # warm up outside capture with every row padded (nothing is appended)
        slots.fill_(-1); step()
    torch.cuda.current_stream().wait_stream(s)
    cache.growable = False
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = step()
    slots.copy_(torch.tensor([1, -1], dtype=torch.int32))
    hk, hv = k0, v0
    for i in range(40):
        k16 = randn_bf16((2, N_KV, 128), seed=500 + i, scale=0.5); v16 = randn_bf16((2, N_KV, 128), seed=600 + i, scale=0.5)
        q16 = randn_bf16((2, N_KV * G, 128), seed=700 + i, scale=0.1)
        kn.copy_(to_bf16(k16, dev)); vn.copy_(to_bf16(v16, dev)); q.copy_(to_bf16(q16, dev))
        g.replay(); torch.cuda.synchronize()
        hk, hv = np.concatenate([hk, k16[:1]]), np.concatenate([hv, v16[:1]])
        got = O.bf16_to_f32(to_u16(out))
        ref = O.ref_attention(q16[0], hk, hv, SCALE)
        assert np.abs(got[0] - ref).max() <= 2e-2 * np.abs(ref).max() + 1e-3, i
        assert np.abs(got[1]).max() == 0
    dk, dv = cache.decompress(1)
    assert np.array_equal(to_u16(dk), hk) and np.array_equal(to_u16(dv), hv)
    cache.check_capacity()


def test_overflow_is_flagged_not_written():
    """A head at capacity drops the token and raises at the next check; an escape stream without room stores a zero-tagged tile."""
    dev = require_gpu()
    from gaac_amd import CompressedKVCache
    cache = CompressedKVCache(n_slots=1, n_kv=N_KV, capacity=32, bases=_bases(12, dev))
    k16, v16 = _prompt(32, 7)
    cache.prefill(0, to_bf16(k16, dev), to_bf16(v16, dev))
    slots = torch.zeros(1, dtype=torch.int32, device=dev)
    for i in range(16):
        cache.append(slots, to_bf16(randn_bf16((1, N_KV, 128), seed=i), dev), to_bf16(randn_bf16((1, N_KV, 128), seed=50 + i), dev))
    assert int(cache.S.max()) == 32 and int(cache.tail_len.max()) == 0
    with pytest.raises(RuntimeError, match="token capacity"):
        cache.check_capacity()
    # escape stream: all-raw tiles (exponents far from the bases) need 1280 B per tile, the stream holds 2*16+8
    cache = CompressedKVCache(n_slots=1, n_kv=N_KV, capacity=64, bases=_bases(12, dev), ovf_bytes_per_tile=8)
    cache.growable = False
    big = to_bf16(np.full((1, N_KV, 128), 0x7F00, dtype=np.uint16), dev)
    for i in range(16): cache.append(slots, big, big)
    with pytest.raises(RuntimeError, match="escape window"):
        cache.check_capacity()
    assert int(cache.k.ovf_used.max()) == 0 and int(cache.k.flags.abs().max()) == 0


@pytest.mark.parametrize("n_kv,G", [(1, 16), (8, 1), (2, 6)])
def test_other_head_shapes_with_random_batches(n_kv, G):
    """Per-sequence bases, random prompt lengths (incl. shorter than one tile), random batches with padded rows, 50 decode steps."""
    dev = require_gpu()
    from gaac_amd import CompressedKVCache
    rng = np.random.default_rng(n_kv * 100 + G)
    n_slots = 5
    cache = CompressedKVCache(n_slots=n_slots, n_kv=n_kv, capacity=300)
    tok = lambda x16: np.ascontiguousarray(x16.transpose(1, 0, 2))
    def kv_like16(H, L, seed, scale_seed=None):      # unit-scale values (spread-out softmax weights) with sparse far-off ones
        x = randn_bf16((H, L, 128), seed=seed)
        x[:, ::5, 3::29] = 0x3580
        return x
    hist = {}
    for s in range(n_slots):
        L = int(rng.choice([1, 7, 16, 33, 150]))
        k16, v16 = tok(kv_like16(n_kv, L, seed=10 + s, scale_seed=77)), tok(kv_like16(n_kv, L, seed=60 + s, scale_seed=78))
        cache.prefill(s, to_bf16(k16, dev), to_bf16(v16, dev)); hist[s] = (k16, v16)
    for step in range(50):
        slots_l = [int(x) for x in rng.permutation(n_slots)[:3]] + [-1]
        rng.shuffle(slots_l)
        k16, v16 = tok(kv_like16(n_kv, 4, seed=500 + step, scale_seed=77)), tok(kv_like16(n_kv, 4, seed=900 + step, scale_seed=78))
        cache.append(torch.tensor(slots_l, dtype=torch.int32, device=dev), to_bf16(k16, dev), to_bf16(v16, dev))
        for b, s in enumerate(slots_l):
            if s >= 0: hist[s] = (np.concatenate([hist[s][0], k16[b:b + 1]]), np.concatenate([hist[s][1], v16[b:b + 1]]))
        if step % 16 == 15: cache.check_capacity()
        if step % 17 == 0 or step == 49:
            q16 = randn_bf16((4, n_kv * G, 128), seed=300 + step, scale=1.0)
            out = O.bf16_to_f32(to_u16(cache.attention(to_bf16(q16, dev), torch.tensor(slots_l, dtype=torch.int32, device=dev), SCALE)))
            for b, s in enumerate(slots_l):
                if s < 0:
                    assert np.abs(out[b]).max() == 0
                    continue
                ref = O.ref_attention(q16[b], hist[s][0], hist[s][1], SCALE)
                assert np.abs(out[b] - ref).max() <= 2e-2 * np.abs(ref).max() + 1e-3, (step, b, s)
    for s in range(n_slots):
        dk, dv = cache.decompress(s)
        assert np.array_equal(to_u16(dk), hist[s][0]) and np.array_equal(to_u16(dv), hist[s][1])


def test_many_rows_with_short_and_tail_only_sequences():
    """A batch of 72 rows over 80 slots (more than 256 blocks: the four-wave block shape, one split per head): sequences of 1..70 tokens,
    many of them shorter than one tile, so the only partial of a head is the one its first wave makes from the raw tail rows."""
    dev = require_gpu()
    from gaac_amd import CompressedKVCache
    n_slots = 80
    cache = CompressedKVCache(n_slots=n_slots, n_kv=N_KV, capacity=128, bases=_bases(12, dev))
    rng = np.random.default_rng(8)
    hist = {}
    order = rng.permutation(n_slots)[:72]
    for s in order:
        L = int(rng.integers(1, 71)) if s % 5 else int(rng.integers(1, 16))
        k16, v16 = _prompt(L, 900 + int(s))
        cache.prefill(int(s), to_bf16(k16, dev), to_bf16(v16, dev)); hist[int(s)] = (k16, v16)
    slots_l = [int(s) for s in order]
    slots_l[5] = -1; slots_l[40] = -1
    q16 = randn_bf16((72, N_KV * G, 128), seed=77, scale=0.1)
    slots = torch.tensor(slots_l, dtype=torch.int32, device=dev)
    out = O.bf16_to_f32(to_u16(cache.attention(to_bf16(q16, dev), slots, SCALE)))
    for b, s in enumerate(slots_l):
        if s < 0:
            assert np.abs(out[b]).max() == 0
            continue
        ref = O.ref_attention(q16[b], hist[s][0], hist[s][1], SCALE)
        assert np.abs(out[b] - ref).max() <= 2e-2 * np.abs(ref).max() + 1e-3, (b, s, len(hist[s][0]))
    # one decode step on every live row, then the same check on a few rows
    k16 = randn_bf16((72, N_KV, 128), seed=78, scale=0.5); v16 = randn_bf16((72, N_KV, 128), seed=79, scale=0.5)
    cache.append(slots, to_bf16(k16, dev), to_bf16(v16, dev))
    for b, s in enumerate(slots_l):
        if s >= 0: hist[s] = (np.concatenate([hist[s][0], k16[b:b + 1]]), np.concatenate([hist[s][1], v16[b:b + 1]]))
    out = O.bf16_to_f32(to_u16(cache.attention(to_bf16(q16, dev), slots, SCALE, nsplit=3)))
    for b in (0, 7, 33, 71):
        s = slots_l[b]
        ref = O.ref_attention(q16[b], hist[s][0], hist[s][1], SCALE)
        assert np.abs(out[b] - ref).max() <= 2e-2 * np.abs(ref).max() + 1e-3
        dk, dv = cache.decompress(s)
        assert np.array_equal(to_u16(dk), hist[s][0]) and np.array_equal(to_u16(dv), hist[s][1])
    cache.check_capacity()


@pytest.mark.parametrize("per_sequence_bases", [True, False])
def test_bytes_per_slot_is_what_the_cache_allocates(per_sequence_bases):
    """bytes_per_slot (/root/reference/gaac/kv_cache.py:142-146) against the tensors a cache really holds: the bytes of every
    per-head tensor of both stores (tile rows, tag words, tile offsets, escape streams, stream starts, counters, raw tails, and for
    per-sequence calibration the base rows) plus the two length vectors add up to n_slots * bytes_per_slot, except for the one closing
    entry of each store's stream-start vector (2 x 4 bytes per cache); per-model base tables (not per slot) are left out, as in the
    reference's formula.  The oracle's restatement of the formula gives the same number."""
    dev = require_gpu()
    from gaac_amd import CompressedKVCache
    from gaac_amd.codec import exponent_hist, bases_from_hist
    for (n_slots, n_kv, cap, ovf) in [(1, 1, 16, 128), (3, 2, 1000, 128), (5, 8, 4096, 512), (2, 4, 65536, 64)]:
        bases = None
        if not per_sequence_bases:
            x = to_bf16(np.ascontiguousarray(kv_like16(n_kv, 256, seed=1).transpose(1, 0, 2)), dev)
            b3, b4 = bases_from_hist(exponent_hist(x, n_kv), n_kv)
            bases = dict(k3=b3, k4=b4, v3=b3, v4=b4)
        c = CompressedKVCache(n_slots, n_kv, cap, bases=bases, ovf_bytes_per_tile=ovf)
        nbytes = lambda t: t.numel() * t.element_size()
        total = nbytes(c.S) + nbytes(c.tail_len)
        for st in (c.k, c.v):
            total += sum(nbytes(t) for t in (st.sm, st.codes, st.flags, st.tile_off, st.ovf, st.head_start, st.ovf_used, st.tail))
            if per_sequence_bases: total += nbytes(st.base3) + nbytes(st.base4)
        want = CompressedKVCache.bytes_per_slot(n_kv, cap, ovf, per_sequence_bases)
        assert total - 2 * 4 == n_slots * want, (n_slots, n_kv, cap, ovf)
        assert want == O.bytes_per_slot(n_kv, cap, ovf, per_sequence_bases)
