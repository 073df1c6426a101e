"""Random operation sequences (fixed seeds) on the slot cache and on the paged pool, checked against the history kept on the host:
decoded contents bit-exact, attention within the reference's tolerance (/root/reference/tests/test_kernel.py:19) plus what the rounding
of the softmax weights to BF16 implies element by element (common.attention_error_bound): the kernel, like the reference's
(kernel.py:178-182), rounds the weights before the second product, and with values of opposite sign that nearly cancel that
rounding is not covered by a bound on |result|.  tests/golden/attention_cancellation_case.npz is such a case, found by these
generators: 40 tokens, values up to 4.9e4, results of magnitude 67, kernel output off by 1.46."""
import numpy as np
import pytest
import torch

from oracle import gaac_oracle as O
import os
from common import kv_like16, to_bf16, to_u16, attention_error_bound
from gpu_util import require_gpu

pytestmark = pytest.mark.gpu
SCALE = 128 ** -0.5


def _rows(rng, n, n_kv, outliers, scale_seed):
    sd = int(rng.integers(1 << 30))
    return (np.ascontiguousarray(kv_like16(n_kv, n, seed=sd, scale_seed=scale_seed, outliers=outliers).transpose(1, 0, 2)),
            np.ascontiguousarray(kv_like16(n_kv, n, seed=sd + 1, scale_seed=scale_seed + 1, outliers=outliers).transpose(1, 0, 2)))


def _close(got, q16, k16, v16):
    ref, tol = attention_error_bound(q16, k16, v16, SCALE)
    return bool((np.abs(got - ref) <= tol).all())


def test_the_cancellation_case_on_the_gpu():
    """The saved case through the slot cache, as it was found (prefill of 40 tokens, one kv head, two query heads)."""
    dev = require_gpu()
    from gaac_amd import CompressedKVCache
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_cancellation_case.npz"))
    q16, k16, v16 = d["q16"], d["k16"], d["v16"]
    cache = CompressedKVCache(n_slots=1, n_kv=1, capacity=64)
    cache.prefill(0, to_bf16(k16, dev), to_bf16(v16, dev))
    for ns in (None, 1, 2):
        out = O.bf16_to_f32(to_u16(cache.attention(to_bf16(q16, dev), torch.zeros(1, dtype=torch.int32, device=dev), SCALE, nsplit=ns)))
        assert _close(out[0], q16[0], k16, v16)


@pytest.mark.parametrize("seed", [2, 12])
def test_slot_cache_random_operations(seed):
    dev = require_gpu()
    from gaac_amd import CompressedKVCache
    from gaac_amd.codec import exponent_hist, bases_from_hist
    rng = np.random.default_rng(seed)
    for _ in range(25):
        n_kv = int(rng.choice([1, 2, 4, 8])); G = int(rng.choice([1, 2, 4, 8])); n_slots = int(rng.integers(1, 7)); cap = int(rng.choice([64, 256, 1024]))
        outl = float(rng.choice([0, 1e-3, 3e-2]))
        bases = None
        if rng.random() < 0.5:
            xs, xv = _rows(rng, 2048, n_kv, 1e-3, 4242)
            k3, k4 = bases_from_hist(exponent_hist(to_bf16(xs, dev), n_kv), n_kv); v3, v4 = bases_from_hist(exponent_hist(to_bf16(xv, dev), n_kv), n_kv)
            bases = dict(k3=k3, k4=k4, v3=v3, v4=v4)
        cache = CompressedKVCache(n_slots=n_slots, n_kv=n_kv, capacity=cap, bases=bases, ovf_bytes_per_tile=int(rng.choice([128, 512])))
        hist = {}
        for op in range(int(rng.integers(5, 40))):
            r = rng.random()
            if r < 0.25 or not hist:
                s = int(rng.integers(0, n_slots)); L = int(rng.integers(1, min(cap, 200)))
                k16, v16 = _rows(rng, L, n_kv, outl, 4242)
                cache.prefill(s, to_bf16(k16, dev), to_bf16(v16, dev)); hist[s] = (k16, v16)
            elif r < 0.8:
                live = [s for s in hist if len(hist[s][0]) < cap - 1]
                Bn = int(rng.integers(1, 6)); seen = set(); sl = []
                for _b in range(Bn):      # a slot at most once per step, some rows padded
                    s = int(rng.choice(live)) if live and rng.random() < 0.85 else -1
                    if s in seen: s = -1
                    seen.add(s); sl.append(s)
                k16, v16 = _rows(rng, Bn, n_kv, outl, 4242)
                cache.append(torch.tensor(sl, dtype=torch.int32, device=dev), to_bf16(k16, dev), to_bf16(v16, dev))
                for b, s in enumerate(sl):
                    if s >= 0: hist[s] = (np.concatenate([hist[s][0], k16[b:b + 1]]), np.concatenate([hist[s][1], v16[b:b + 1]]))
                if op % 8 == 0: cache.check_capacity()
            else:
                Bn = int(rng.integers(1, 5))
                sl = [int(rng.choice(list(hist))) if rng.random() < 0.85 else -1 for _b in range(Bn)]
                q16 = O.f32_to_bf16_rne((rng.standard_normal((Bn, n_kv * G, 128)) * 0.1).astype(np.float32))
                ns = None if rng.random() < 0.5 else int(rng.choice([1, 2, 5, 33]))
                out = O.bf16_to_f32(to_u16(cache.attention(to_bf16(q16, dev), torch.tensor(sl, dtype=torch.int32, device=dev), SCALE, nsplit=ns)))
                for b, s in enumerate(sl):
                    if s < 0: assert np.abs(out[b]).max() == 0
                    else: assert _close(out[b], q16[b], hist[s][0], hist[s][1]), (n_kv, G, s, len(hist[s][0]), ns)
        cache.check_capacity()
        for s in hist:
            dk, dv = cache.decompress(s)
            assert np.array_equal(to_u16(dk), hist[s][0]) and np.array_equal(to_u16(dv), hist[s][1]), (n_kv, s, len(hist[s][0]))
        assert cache.stats()["tokens"] == sum(len(h[0]) for h in hist.values())


@pytest.mark.parametrize("seed", [3, 13])
def test_paged_pool_random_operations(seed):
    dev = require_gpu()
    from gaac_amd.paged import LayerState, build_store_entries, choose_nsplit
    from gaac_amd.codec import exponent_hist, bases_from_hist
    rng = np.random.default_rng(seed)
    for _ in range(25):
        n_kv = int(rng.choice([1, 2, 4, 8])); G = int(rng.choice([1, 2, 4])); n_seq = int(rng.integers(1, 7)); max_blocks = int(rng.choice([8, 30, 70]))
        num_blocks = n_seq * max_blocks + int(rng.integers(0, 50)); ovf_slot = int(rng.choice([16, 64, 128])); outl = float(rng.choice([0, 1e-3, 2e-2]))
        raw_tiles = 2 * n_kv * n_seq + (num_blocks * 2 * n_kv if ovf_slot < 128 or outl > 1e-3 else num_blocks * 2 * n_kv // 4) + 8
        ck, cv = _rows(rng, 2048, n_kv, 1e-3, 77)
        k3, k4 = bases_from_hist(exponent_hist(to_bf16(ck, dev), n_kv), n_kv); v3, v4 = bases_from_hist(exponent_hist(to_bf16(cv, dev), n_kv), n_kv)
        st = LayerState(num_blocks, n_kv, raw_tiles, dict(k3=k3, k4=k4, v3=v3, v4=v4), ovf_slot, dev)
        buf = torch.zeros(LayerState.pool_bytes(num_blocks, n_kv, ovf_slot), dtype=torch.uint8, device=dev)
        bt_cpu = rng.permutation(num_blocks)[:n_seq * max_blocks].reshape(n_seq, max_blocks).astype(np.int32); bt = torch.from_numpy(bt_cpu).to(dev)
        empty = (np.zeros((0, n_kv, 128), np.uint16), np.zeros((0, n_kv, 128), np.uint16))
        lens = [0] * n_seq; hist = [empty for _s in range(n_seq)]
        cap = max_blocks * 16
        for op in range(int(rng.integers(4, 25))):
            r = rng.random()
            if r < 0.6:
                new = {}
                for s in sorted(set(int(x) for x in rng.integers(0, n_seq, int(rng.integers(1, n_seq + 1))))):
                    n = min(int(rng.choice([1, 1, 1, 5, 16, 40, 200])), cap - lens[s])
                    if n > 0: new[s] = _rows(rng, n, n_kv, outl, 77)
                if not new: continue
                seqs = sorted(new)
                ent = build_store_entries([lens[s] for s in seqs], [len(new[s][0]) for s in seqs], [bt_cpu[s] for s in seqs])
                st.store(to_bf16(np.concatenate([new[s][0] for s in seqs]), dev), to_bf16(np.concatenate([new[s][1] for s in seqs]), dev), buf,
                         torch.from_numpy(ent).to(dev))
                for s in seqs:
                    hist[s] = (np.concatenate([hist[s][0], new[s][0]]), np.concatenate([hist[s][1], new[s][1]])); lens[s] += len(new[s][0])
            elif r < 0.7:      # a sequence ends: its blocks are released and it starts over
                s = int(rng.integers(0, n_seq))
                if lens[s]:
                    st.release_blocks(torch.from_numpy(bt_cpu[s][:-(-lens[s] // 16)].copy()).to(dev))
                    lens[s] = 0; hist[s] = empty
            else:
                seqs = [int(x) for x in rng.permutation(n_seq)[:int(rng.integers(1, n_seq + 1))]]
                q16 = O.f32_to_bf16_rne((rng.standard_normal((len(seqs), n_kv * G, 128)) * 0.1).astype(np.float32))
                sl = torch.tensor([lens[s] for s in seqs], dtype=torch.int32, device=dev)
                ns = int(rng.choice([1, 2, 3, 9])) if rng.random() < 0.5 else choose_nsplit(len(seqs), n_kv, max(max(lens), 1))
                out = st.attention(to_bf16(q16, dev), buf, bt[torch.tensor(seqs, device=dev)].contiguous(), sl, ns, max_seq_len=max(max(lens), 1))
                got = O.bf16_to_f32(to_u16(out)).reshape(len(seqs), n_kv * G, 128)
                for b, s in enumerate(seqs):
                    if lens[s] == 0: assert np.abs(got[b]).max() == 0
                    else: assert _close(got[b], q16[b], hist[s][0], hist[s][1]), (n_kv, G, s, lens[s], ns)
        st.check()
        pairs, row, live = [], 0, [s for s in range(n_seq) if lens[s]]
        for s in live:
            for lb in range(-(-lens[s] // 16)):
                nv = min(16, lens[s] - 16 * lb); pairs.append((int(bt_cpu[s][lb]), row, nv)); row += nv
        if pairs:
            sk = torch.zeros(row, n_kv, 128, dtype=torch.bfloat16, device=dev); sv = torch.zeros_like(sk)
            st.decode_blocks(buf, torch.tensor(pairs, dtype=torch.int32, device=dev), sk, sv)
            assert np.array_equal(to_u16(sk), np.concatenate([hist[s][0] for s in live])), (n_kv, lens)
            assert np.array_equal(to_u16(sv), np.concatenate([hist[s][1] for s in live])), (n_kv, lens)
