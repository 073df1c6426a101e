"""GPU tests of the paged slot pool: store path (filling blocks stay raw, full blocks are compressed in their slot or stay raw when
their escapes do not fit), block decode (bit-exact) and decode attention through a permuted block table, against the history
kept on the host and the oracle's fp32 attention.  Tolerance of /root/reference/tests/test_kernel.py:19."""
import numpy as np
import pytest
import torch

from oracle import gaac_oracle as O
from common import kv_like16, to_bf16, to_u16, randn_bf16, attention_error_bound
from gpu_util import require_gpu

pytestmark = pytest.mark.gpu
N_KV, G = 4, 4
SCALE = 128 ** -0.5


def _tok16(x16):
    return np.ascontiguousarray(x16.transpose(1, 0, 2))


def _bases(dev, seed=30):
    from gaac_amd.codec import exponent_hist, bases_from_hist
    out = {}
    for name, sd, ss in (("k", seed, 2000), ("v", seed + 1, 2001)):
        x = to_bf16(_tok16(kv_like16(N_KV, 2048, seed=sd, scale_seed=ss)), dev)
        out[name + "3"], out[name + "4"] = bases_from_hist(exponent_hist(x, N_KV), N_KV)
    return out


class _Pool:
    """A little scheduler: block pool + permuted block table + per-sequence history on the host."""
    def __init__(self, dev, n_seq, max_blocks, num_blocks, raw_tiles, ovf_slot=128, seed=0):
        from gaac_amd.paged import LayerState
        self.dev = dev
        self.st = LayerState(num_blocks, N_KV, raw_tiles, _bases(dev), ovf_slot, dev)
        self.buf = torch.zeros(LayerState.pool_bytes(num_blocks, N_KV, ovf_slot), dtype=torch.uint8, device=dev)
        perm = np.random.default_rng(seed).permutation(num_blocks)[:n_seq * max_blocks].reshape(n_seq, max_blocks)
        self.bt_cpu = perm.astype(np.int32)
        self.bt = torch.from_numpy(self.bt_cpu).to(dev)
        self.lens = [0] * n_seq
        self.hist = [(np.zeros((0, N_KV, 128), np.uint16), np.zeros((0, N_KV, 128), np.uint16)) for _ in range(n_seq)]

    def step(self, new):
        """new: {seq: (k16 [n, n_kv, 128], v16)}; stores the rows and extends the history."""
        from gaac_amd.paged import build_store_entries
        seqs = sorted(new)
        ent = build_store_entries([self.lens[s] for s in seqs], [len(new[s][0]) for s in seqs], [self.bt_cpu[s] for s in seqs])
        k = to_bf16(np.concatenate([new[s][0] for s in seqs]), self.dev); v = to_bf16(np.concatenate([new[s][1] for s in seqs]), self.dev)
        self.st.store(k, v, self.buf, torch.from_numpy(ent).to(self.dev))
        for s in seqs:
            self.hist[s] = (np.concatenate([self.hist[s][0], new[s][0]]), np.concatenate([self.hist[s][1], new[s][1]]))
            self.lens[s] += len(new[s][0])

    def check(self, seqs, q16, nsplit=None):
        from gaac_amd.paged import choose_nsplit
        sl = torch.tensor([self.lens[s] for s in seqs], dtype=torch.int32, device=self.dev)
        bt = self.bt[torch.tensor(seqs, device=self.dev)].contiguous()
        ns = nsplit or choose_nsplit(len(seqs), N_KV, max(self.lens))
        out = self.st.attention(to_bf16(q16, self.dev), self.buf, bt, sl, ns, max_seq_len=max(max(self.lens), 1))
        got = O.bf16_to_f32(to_u16(out)).reshape(len(seqs), N_KV * G, 128)
        for b, s in enumerate(seqs):
            if self.lens[s] == 0:
                assert np.abs(got[b]).max() == 0
                continue
            ref = O.ref_attention(q16[b], self.hist[s][0], self.hist[s][1], SCALE)
            assert np.abs(got[b] - ref).max() <= 2e-2 * np.abs(ref).max() + 1e-3, (s, self.lens[s])
        self.check_decode(seqs)

    def check_decode(self, seqs):
        pairs, row = [], 0
        for s in seqs:
            for lb in range(-(-self.lens[s] // 16)):
                nv = min(16, self.lens[s] - 16 * lb)
                pairs.append((int(self.bt_cpu[s][lb]), row, nv)); row += nv
        if not pairs: return
        sk = torch.zeros(row, N_KV, 128, dtype=torch.bfloat16, device=self.dev); sv = torch.zeros_like(sk)
        self.st.decode_blocks(self.buf, torch.tensor(pairs, dtype=torch.int32, device=self.dev), sk, sv)
        wk = np.concatenate([self.hist[s][0] for s in seqs]); wv = np.concatenate([self.hist[s][1] for s in seqs])
        assert np.array_equal(to_u16(sk), wk) and np.array_equal(to_u16(sv), wv)


def _rows(n, seed):
    return _tok16(kv_like16(N_KV, n, seed=seed, scale_seed=2000)), _tok16(kv_like16(N_KV, n, seed=seed + 500, scale_seed=2001))


def test_prefill_then_decode_steps_through_a_permuted_block_table():
    dev = require_gpu()
    P = _Pool(dev, n_seq=4, max_blocks=40, num_blocks=200, raw_tiles=64)
    P.step({0: _rows(37, 1), 1: _rows(500, 2), 3: _rows(16, 3)})          # prompts (sequence 2 stays empty for now)
    P.check([1, 0, 3, 2], randn_bf16((4, N_KV * G, 128), seed=9, scale=0.1))
    compressed = int((P.st.mt >= 0).sum()); total = P.st.mt.numel()
    # sequences 0, 1 have one filling block each (2*n_kv raw tiles per block); every full block is compressed in place
    assert total - compressed == 2 * 2 * N_KV and int(P.st.top) == 64 - 2 * 2 * N_KV
    for step in range(36):
        live = [0, 1, 3] if step % 3 else [1, 3, 2]
        P.step({s: _rows(1, 1000 + 7 * step + s) for s in live})
        if step % 11 == 0 or step == 35:
            P.check([3, 2, 0, 1], randn_bf16((4, N_KV * G, 128), seed=200 + step, scale=0.1))
    P.st.check()
    # pops and pushes balance: the tiles off the stack are exactly the raw entries of the mode table, at least the filling blocks
    filling = sum(1 for L in P.lens if L % 16)
    n_raw = int((P.st.mt < 0).sum())
    assert int(P.st.top) == 64 - n_raw and n_raw >= filling * 2 * N_KV
    P.check([0, 1, 2, 3], randn_bf16((4, N_KV * G, 128), seed=77, scale=0.1), nsplit=1)
    P.check([0, 1, 2, 3], randn_bf16((4, N_KV * G, 128), seed=78, scale=0.1), nsplit=7)
    P.check([0, 1, 2, 3], randn_bf16((4, N_KV * G, 128), seed=79, scale=0.1), nsplit=20)      # 320 blocks: the four-wave block shape


def test_pool_beyond_4_gib_and_ragged_lengths_taken_longest_first():
    """A slot pool of 4.8 GB: most of the permuted block table points beyond 32-bit byte offsets.  Six sequences of very different
    lengths in an order that is neither ascending nor descending (the kernel takes them longest first; outputs stay in batch order)."""
    dev = require_gpu()
    P = _Pool(dev, n_seq=6, max_blocks=84, num_blocks=200_000, raw_tiles=128, seed=5)
    assert P.buf.numel() > (1 << 32) and int(P.bt_cpu.max()) * 2 * N_KV * P.st.TS > (1 << 32)
    lens = {0: 300, 1: 1270, 2: 16, 3: 777, 4: 1270, 5: 45}
    P.step({s: _rows(n, 40 + s) for s, n in lens.items()})
    P.check([0, 1, 2, 3, 4, 5], randn_bf16((6, N_KV * G, 128), seed=91, scale=0.1))
    P.check([5, 3, 1], randn_bf16((3, N_KV * G, 128), seed=92, scale=0.1), nsplit=3)
    for step in range(20):
        P.step({s: _rows(1, 3000 + 11 * step + s) for s in range(6)})
    P.check([2, 4, 0, 5, 1, 3], randn_bf16((6, N_KV * G, 128), seed=93, scale=0.1), nsplit=5)
    P.st.check()


def test_tiles_whose_escapes_do_not_fit_stay_raw_and_blocks_are_released():
    dev = require_gpu()
    P = _Pool(dev, n_seq=2, max_blocks=8, num_blocks=32, raw_tiles=72, ovf_slot=32)
    # sequence 0: ordinary rows (about 30 escape bytes per tile: some tiles fit the 32-byte slot, some do not);
    # sequence 1: exponents far from every base -> every group raw (1280 escape bytes per tile)
    rng = np.random.default_rng(3)
    k_far = (rng.integers(0, 2, (48, N_KV, 128)) << 15 | 95 << 7 | rng.integers(0, 128, (48, N_KV, 128))).astype(np.uint16)      # ~2^-32
    v_far = (rng.integers(0, 2, (48, N_KV, 128)) << 15 | 150 << 7 | rng.integers(0, 128, (48, N_KV, 128))).astype(np.uint16)     # ~2^23
    P.step({0: _rows(64, 5), 1: (k_far, v_far)})
    P.st.check()
    n_raw = int((P.st.mt < 0).sum())
    assert n_raw >= 3 * 2 * N_KV                                 # at least all of sequence 1
    assert int(P.st.top) == 72 - n_raw
    P.check([0, 1], randn_bf16((2, N_KV * G, 128), seed=5, scale=0.2), nsplit=2)
    # a mixed tile (K compressed, V raw or the other way round) must have occurred for the check above to cover that path
    mt = P.st.mt.cpu().numpy().reshape(-1, N_KV, 2)
    used = np.unique(P.bt_cpu[0][:4])
    mixed = sum(int((mt[b, h, 0] < 0) != (mt[b, h, 1] < 0)) for b in used for h in range(N_KV))
    assert mixed > 0, "no tile with exactly one raw side: pick another seed or slot size"
    # free sequence 1: its tiles return to the stack and its mode entries are reset
    blocks = torch.from_numpy(P.bt_cpu[1][:3].copy()).to(dev)
    P.st.release_blocks(blocks)
    torch.cuda.synchronize()
    mt1 = P.st.mt.cpu().numpy().reshape(-1, 2 * N_KV)
    for b in P.bt_cpu[1][:3]:
        assert np.array_equal(mt1[b], np.arange(b * 2 * N_KV, (b + 1) * 2 * N_KV))
    assert int(P.st.top) == 72 - int((P.st.mt < 0).sum())
    assert sorted(P.st.stack[:int(P.st.top)].cpu().tolist() + [int(~m) for m in P.st.mt.cpu().tolist() if m < 0]) == list(range(72))


def test_raw_pool_exhaustion_is_counted_not_written():
    dev = require_gpu()
    P = _Pool(dev, n_seq=2, max_blocks=4, num_blocks=8, raw_tiles=2 * N_KV)      # room for ONE filling block
    P.step({0: _rows(5, 1), 1: _rows(3, 2)})
    torch.cuda.synchronize()
    assert int(P.st.err) == 2 * N_KV and int(P.st.top) == 0
    with pytest.raises(RuntimeError, match="raw side pool exhausted"):
        P.st.check()


def test_full_tile_that_fits_nowhere_leaves_a_slot_that_is_safe_to_read():
    """A finished tile whose escape bytes exceed the slot, stored while the raw side pool is empty: the error counter goes up and the
    slot is marked compressed with stale content.  Its tag words must be zero (no escape bytes): the sizing pass had written the real
    ones, whose 1280 escape bytes would send a reader far past the slot, for the pool's last block past the allocation."""
    dev = require_gpu()
    from gaac_amd.paged import LayerState, build_store_entries
    num_blocks = 4
    st = LayerState(num_blocks, N_KV, 1, _bases(dev), 128, dev)
    buf = torch.zeros(LayerState.pool_bytes(num_blocks, N_KV, 128), dtype=torch.uint8, device=dev)
    st.top.zero_()                                          # an empty side pool
    rng = np.random.default_rng(5)
    k16 = (rng.integers(0, 1 << 16, (16, N_KV, 128)) & 0xBFFF).astype(np.uint16)      # random exponents: every group is raw
    v16 = (rng.integers(0, 1 << 16, (16, N_KV, 128)) & 0xBFFF).astype(np.uint16)
    last = num_blocks - 1
    ent = build_store_entries([0], [16], [np.array([last], np.int32)])
    st.store(to_bf16(k16, dev), to_bf16(v16, dev), buf, torch.from_numpy(ent).to(dev))
    torch.cuda.synchronize()
    assert int(st.err) == 2 * N_KV
    nt = 2 * N_KV
    mt = st.mt.cpu().numpy()
    assert np.array_equal(mt[last * nt:(last + 1) * nt], np.arange(last * nt, (last + 1) * nt))
    slots = buf[:num_blocks * nt * st.TS].view(num_blocks * nt, st.TS)[last * nt:(last + 1) * nt]
    assert int(slots[:, 2816:2880].max()) == 0              # tag words
    q = to_bf16(randn_bf16((1, N_KV * G, 128), seed=3, scale=0.1), dev)
    bt = torch.tensor([[last]], dtype=torch.int32, device=dev); sl = torch.tensor([16], dtype=torch.int32, device=dev)
    out = st.attention(q, buf, bt, sl, nsplit=1, max_seq_len=16)
    torch.cuda.synchronize()
    assert out.shape == (1, N_KV * G * 128)
    with pytest.raises(RuntimeError, match="raw side pool exhausted"):
        st.check()


def test_bad_arguments_raise():
    dev = require_gpu()
    from gaac_amd.paged import LayerState
    st = LayerState(8, N_KV, 8, _bases(dev), 128, dev)
    buf = torch.zeros(LayerState.pool_bytes(8, N_KV), dtype=torch.uint8, device=dev)
    q = torch.zeros(1, N_KV * G, 128, dtype=torch.bfloat16, device=dev)
    bt = torch.zeros(1, 2, dtype=torch.int32, device=dev); sl = torch.ones(1, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="max_seq_len"):
        st.attention(q, buf, bt, sl, nsplit=1, max_seq_len=16 * 3)       # more blocks than the table holds
    with pytest.raises(RuntimeError, match="GQA"):
        st.attention(torch.zeros(1, N_KV * 17, 128, dtype=torch.bfloat16, device=dev), buf, bt, sl, nsplit=1)


def test_escape_bytes_at_the_very_end_of_the_pools_last_slot():
    """The pool is exactly num_blocks * 2 * n_kv slots long (an engine's own block buffer has no slack behind it), and the attention kernel
    prefetches a lane's escape bytes as one 8-byte load: a tile whose escape bytes fill the slot's 128-byte room to within its last
    bytes, stored in the LAST slot of the pool (last block, last kv head, V; the K slot before it likewise), must be read without
    touching a byte behind the pool and decode right.  Lanes whose bytes start in the slot's last 7 bytes take the slow look-up."""
    dev = require_gpu()
    from gaac_amd.paged import LayerState, build_store_entries
    bases = _bases(dev)
    b = {k: v.cpu().numpy() for k, v in bases.items()}
    # rows whose last kv head carries, per kind, a tile with 124..128 escape bytes (4-bit and raw groups): a random subset of elements
    # is scaled by 8, the subset's density searched until the tile's byte count lands there
    def tile_with_full_slot(kind, seed0):
        for seed in range(seed0, seed0 + 2000):
            rng = np.random.default_rng(seed)
            x = kv_like16(N_KV, 16, seed=seed, outliers=0.0, scale_seed=2000 if kind == "k" else 2001)
            f = O.bf16_to_f32(x)
            hit = rng.random(f.shape) < rng.uniform(0.012, 0.03)
            x = O.f32_to_bf16_rne(np.where(hit, f * 8.0, f).astype(np.float32))
            tm = O.encode_token_major(x, kind, b[kind + "3"], b[kind + "4"], N_KV)
            nbytes = int(tm["row_bytes"][N_KV - 1].sum())
            if 124 <= nbytes <= 128: return x, nbytes
        raise AssertionError("no candidate tile found")
    xk, nk = tile_with_full_slot("k", 1000)
    xv, nv = tile_with_full_slot("v", 3000)
    num_blocks = 3
    st = LayerState(num_blocks, N_KV, 16, bases, 128, dev)
    buf = torch.zeros(LayerState.pool_bytes(num_blocks, N_KV, 128), dtype=torch.uint8, device=dev)
    assert buf.numel() == num_blocks * 2 * N_KV * 3008
    k0, v0 = _rows(16, 77)
    k16 = np.concatenate([k0, _tok16(xk)]); v16 = np.concatenate([v0, _tok16(xv)])      # [32, n_kv, 128]
    bt_cpu = np.array([[0, num_blocks - 1]], np.int32)
    st.store(to_bf16(k16, dev), to_bf16(v16, dev), buf, torch.from_numpy(build_store_entries([0], [32], bt_cpu)).to(dev))
    st.check()
    mt = st.mt.cpu().numpy()
    last = (num_blocks - 1) * 2 * N_KV
    assert mt[last + 2 * N_KV - 1] == last + 2 * N_KV - 1 and mt[last + 2 * N_KV - 2] == last + 2 * N_KV - 2      # compressed in their slots
    q16 = randn_bf16((1, N_KV * G, 128), seed=5, scale=0.05)
    bt = torch.from_numpy(bt_cpu).to(dev); sl = torch.tensor([32], dtype=torch.int32, device=dev)
    for ns in (1, 2):
        out = O.bf16_to_f32(to_u16(st.attention(to_bf16(q16, dev), buf, bt, sl, ns, max_seq_len=32))).reshape(N_KV * G, 128)
        ref, tol = attention_error_bound(q16[0], k16, v16, SCALE)
        assert (np.abs(out - ref) <= tol).all(), (ns, nk, nv)
    sk = torch.zeros(32, N_KV, 128, dtype=torch.bfloat16, device=dev); sv = torch.zeros_like(sk)
    st.decode_blocks(buf, torch.tensor([(0, 0, 16), (num_blocks - 1, 16, 16)], dtype=torch.int32, device=dev), sk, sv)
    assert np.array_equal(to_u16(sk), k16) and np.array_equal(to_u16(sv), v16)


def test_attention_launch_that_also_frees_equals_the_separate_free_launch():
    """LayerState.store(defer_free=True) leaves the raw tiles it gives back to the next attention launch (two launches per decode step
    instead of three).  Two pools go through the same prompts and 40 decode steps, one with the separate free launch, one deferring: after
    every step the same tiles are compressed or raw, the number of free tiles is the same and no raw tile is lost or handed out twice, the
    attention outputs are equal bit for bit, and a store that follows a deferred store without an attention in between pushes the queue itself."""
    dev = require_gpu()
    from gaac_amd.paged import build_store_entries
    pools = [_Pool(dev, n_seq=3, max_blocks=12, num_blocks=40, raw_tiles=40, seed=4) for _ in range(2)]
    def step(P, new, defer):
        seqs = sorted(new)
        ent = build_store_entries([P.lens[s] for s in seqs], [len(new[s][0]) for s in seqs], [P.bt_cpu[s] for s in seqs])
        k = to_bf16(np.concatenate([new[s][0] for s in seqs]), dev); v = to_bf16(np.concatenate([new[s][1] for s in seqs]), dev)
        P.st.store(k, v, P.buf, torch.from_numpy(ent).to(dev), defer_free=defer)
        for s in seqs:
            P.hist[s] = (np.concatenate([P.hist[s][0], new[s][0]]), np.concatenate([P.hist[s][1], new[s][1]]))
            P.lens[s] += len(new[s][0])
    def attend(P, q16):
        sl = torch.tensor(P.lens, dtype=torch.int32, device=dev)
        return to_u16(P.st.attention(to_bf16(q16, dev), P.buf, P.bt, sl, 2, max_seq_len=max(P.lens)))
    def same_state():
        a, b = pools
        ta, tb = int(a.st.top), int(b.st.top)
        ma, mb = a.st.mt.cpu().numpy(), b.st.mt.cpu().numpy()
        # the same tiles are compressed in place / raw (which raw tile a slot got depends on the order of the pushes)
        assert ta == tb and np.array_equal(ma >= 0, mb >= 0) and np.array_equal(ma[ma >= 0], mb[mb >= 0])
        for P, m, t in ((a, ma, ta), (b, mb, tb)):      # every raw tile is either in use exactly once or on the free stack exactly once
            assert sorted((~m[m < 0]).tolist() + P.st.stack[:t].tolist()) == list(range(P.st.raw.shape[0]))
    prompts = {0: _rows(30, 1), 1: _rows(47, 2), 2: _rows(15, 3)}
    for P, d in zip(pools, (False, True)): step(P, prompts, d)
    for P, d in zip(pools, (False, True)): step(P, {2: _rows(1, 4)}, d)      # sequence 2's block fills up; a second store in a row
    q16 = randn_bf16((3, N_KV * G, 128), seed=8, scale=0.1)
    assert np.array_equal(attend(pools[0], q16), attend(pools[1], q16))
    same_state()
    for t in range(40):
        new = {s: _rows(1, 100 + 3 * t + s) for s in range(3)}
        for P, d in zip(pools, (False, True)): step(P, new, d)
        assert pools[1].st._pending_free is not None and pools[0].st._pending_free is None
        q16 = randn_bf16((3, N_KV * G, 128), seed=300 + t, scale=0.1)
        assert np.array_equal(attend(pools[0], q16), attend(pools[1], q16))
        assert pools[1].st._pending_free is None
        same_state()
    pools[1].check([0, 1, 2], randn_bf16((3, N_KV * G, 128), seed=9, scale=0.1))
    for P in pools: P.st.check()
