"""Pins the CPU oracle (oracle/gaac_oracle.py) before anything is compared against it.

 * golden pages written by the reference's own codec (tests/golden/codec_{k,v}.npz) - field by field;
 * an independent scalar encoder/decoder written straight from the format rules (pure Python loops, token-major,
   no storage permutation) on small inputs;
 * closed forms: 11.25 / 12.25 / 16.25 bits per element, nbytes formula, worst-case tile, bijections;
 * brute force: tier rule over every exponent, sliding-window argmax with first-max tie break;
 * round trip over every class of bit pattern.
"""
import os
import numpy as np
import pytest

from oracle import gaac_oracle as O
from common import kv_like16, randn_bf16

GOLD = os.path.join(os.path.dirname(__file__), "golden")


# ------------------------------------------------------------------------------------------- golden (reference-made)
@pytest.mark.parametrize("kind", ["k", "v"])
def test_encode_matches_reference_golden(kind):
    g = np.load(os.path.join(GOLD, f"codec_{kind}.npz"))
    page = O.encode(g["x16"], kind, g["base3"], g["base4"], int(g["n_kv"]))
    for f in ("sm", "codes", "flags", "ovf_off", "ovf_head_start", "tile_off"):
        assert np.array_equal(getattr(page, f), g[f]), f
    n = int(g["ovf_head_start"][-1])
    assert np.array_equal(page.ovf[:n], g["ovf"][:n]) and page.ovf.size == g["ovf"].size
    assert O.page_nbytes(page.H, page.S, n) == int(g["nbytes"])
    # the fixture exercises all three tiers
    tags = np.stack([(g["flags"].astype(np.int64) >> (2 * i)) & 3 for i in range(16)], -1)
    assert (tags == 0).any() and (tags == 1).any() and (tags == 3).any() and not (tags == 2).any()


@pytest.mark.parametrize("kind", ["k", "v"])
def test_decode_matches_reference_golden(kind):
    g = np.load(os.path.join(GOLD, f"codec_{kind}.npz"))
    page = O.OPage(g["sm"], g["codes"], g["flags"], g["ovf_off"], g["ovf"], g["ovf_head_start"], g["tile_off"],
                   g["base3"], g["base4"], g["x16"].shape[0], g["x16"].shape[1], int(g["n_kv"]), kind)
    out = O.decode(page)
    assert np.array_equal(out, g["decoded"]) and np.array_equal(out, g["x16"])
    assert np.array_equal(O.row_offsets(g["flags"], page.S), g["ovf_off"])


@pytest.mark.parametrize("kind", ["k", "v"])
def test_torch_restatement_of_the_cpu_path_matches_the_golden_pages_and_the_numpy_oracle(kind):
    """oracle/gaac_oracle_torch.py (the CPU baseline bench.py times): decode_torch on the reference-written golden page gives the golden
    rows, also when cut into chunks that end inside a tile's run of rows; sdpa_torch equals the oracle's attention."""
    import torch
    from oracle.gaac_oracle_torch import decode_torch, sdpa_torch
    g = np.load(os.path.join(GOLD, f"codec_{kind}.npz"))
    page = O.OPage(g["sm"], g["codes"], g["flags"], g["ovf_off"], g["ovf"], g["ovf_head_start"], g["tile_off"],
                   g["base3"], g["base4"], g["x16"].shape[0], g["x16"].shape[1], int(g["n_kv"]), kind)
    for chunk in (8192, 16, 32):
        assert np.array_equal(decode_torch(page, chunk).numpy().view(np.uint16), g["decoded"])
    x = kv_like16(4, 333, seed=17)      # ragged length, all three tiers, per-head pooling h % n_kv
    b3, b4 = O.calibrate(x, 2)
    pg = O.encode(x, kind, b3, b4, 2)
    d = decode_torch(pg, 48)
    assert np.array_equal(d.numpy().view(np.uint16), x)
    q16 = randn_bf16((8, 128), seed=5, scale=0.3)
    want = O.ref_attention(q16, x.transpose(1, 0, 2), x.transpose(1, 0, 2), 128 ** -0.5)
    got = sdpa_torch(q16, d, d, 128 ** -0.5).numpy()
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max() + 1e-6


# ------------------------------------------------------------------------------------------- independent scalar codec
def scalar_encode_row(row16, chan_of_pos, b3, b4):
    """One token row by the format rules.  Returns (sm[128], code[128], tags[16], escapes bytes) in stored-position order."""
    sm, code, tags, esc = [], [], [], []
    for g in range(16):
        es, d3s, d4s = [], [], []
        for i in range(8):
            c = chan_of_pos[8 * g + i]
            x = int(row16[c])
            e = (x >> 7) & 0xFF
            sm.append(((x >> 8) & 0x80) | (x & 0x7F))
            es.append(e); d3s.append(e - int(b3[c])); d4s.append(e - int(b4[c]))
        if all(0 <= d < 8 for d in d3s):
            tags.append(0); code += d3s
        elif all(0 <= d < 16 for d in d4s):
            tags.append(1); code += [d & 7 for d in d4s]
            esc.append(sum(((d >> 3) & 1) << i for i, d in enumerate(d4s)))
        else:
            tags.append(3); code += [e & 7 for e in es]
            w = sum((e >> 3) << (5 * i) for i, e in enumerate(es))
            esc += [(w >> (8 * k)) & 0xFF for k in range(5)]
    return sm, code, tags, esc


def scalar_decode_row(sm, code, tags, esc, chan_of_pos, b3, b4):
    out = [0] * 128
    pos = 0
    for g in range(16):
        if tags[g] == 1:
            byte = esc[pos]; pos += 1
        elif tags[g] == 3:
            w = sum(esc[pos + k] << (8 * k) for k in range(5)); pos += 5
        for i in range(8):
            c = chan_of_pos[8 * g + i]
            if tags[g] == 0: e = int(b3[c]) + code[8 * g + i]
            elif tags[g] == 1: e = int(b4[c]) + code[8 * g + i] + 8 * ((byte >> i) & 1)
            else: e = code[8 * g + i] | (((w >> (5 * i)) & 31) << 3)
            s = sm[8 * g + i]
            out[c] = ((s & 0x80) << 8) | (e << 7) | (s & 0x7F)
    return out


@pytest.mark.parametrize("kind", ["k", "v"])
def test_oracle_vs_scalar_codec(kind):
    n_kv, H, S = 2, 4, 21
    x16 = kv_like16(H, S, seed=5, outliers=5e-3, scale_seed=11)
    b3, b4 = O.calibrate(kv_like16(H, 128, seed=6, scale_seed=11), n_kv)
    tm = O.encode_token_major(x16, kind, b3, b4, n_kv)
    chan = O.perm(kind)
    seen = set()
    for h in range(H):
        esc_all = []
        for s in range(S):
            sm, code, tags, esc = scalar_encode_row(x16[h, s], chan, b3[h % n_kv], b4[h % n_kv])
            assert list(tm["sm"][h, s]) == sm
            bits = np.unpackbits(tm["codes"][h, s], bitorder="little")
            assert [int(bits[3 * i] | (bits[3 * i + 1] << 1) | (bits[3 * i + 2] << 2)) for i in range(128)] == code
            assert [int((int(tm["flags"][h, s]) >> (2 * g)) & 3) for g in range(16)] == tags
            assert int(tm["row_bytes"][h, s]) == len(esc)
            assert scalar_decode_row(sm, code, tags, esc, chan, b3[h % n_kv], b4[h % n_kv]) == list(x16[h, s])
            esc_all += esc; seen |= set(tags)
        assert list(tm["esc"][h]) == esc_all
    assert seen == {0, 1, 3}
    assert np.array_equal(O.decode(O.encode(x16, kind, b3, b4, n_kv)), x16)


# ------------------------------------------------------------------------------------------- closed forms / invariants
def test_perms_and_storage_index_are_bijections_with_the_documented_closed_forms():
    pk, pv = O.perm_k(), O.perm_v()
    assert sorted(pk) == list(range(128)) and sorted(pv) == list(range(128))
    assert [int(pk[32 * 1 + 4 * 2 + q]) for q in range(4)] == [34, 35, 42, 43]      # dim 16s+2j+(0,1,8,9), j=1, s=2
    assert int(pv[16 * 3 + 5]) == 8 * 5 + 3
    # group membership that fixes the tier shares: K group g = channels 32(g%4)+2(g//4)+{0,1,8,9,16,17,24,25}
    for g in range(16):
        assert sorted(pk[8 * g:8 * g + 8]) == sorted(32 * (g % 4) + 2 * (g // 4) + o for o in (0, 1, 8, 9, 16, 17, 24, 25))
        assert sorted(pv[8 * g:8 * g + 8]) == [64 * (g % 2) + (g // 2) + 8 * i for i in range(8)]
    for kind in ("k", "v"):
        si, ci = O.storage_index(kind)
        assert sorted(si) == list(range(2048)) and sorted(ci) == list(range(768))
    si, ci = O.storage_index("k")
    assert int(si[1024 + 32 * 5 + 3]) == (8 + 1) * 128 + 32 * 1 + 3 and int(ci[384 + 12 * 5 + 2]) == 9 * 48 + 12 * 1 + 2
    si, ci = O.storage_index("v")      # lane 6: j=2, r=1 -> tokens 4,5,12,13; second token block starts at byte 16
    assert int(si[64 * 6 + 16]) == 5 * 128 + 16 * 1 and int(ci[24 * 6 + 6]) == 5 * 48 + 6 * 1


def test_bits_per_element_closed_forms():
    """One tile where every group has the same tier costs 11.25 / 12.25 / 16.25 bits per element."""
    b3 = np.full((1, 128), 120, np.uint8); b4 = np.full((1, 128), 116, np.uint8)
    for exp, bits in ((123, 11.25), (117, 12.25), (200, 16.25)):
        x16 = np.full((1, 16, 128), exp << 7, dtype=np.uint16)
        page = O.encode(x16, "k", b3, b4, 1)
        esc = int(page.ovf_head_start[-1])
        tile_bytes = 2048 + 768 + 64 + esc          # tile offset word excluded, as in the published figure
        assert tile_bytes * 8 / 2048 == bits
        assert O.page_nbytes(1, 16, esc) == tile_bytes + 4
    assert O.TILE_MAX_ESC == 1280 and esc == 1280


def test_tier_rule_brute_force_every_exponent():
    """Single varying element in an otherwise in-window group, all 256 exponents x a few bases."""
    for b3v, b4v in ((120, 116), (0, 0), (248, 240), (100, 110), (130, 120)):
        b3 = np.full((1, 128), b3v, np.uint8); b4 = np.full((1, 128), b4v, np.uint8)
        inside = max(b3v, b4v)
        ok_fill = (0 <= inside - b3v < 8) and (0 <= inside - b4v < 16)
        x16 = np.full((1, 256, 128), inside << 7, dtype=np.uint16)
        x16[0, :, 0] = (np.arange(256) << 7).astype(np.uint16)       # channel 0 sits in K group 0
        page = O.encode(x16, "k", b3, b4, 1)
        tag0 = page.flags[0, :256] & 3
        for e in range(256):
            fit3 = ok_fill and 0 <= e - b3v < 8 and 0 <= inside - b3v < 8
            fit4 = 0 <= e - b4v < 16 and 0 <= inside - b4v < 16
            want = 0 if fit3 else (1 if fit4 else 3)
            assert int(tag0[e]) == want, (b3v, b4v, e)
        assert set(np.unique((page.flags[:, :, None] >> (2 * np.arange(16))) & 3)) <= {0, 1, 3}
        assert np.array_equal(O.decode(page), x16)


def test_round_trip_every_bit_pattern():
    """All 65536 BF16 bit patterns (NaN, Inf, denormals, -0 included) survive encode -> decode."""
    x16 = np.arange(65536, dtype=np.uint16).reshape(4, 128, 128)
    rng = np.random.default_rng(0)
    x16 = rng.permuted(x16.reshape(-1)).reshape(4, 128, 128)
    b3, b4 = O.calibrate(x16, 4)
    for kind in ("k", "v"):
        page = O.encode(x16, kind, b3, b4, 4)
        assert np.array_equal(O.decode(page), x16)


def test_adversarial_size_bound():
    """/root/reference/tests/test_codec.py:22-29: random bit patterns never cost more than raw + metadata."""
    rng = np.random.default_rng(1)
    x = rng.integers(-32768, 32767, (4, 256, 128)).astype(np.int16)
    x = np.where(((x >> 7) & 0xFF) == 0xFF, x & ~0x4000, x).astype(np.int16).view(np.uint16)
    b3, b4 = O.calibrate(x, 4)
    page = O.encode(x, "k", b3, b4, 4)
    assert np.array_equal(O.decode(page), x)
    assert O.page_nbytes(4, 256, int(page.ovf_head_start[-1])) <= x.size * 2 + 4 * 256 * 5


def test_bases_from_hist_brute_force_and_ties():
    rng = np.random.default_rng(2)
    hist = rng.integers(0, 50, (2 * 128, 256)).astype(np.int64)
    hist[0] = 0; hist[0, 10:18] = 5; hist[0, 100:108] = 5          # tie -> lowest start
    hist[1] = 0                                                     # empty row -> 0
    hist[2] = 0; hist[2, 250:256] = 9                               # window clamps at the top of the range
    b3, b4 = O.bases_from_hist(hist, 2)
    for r in range(256):
        for w, got in ((8, b3), (16, b4)):
            sums = [int(hist[r, s:s + w].sum()) for s in range(256 - w + 1)]
            assert int(got.reshape(-1)[r]) == sums.index(max(sums))
    assert int(b3[0, 0]) == 10 and int(b3[0, 1]) == 0 and int(b3[0, 2]) == 248 and int(b4[0, 2]) == 240


def test_exponent_hist_and_calibrate_pooling():
    x16 = kv_like16(6, 50, seed=3)                                  # heads 0..5, n_kv = 3: head h pools into h % 3
    hist = O.exponent_hist(x16.reshape(2, 3, 50, 128).transpose(0, 2, 1, 3), 3)
    for kvh in range(3):
        for c in (0, 17, 127):
            e = np.concatenate([(x16[kvh, :, c] >> 7) & 0xFF, (x16[kvh + 3, :, c] >> 7) & 0xFF])
            assert np.array_equal(hist[kvh * 128 + c], np.bincount(e, minlength=256))
    assert hist.sum() == x16.size
    b3, b4 = O.calibrate(x16, 3)
    b3b, b4b = O.bases_from_hist(hist, 3)
    assert np.array_equal(b3, b3b) and np.array_equal(b4, b4b)


def test_row_and_tile_offsets():
    x16 = kv_like16(2, 100, seed=4, outliers=1e-2)
    b3, b4 = O.calibrate(x16, 2)
    page = O.encode(x16, "v", b3, b4, 2)
    tags = np.stack([(page.flags[:, :100].astype(np.int64) >> (2 * g)) & 3 for g in range(16)], -1)
    rb = (tags == 1).sum(-1) + 5 * (tags == 3).sum(-1)
    assert np.array_equal(page.ovf_off, np.cumsum(rb, 1) - rb)
    assert np.array_equal(O.row_offsets(page.flags, 100), page.ovf_off)
    assert np.array_equal(page.tile_off, page.ovf_off[:, ::16])
    assert np.array_equal(np.diff(page.ovf_head_start), rb.sum(1))
    assert page.sm.shape == (2, 112 * 128) and not page.flags[:, 100:].any()
    # padded rows are stored as zeros
    si, _ = O.storage_index("v")
    sm_tm = np.empty(16 * 128, np.uint8); sm_tm[si] = page.sm[0, 6 * 2048:]
    assert not sm_tm.reshape(16, 128)[4:].any()


def test_ref_attention_against_explicit_float64_loops():
    rng = np.random.default_rng(5)
    n_q, n_kv, L = 6, 2, 37
    q16 = O.f32_to_bf16_rne((rng.standard_normal((n_q, 128)) * 0.3).astype(np.float32))
    k16 = O.f32_to_bf16_rne(rng.standard_normal((L, n_kv, 128)).astype(np.float32))
    v16 = O.f32_to_bf16_rne(rng.standard_normal((L, n_kv, 128)).astype(np.float32))
    out = O.ref_attention(q16, k16, v16, 0.125)
    q, k, v = (O.bf16_to_f32(a).astype(np.float64) for a in (q16, k16, v16))
    for j in range(n_q):
        h = j // 3
        s = np.array([sum(q[j, d] * k[t, h, d] for d in range(128)) * 0.125 for t in range(L)])
        p = np.exp(s - s.max()); p /= p.sum()
        ref = sum(p[t] * v[t, h] for t in range(L))
        assert np.abs(out[j] - ref).max() < 1e-5
    # special cases: q = 0 -> mean of V; all V rows equal -> that row
    z = O.ref_attention(np.zeros_like(q16), k16, v16, 0.125)
    assert np.abs(z[0] - O.bf16_to_f32(v16[:, 0]).mean(0)).max() < 1e-5
    vc = np.broadcast_to(v16[:1], v16.shape)
    assert np.abs(O.ref_attention(q16, k16, vc, 0.125)[4] - O.bf16_to_f32(v16[0, 1])).max() < 1e-5


def test_bf16_helpers():
    x = np.array([1.0, -2.5, 3.1415927, 1e-40, 65504.0, 1.00390625, 1.01171875], dtype=np.float32)
    import torch
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_rne(x), want)
    assert np.array_equal(O.bf16_to_f32(want), torch.from_numpy(want.view(np.int16)).view(torch.bfloat16).float().numpy())


def test_byte_accounting_closed_forms():
    assert O.bytes_per_slot(8, 1000, 128, True) == 2 * 8 * (1008 * 180 + 63 * 4 + 63 * 128 + 16 + 16 * 256 + 256) + 64
    st = O.cache_stats(S_sum=64, tail_sum=8, esc=10, n_kv=4)
    assert st["bytes_used"] == 2 * (64 * 180 + 16 + 8 * 256) + 10 and st["bf16_bytes"] == 72 * 512 and st["tokens"] == 18
    assert O.slot_fits(128) and not O.slot_fits(129) and O.OVF_OFF + 128 == 3008


def test_attention_error_bound_covers_the_saved_cancellation_case():
    """tests/golden/attention_cancellation_case.npz: a kernel output (rounded softmax weights) that the reference's tolerance alone
    rejects (error 1.46 at |ref| <= 67) and that the elementwise bound of common.attention_error_bound accepts, while a result that is
    off by a few percent of the attended values is still rejected."""
    import os
    from common import attention_error_bound
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_cancellation_case.npz"))
    q16, k16, v16, out = d["q16"][0], d["k16"], d["v16"], d["out"][0]
    ref, tol = attention_error_bound(q16, k16, v16, 128 ** -0.5)
    err = np.abs(out - ref)
    assert err.max() > 2e-2 * np.abs(ref).max() + 1e-3          # the reference's tolerance alone does not cover it
    assert (err <= tol).all()
    assert tol.max() < 2.0 ** -7 * np.abs(O.bf16_to_f32(v16)).max() / 4      # far tighter than a bound by the largest value
    rnd = tol - (2e-2 * np.abs(ref).max() + 1e-3)
    assert not (np.abs((ref + 8 * rnd + 0.1 * np.abs(ref).max()) - ref) <= tol).all()
