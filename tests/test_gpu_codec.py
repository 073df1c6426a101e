"""GPU parity of the codec path against the CPU oracle: calibration, HIP tile encoder, HIP decoder.
Mirrors /root/reference/tests/test_codec.py (field-by-field encoder parity, bit-exact round trip, adversarial input)."""
import os
import numpy as np
import pytest
import torch

from oracle import gaac_oracle as O
from common import kv_like16, to_bf16, to_u16
from gpu_util import require_gpu, native_to_reference_page, assert_pages_equal

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def test_calibration_matches_oracle():
    dev = require_gpu()
    from gaac_amd.codec import Codec, exponent_hist, bases_from_hist
    n_kv = 4
    x16 = kv_like16(2 * n_kv, 300, seed=1)
    want3, want4 = O.calibrate(x16, n_kv)
    c = Codec(n_kv).calibrate(to_bf16(x16))
    assert np.array_equal(c.base3.cpu().numpy(), want3) and np.array_equal(c.base4.cpu().numpy(), want4)
    tm = x16.reshape(2, n_kv, 300, 128).transpose(0, 2, 1, 3)
    hist = exponent_hist(to_bf16(np.ascontiguousarray(tm), dev), n_kv)
    assert hist.dtype == torch.int64 and np.array_equal(hist.cpu().numpy(), O.exponent_hist(tm, n_kv))
    # ties, empty rows and the clamp at the top of the exponent range
    h = np.zeros((n_kv * 128, 256), np.int64); h[0, 10:18] = 5; h[0, 100:108] = 5; h[2, 250:256] = 9
    rng = np.random.default_rng(0); h[3:] = rng.integers(0, 1 << 40, (n_kv * 128 - 3, 256))
    b3, b4 = bases_from_hist(torch.from_numpy(h).to(dev), n_kv)
    w3, w4 = O.bases_from_hist(h, n_kv)
    assert np.array_equal(b3.cpu().numpy(), w3) and np.array_equal(b4.cpu().numpy(), w4)


@pytest.mark.parametrize("kind", ["k", "v"])
@pytest.mark.parametrize("S", [16, 100, 1024])
def test_hip_encoder_matches_oracle_and_roundtrips(kind, S):
    dev = require_gpu()
    from gaac_amd import Codec, TileEncoder
    n_kv = 4
    calib16, x16 = kv_like16(2 * n_kv, 2048, seed=1, scale_seed=9), kv_like16(2 * n_kv, S, seed=2, scale_seed=9)
    b3, b4 = O.calibrate(calib16, n_kv)
    ref = O.encode(x16, kind, b3, b4, n_kv)
    codec = Codec(n_kv).calibrate(to_bf16(calib16))
    x = to_bf16(x16, dev)
    for page in (TileEncoder(kind).encode(codec, x), codec.encode(x, kind)):
        assert_pages_equal(native_to_reference_page(page), ref)
        assert page.nbytes == O.page_nbytes(ref.H, ref.S, int(ref.ovf_head_start[-1]))
        assert np.array_equal(to_u16(Codec.decode(page)), x16)
    tags = np.stack([(ref.flags.astype(np.int64) >> (2 * g)) & 3 for g in range(16)], -1)
    if S >= 100: assert (tags == 1).any() and (tags == 3).any()


@pytest.mark.parametrize("kind", ["k", "v"])
def test_golden_pages_from_the_reference(kind):
    """Pages the reference codec itself wrote: the HIP encoder reproduces them (after the documented byte re-ordering)
    and the HIP decoder returns the reference decoder's output."""
    dev = require_gpu()
    from gaac_amd import Codec, TileEncoder
    g = np.load(os.path.join(GOLD, f"codec_{kind}.npz"))
    n_kv = int(g["n_kv"])
    codec = Codec(n_kv).set_bases(torch.from_numpy(g["base3"]), torch.from_numpy(g["base4"]))
    page = TileEncoder(kind).encode(codec, to_bf16(g["x16"], dev))
    got = native_to_reference_page(page)
    for f in ("sm", "codes", "flags", "ovf_off", "ovf_head_start", "tile_off"):
        assert np.array_equal(getattr(got, f), g[f]), f
    n = int(g["ovf_head_start"][-1])
    assert np.array_equal(got.ovf[:n], g["ovf"][:n]) and page.nbytes == int(g["nbytes"])
    assert np.array_equal(to_u16(Codec.decode(page)), g["decoded"])


def test_adversarial_never_expands_beyond_raw():
    """/root/reference/tests/test_codec.py:22-29."""
    dev = require_gpu()
    from gaac_amd import Codec, TileEncoder
    rng = np.random.default_rng(1)
    x = rng.integers(-32768, 32767, (4, 256, 128)).astype(np.int16)
    x16 = np.where(((x >> 7) & 0xFF) == 0xFF, x & ~0x4000, x).astype(np.int16).view(np.uint16)
    xt = to_bf16(x16, dev)
    codec = Codec(4).calibrate(xt)
    for kind in ("k", "v"):
        page = TileEncoder(kind).encode(codec, xt)
        assert np.array_equal(to_u16(Codec.decode(page)), x16)
        assert page.nbytes <= x16.size * 2 + 4 * 256 * 5
        b3, b4 = O.calibrate(x16, 4)
        assert_pages_equal(native_to_reference_page(page), O.encode(x16, kind, b3, b4, 4))


def test_every_bit_pattern_round_trips():
    dev = require_gpu()
    from gaac_amd import Codec, TileEncoder
    x16 = np.random.default_rng(0).permuted(np.arange(65536, dtype=np.uint16)).reshape(4, 128, 128)
    xt = to_bf16(x16, dev)
    codec = Codec(4).calibrate(xt)
    for kind in ("k", "v"):
        assert np.array_equal(to_u16(Codec.decode(TileEncoder(kind).encode(codec, xt))), x16)


def test_row_offsets_matches_oracle():
    dev = require_gpu()
    from gaac_amd.codec import row_offsets
    rng = np.random.default_rng(3)
    tags = rng.choice([0, 1, 3], size=(3, 700, 16), p=[0.8, 0.15, 0.05]).astype(np.int64)
    flags = (tags << (2 * np.arange(16))).sum(-1).astype(np.uint32).view(np.int32)
    got = row_offsets(torch.from_numpy(flags).to(dev), 690)
    assert np.array_equal(got.cpu().numpy(), O.row_offsets(flags, 690))


def test_row_offsets_over_many_chunks_and_a_ragged_end():
    """The two-pass scan: several 2048-row chunks per head, a last chunk that is partly filled, S < S_pad."""
    dev = require_gpu()
    from gaac_amd.codec import row_offsets
    rng = np.random.default_rng(4)
    for S_pad, S in ((2048 * 3 + 16, 2048 * 3 + 5), (2048, 2048), (4096 + 2048, 4097)):
        tags = rng.choice([0, 1, 3], size=(2, S_pad, 16), p=[0.7, 0.2, 0.1]).astype(np.int64)
        flags = (tags << (2 * np.arange(16))).sum(-1).astype(np.uint32).view(np.int32)
        got = row_offsets(torch.from_numpy(flags).to(dev), S)
        assert np.array_equal(got.cpu().numpy(), O.row_offsets(flags, S)), (S_pad, S)


def test_histogram_over_several_token_chunks():
    """More tokens than one block's chunk, a token count that no loop stride divides, every exponent value present."""
    dev = require_gpu()
    from gaac_amd.codec import exponent_hist
    n_kv, n_tok = 2, 5000 + 77
    rng = np.random.default_rng(5)
    x16 = rng.integers(0, 1 << 16, (n_tok, n_kv, 128), dtype=np.uint16)
    hist = exponent_hist(to_bf16(x16, dev), n_kv)
    assert np.array_equal(hist.cpu().numpy(), O.exponent_hist(x16, n_kv))
    assert int(hist.sum()) == n_tok * n_kv * 128


@pytest.mark.parametrize("kind", ["k", "v"])
def test_encoder_reads_a_token_major_prompt_through_strides(kind):
    """encode_tiles takes head and row strides: a transposed view of [L, n_kv, 128] encodes like its head-major copy; the page spans
    several 16-tile blocks of the encoder with a partly filled last block and a partly filled last tile."""
    dev = require_gpu()
    from gaac_amd import Codec, TileEncoder
    n_kv, L = 3, 16 * 37 + 9
    x16 = kv_like16(n_kv, L, seed=21)
    tm = to_bf16(np.ascontiguousarray(x16.transpose(1, 0, 2)), dev)          # [L, n_kv, 128]
    view = tm.transpose(0, 1)
    assert not view.is_contiguous()
    codec = Codec(n_kv).calibrate(view[:, :200])
    b3, b4 = O.calibrate(x16[:, :200], n_kv)
    assert np.array_equal(codec.base3.cpu().numpy(), b3)
    enc = TileEncoder(kind)
    page_v, page_c = enc.encode(codec, view), enc.encode(codec, view.contiguous())
    for f in ("sm", "codes", "flags", "ovf_off", "ovf", "ovf_head_start", "tile_off"):
        assert torch.equal(getattr(page_v, f), getattr(page_c, f)), f
    assert_pages_equal(native_to_reference_page(page_v), O.encode(x16, kind, b3, b4, n_kv))
    assert np.array_equal(to_u16(Codec.decode(page_v)), x16)


def test_base_collector_accumulates_over_steps_and_round_trips_its_file(tmp_path):
    """BaseCollector (calibration.py of the reference): histograms add up over prefill steps; bases equal the oracle's on the
    concatenated tokens; the saved file holds {layer: {k3,k4,v3,v4}} uint8 [n_kv,128] CPU tables and loads with weights_only."""
    dev = require_gpu()
    from gaac_amd import BaseCollector
    from gaac_amd.calibration import load_bases
    n_kv = 2
    col = BaseCollector()
    parts = {0: [], 1: []}
    for step in range(3):
        for layer in (0, 1):
            k16 = np.ascontiguousarray(kv_like16(n_kv, 100 + 37 * step, seed=10 * step + layer).transpose(1, 0, 2))
            v16 = np.ascontiguousarray(kv_like16(n_kv, 100 + 37 * step, seed=50 + 10 * step + layer).transpose(1, 0, 2))
            col.observe(layer, to_bf16(k16, dev), to_bf16(v16, dev)); parts[layer].append((k16, v16))
    path = str(tmp_path / "bases.pt")
    assert col.save(path) == 2
    tables = load_bases(path)
    assert sorted(tables) == [0, 1]
    for layer in (0, 1):
        kall = np.concatenate([p[0] for p in parts[layer]]); vall = np.concatenate([p[1] for p in parts[layer]])
        k3, k4 = O.bases_from_hist(O.exponent_hist(kall, n_kv), n_kv); v3, v4 = O.bases_from_hist(O.exponent_hist(vall, n_kv), n_kv)
        t = tables[layer]
        assert all(t[n].dtype == torch.uint8 and tuple(t[n].shape) == (n_kv, 128) and not t[n].is_cuda for n in ("k3", "k4", "v3", "v4"))
        assert np.array_equal(t["k3"].numpy(), k3) and np.array_equal(t["k4"].numpy(), k4)
        assert np.array_equal(t["v3"].numpy(), v3) and np.array_equal(t["v4"].numpy(), v4)


def test_config_0_recipe_equals_the_oracle():
    """Config 0 as BASELINE.json words it (the reference's own CPU-runnable case, /root/reference/tests/test_codec.py:6-19 and
    examples/compress_decompress.py:23-26): K [8 kv heads, 4096 tokens, 128] seed 0, element = N(0,1) * sigma_c with sigma_c log-uniform
    in [2^-4, 2^4], with probability 0.002 per 8-element group one element x 2^12, bases from the first 1024 tokens, encoded as 16-token
    tiles and decoded.  Bases, every page field, the page size, the tier shares and the decoded rows equal the CPU oracle's."""
    dev = require_gpu()
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    from bench import make_kv, tier_shares
    from gaac_amd import Codec, TileEncoder
    x = make_kv(0, 8, 4096)
    x16 = to_u16(x)
    xd = x.to(dev)
    codec = Codec(8, dev).calibrate(xd[:, :1024])
    b3, b4 = O.calibrate(x16[:, :1024], 8)
    assert np.array_equal(codec.base3.cpu().numpy(), b3) and np.array_equal(codec.base4.cpu().numpy(), b4)
    page = TileEncoder("k", dev).encode(codec, xd)
    want = O.encode(x16, "k", b3, b4, 8)
    assert_pages_equal(native_to_reference_page(page), want)
    n_esc = int(want.ovf_head_start[-1])
    assert page.nbytes == O.page_nbytes(8, 4096, n_esc) and abs(page.ratio - 8 * 4096 * 256 / page.nbytes) < 1e-12
    assert 1.39 < page.ratio < 1.42
    s3, s4, sr = tier_shares(page)
    tags = np.stack([(want.flags.astype(np.int64) >> (2 * g)) & 3 for g in range(16)], -1)
    assert abs(s4 - (tags == 1).mean()) < 1e-12 and abs(sr - (tags == 3).mean()) < 1e-12 and 0.85 < s3 < 0.93 and 0.001 < sr < 0.006
    back = to_u16(Codec.decode(page))
    assert np.array_equal(back, x16) and np.array_equal(O.decode(want), x16)
