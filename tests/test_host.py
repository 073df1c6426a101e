"""CPU checks of the host side: the C-ABI library loads and exports every symbol the header declares, the ctypes table matches
the header's parameter lists, calls without a device fail loudly (no fallback), and the closed-form byte accounting."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gaac_hip.h")


def _declarations():
    """{name: [parameter type strings]} of every function declared in include/gaac_hip.h."""
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    out = {}
    for m in re.finditer(r"\b(?:int|const char\*)\s+(gaac_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        params = [p.strip() for p in m.group(2).replace("\n", " ").split(",")]
        out[m.group(1)] = [] if params == ["void"] else params
    return out


def test_library_exports_every_declared_symbol():
    from gaac_amd import _lib
    decl = _declarations()
    assert len(decl) >= 12 and "gaac_attn_launch" in decl and "gaac_cache_append" in decl
    assert os.path.exists(_lib.lib_path()), "build the library first: python -m gaac_amd.build"
    lib = ctypes.CDLL(_lib.lib_path())
    for name in decl:
        assert hasattr(lib, name), f"{name} is declared in include/gaac_hip.h but not exported"
    assert sorted(decl) == sorted(_lib.exported_symbols())


def test_ctypes_table_matches_the_header():
    from gaac_amd import _lib
    kind = {"int": ctypes.c_int, "long": ctypes.c_long, "float": ctypes.c_float}
    for name, params in _declarations().items():
        if name == "gaac_last_error": continue
        want = []
        for p in params:
            base = p.rsplit(" ", 1)[0].strip()
            want.append(ctypes.c_void_p if "*" in p else kind[base])
        assert _lib._SIGNATURES[name] == want, name


def test_every_entry_point_rejects_null_arguments_before_it_touches_a_device():
    """All-null, all-zero argument lists come back as -1 with a message on the calling thread: the argument checks stand in front
    of the first HIP call of every entry point.  (The two calls that only take a stream are left out: they do go to the device.)"""
    from gaac_amd import _lib
    lib = _lib.load()
    for name, args in _lib._SIGNATURES.items():
        if name in ("gaac_static_init", "gaac_static_reset"): continue
        zeros = [None if a is ctypes.c_void_p else (0.0 if a is ctypes.c_float else 0) for a in args]
        assert getattr(lib, name)(*zeros) == -1, name
        assert len(lib.gaac_last_error()) > 8, name


def test_no_device_no_fallback():
    """Without a GPU (or with CPU tensors) the product path raises instead of computing on the host."""
    from gaac_amd import Codec
    from gaac_amd.codec import exponent_hist
    x = torch.zeros(16, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        exponent_hist(x, 2)
    with pytest.raises(RuntimeError):
        Codec(2, "cpu").calibrate(torch.zeros(2, 16, 128, dtype=torch.bfloat16))


def test_product_code_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "gaac_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the test oracle"


def test_storage_index_is_a_bijection_and_perms_match_closed_forms():
    from gaac_amd.codec import storage_index, perm_k, perm_v
    for kind in ("k", "v"):
        sm, cd = storage_index(kind, "cpu")
        assert sorted(sm.tolist()) == list(range(2048)) and sorted(cd.tolist()) == list(range(768))
    pk, pv = perm_k().tolist(), perm_v().tolist()
    assert sorted(pk) == list(range(128)) and sorted(pv) == list(range(128))
    for j in range(4):
        for s in range(8):
            for q in range(4):
                assert pk[32 * j + 4 * s + q] == 16 * s + 2 * j + (0, 1, 8, 9)[q]
    for r in range(8):
        for n in range(16):
            assert pv[16 * r + n] == 8 * n + r


def test_choose_nsplit_bounds():
    from gaac_amd.kernel import choose_nsplit
    assert choose_nsplit(1, 8, 65536) == 32            # 256 blocks over 8 kv heads
    assert choose_nsplit(1, 8, 300) == 1               # never below 256 tokens per split
    assert choose_nsplit(64, 8, 65536) == 1
    assert choose_nsplit(1, 1, 1 << 20) == 256         # cap


def test_bytes_per_slot_closed_form():
    from gaac_amd.kv_cache import CompressedKVCache
    # 8 kv heads, capacity rounded to 65552 tokens, 128 B of escape room per tile, per-sequence bases: term by term
    cap = 65552; tiles = cap // 16
    head = cap * 128 + cap * 48 + cap * 4 + tiles * 4 + tiles * 128 + 8 + 4 + 4 + 16 * 128 * 2 + 2 * 128
    assert CompressedKVCache.bytes_per_slot(8, 65537) == 8 * (2 * head + 4 + 4)
    assert CompressedKVCache.bytes_per_slot(8, 65537, per_sequence_bases=False) == 8 * (2 * (head - 256) + 8)


def test_engine_context_and_attention_layer_without_a_cache():
    """The engine-shaped surface on the host (/root/reference/nanovllm/utils/context.py:5-31): the context is one module-level object
    with the reference's fields; an attention layer without a cache refuses to run instead of falling back to anything."""
    import dataclasses
    import torch
    from gaac_amd import serving
    names = [f.name for f in dataclasses.fields(serving.Context)]
    assert names == ["is_prefill", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k", "slot_mapping", "context_lens",
                     "block_tables", "kv_slots", "prefill_spans"]
    serving.set_context(True, max_seqlen_q=5, prefill_spans=[(1, 0, 5)])
    c = serving.get_context()
    assert c.is_prefill and c.max_seqlen_q == 5 and c.prefill_spans == [(1, 0, 5)] and c.kv_slots is None
    serving.reset_context()
    c = serving.get_context()
    assert not c.is_prefill and c.prefill_spans is None and c.max_seqlen_k == 0
    layer = serving.Attention(8, 128, 128 ** -0.5, 2)
    assert layer.gaac is None and layer.k_cache.numel() == 0
    q = torch.zeros(1, 8, 128, dtype=torch.bfloat16); k = torch.zeros(1, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no KV cache attached"):
        layer(q, k, k)
    with pytest.raises(AssertionError, match="head_dim"):
        serving.Attention(8, 64, 0.125, 2)
    # slots from a byte budget: the closed form of the cache, no device needed for the arithmetic
    from gaac_amd.kv_cache import CompressedKVCache
    per_slot = 4 * CompressedKVCache.bytes_per_slot(8, 4096)
    assert min(16, (3 * per_slot + 5) // per_slot) == 3
