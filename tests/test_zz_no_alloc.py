"""The entry point that allocates nothing (gaac_attn_fused_static: workspace in a device array built into the library) against
gaac_attn_fused with caller memory, through the C-ABI: same kernel, same arithmetic, so the outputs are equal bit for bit.  Two calls
in a row, the second with a smaller input (fewer rows, heads, tokens and splits), then the first again; launches beyond the built-in
workspace are rejected.  gaac_static_init resolves the array's address ahead of a capture, gaac_static_flags copies its failure bits
out, gaac_static_reset re-arms it (by a kernel), and a captured call replays right."""
import numpy as np
import pytest
import torch

from common import kv_like16, to_bf16, randn_bf16
from gpu_util import require_gpu

pytestmark = pytest.mark.gpu
SCALE = 128 ** -0.5


def _case(dev, B, n_kv, G, S, ns, seed, tail):
    from gaac_amd import Codec, TileEncoder
    from gaac_amd.kernel import AttnWorkspace, _store_args
    k = to_bf16(kv_like16(B * n_kv, S, seed=seed), dev); v = to_bf16(kv_like16(B * n_kv, S, seed=seed + 1), dev)
    kp = TileEncoder("k").encode(Codec(n_kv).calibrate(k), k); vp = TileEncoder("v").encode(Codec(n_kv).calibrate(v), v)
    n_q = n_kv * G
    q = to_bf16(randn_bf16((B * n_q, 128), seed=seed + 2, scale=0.3), dev)
    SL = torch.full((B * n_kv,), S, dtype=torch.int32, device=dev)
    kt = to_bf16(kv_like16(B * n_kv, 16, seed=seed + 3), dev); vt = to_bf16(kv_like16(B * n_kv, 16, seed=seed + 4), dev)
    TL = torch.full((B * n_kv,), tail, dtype=torch.int32, device=dev)
    ws = AttnWorkspace(B * n_q, ns, torch.bfloat16, dev)
    common = (*_store_args(kp), *_store_args(vp), q.data_ptr(), None, B, n_q, n_kv, SL.data_ptr(), kp.sm.shape[1] // 128, SCALE, ns, kp.base3.shape[0],
              kt.data_ptr(), vt.data_ptr(), TL.data_ptr(), 16, -1)
    keep = (kp, vp, q, SL, kt, vt, TL, ws)
    return common, ws, B * n_q, keep


def test_static_workspace_entry_equals_the_caller_memory_entry():
    dev = require_gpu()
    from gaac_amd import _lib
    big = _case(dev, 2, 4, 4, 4096, 16, seed=51, tail=7)
    small = _case(dev, 1, 2, 2, 333, 3, seed=61, tail=0)
    stream = _lib.stream()
    _lib.call("gaac_static_init")
    flags = torch.full((1,), 7, dtype=torch.int32, device=dev)
    for common, ws, rows, _keep in (big, small, big, small):
        want = torch.empty(rows, 128, dtype=torch.bfloat16, device=dev); got = torch.full_like(want, float("nan"))
        p = _lib.ptr
        _lib.call("gaac_attn_fused", *common, p(ws.pm), p(ws.pl), p(ws.pa), p(ws.epoch), p(want), stream)
        _lib.call("gaac_attn_fused_static", *common, p(got), stream)
        torch.cuda.synchronize()
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    _lib.call("gaac_static_flags", _lib.ptr(flags), stream)
    torch.cuda.synchronize()
    assert int(flags) == 0
    # re-arm (epoch words and records back to zero, by a kernel), then a call captured in a graph and replayed
    _lib.call("gaac_static_reset", stream)
    common, ws, rows, _keep = small
    want = torch.empty(rows, 128, dtype=torch.bfloat16, device=dev); got = torch.full_like(want, float("nan"))
    _lib.call("gaac_attn_fused", *common, _lib.ptr(ws.pm), _lib.ptr(ws.pl), _lib.ptr(ws.pa), _lib.ptr(ws.epoch), _lib.ptr(want), stream)
    side = torch.cuda.Stream(); side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            _lib.call("gaac_attn_fused_static", *common, _lib.ptr(got), _lib.stream())
    for _ in range(3):
        got.fill_(float("nan")); torch.cuda.synchronize()
        g.replay(); torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    _lib.call("gaac_static_flags", _lib.ptr(flags), stream)
    torch.cuda.synchronize()
    assert int(flags) == 0
    # beyond the built-in workspace: 4 x 32 query rows x 32 splits = 4096 > 4000 partial rows
    common, ws, rows, _keep = _case(dev, 4, 8, 4, 512, 32, seed=71, tail=0)
    out = torch.empty(rows, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="exceeds"):
        _lib.call("gaac_attn_fused_static", *common, _lib.ptr(out), stream)
