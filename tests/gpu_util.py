"""Helpers for the GPU parity tests: device availability, native page -> reference-layout page."""
import numpy as np
import pytest
import torch

from oracle import gaac_oracle as O


def require_gpu():
    if not torch.cuda.is_available():
        pytest.fail("this test is marked gpu and needs a real device; run CPU tests with -m 'not gpu'")
    return "cuda"


def native_to_reference_page(page) -> O.OPage:
    """Re-order the sign/mantissa and code bytes of a gaac_amd Page (native gfx950 tile order) into the reference's tile
    order, through token-major order, so the result can be compared field by field with the oracle's page."""
    from gaac_amd.codec import storage_index
    H = page.H
    S_pad = page.sm.shape[1] // 128
    nt = S_pad // 16
    si_n, ci_n = (t.numpy() for t in storage_index(page.kind, "cpu"))
    si_r, ci_r = O.storage_index(page.kind)
    sm = page.sm.cpu().numpy().reshape(H, nt, 2048)
    cd = page.codes.cpu().numpy().reshape(H, nt, 768)
    sm_tm = np.empty_like(sm); sm_tm[:, :, si_n] = sm
    cd_tm = np.empty_like(cd); cd_tm[:, :, ci_n] = cd
    return O.OPage(np.ascontiguousarray(sm_tm[:, :, si_r]).reshape(H, -1), np.ascontiguousarray(cd_tm[:, :, ci_r]).reshape(H, -1),
                   page.flags.cpu().numpy(), page.ovf_off.cpu().numpy(), page.ovf.cpu().numpy(), page.ovf_head_start.cpu().numpy(),
                   page.tile_off.cpu().numpy(), page.base3.cpu().numpy(), page.base4.cpu().numpy(), page.H, page.S, page.n_kv, page.kind)


def assert_pages_equal(got: O.OPage, want: O.OPage):
    for f in ("sm", "codes", "flags", "ovf_off", "ovf_head_start", "tile_off"):
        a, b = getattr(got, f), getattr(want, f)
        assert a.shape == b.shape and np.array_equal(a, b), f
    n = int(want.ovf_head_start[-1])
    assert np.array_equal(got.ovf[:n], want.ovf[:n]), "ovf"
