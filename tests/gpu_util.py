"""Helpers for the GPU parity tests: device availability, native page -> reference-layout page."""
import numpy as np
import pytest
import torch

from oracle import gaac_oracle as O


def require_gpu():
    if not torch.cuda.is_available():
        pytest.fail("this test is marked gpu and needs a real device; run CPU tests with -m 'not gpu'")
    return "cuda"


def _v_tags_and_escapes_to_reference(flags, ovf, head_start, tile_off, S):
    """V pages keep, per tile, the TRANSPOSE of the reference's 16 x 16 tag matrix (word g = tags of the 16 tokens for group g)
    and their escape bytes in (group, token) order.  Returns (flags, ovf) in the reference's (token, group) order."""
    H, S_pad = flags.shape
    f_out = np.zeros_like(flags); o_out = ovf.copy()
    size = {0: 0, 1: 1, 3: 5}
    for h in range(H):
        for t in range(S_pad // 16):
            words = flags[h, 16 * t:16 * t + 16].astype(np.int64) & 0xFFFFFFFF
            tag = np.array([[(int(words[g]) >> (2 * tok)) & 3 for tok in range(16)] for g in range(16)])      # [group][token]
            for tok in range(16):
                f_out[h, 16 * t + tok] = np.uint32(sum(int(tag[g, tok]) << (2 * g) for g in range(16))).astype(np.uint32).view(np.int32)
            base = int(head_start[h]) + int(tile_off[h, t])
            pos, chunks = base, {}
            for g in range(16):
                for tok in range(16):
                    n = size[int(tag[g, tok])]
                    chunks[(tok, g)] = ovf[pos:pos + n]; pos += n
            out = base
            for tok in range(16):
                for g in range(16):
                    c = chunks[(tok, g)]
                    o_out[out:out + len(c)] = c; out += len(c)
            assert out == pos
    return f_out, o_out


def native_to_reference_page(page) -> O.OPage:
    """Re-order a gaac_amd Page (native gfx950 tile order) into the reference's order so that it can be compared field by
    field with the oracle's page: sign/mantissa and code bytes through token-major order; for V also the per-tile tag matrix
    and escape order (transposed natively); row offsets are re-derived from the re-ordered tags."""
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
    flags, ovf, ovf_off = page.flags.cpu().numpy(), page.ovf.cpu().numpy(), page.ovf_off.cpu().numpy()
    assert np.array_equal(ovf_off, O.row_offsets(flags, page.S))          # offsets of the native lines
    if page.kind == "v":
        flags, ovf = _v_tags_and_escapes_to_reference(flags, ovf, page.ovf_head_start.cpu().numpy(), page.tile_off.cpu().numpy(), page.S)
        ovf_off = O.row_offsets(flags, page.S)
    return O.OPage(np.ascontiguousarray(sm_tm[:, :, si_r]).reshape(H, -1), np.ascontiguousarray(cd_tm[:, :, ci_r]).reshape(H, -1),
                   flags, ovf_off, ovf, page.ovf_head_start.cpu().numpy(),
                   page.tile_off.cpu().numpy(), page.base3.cpu().numpy(), page.base4.cpu().numpy(), page.H, page.S, page.n_kv, page.kind)


def assert_pages_equal(got: O.OPage, want: O.OPage):
    for f in ("sm", "codes", "flags", "ovf_off", "ovf_head_start", "tile_off"):
        a, b = getattr(got, f), getattr(want, f)
        assert a.shape == b.shape and np.array_equal(a, b), f
    n = int(want.ovf_head_start[-1])
    assert np.array_equal(got.ovf[:n], want.ovf[:n]), "ovf"
