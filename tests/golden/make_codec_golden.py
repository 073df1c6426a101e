"""Writes tests/golden/codec_{k,v}.npz: input bit patterns, bases, and every field of the page the REFERENCE codec
produces for them, plus what its decoder returns.  Run once in the build container (the reference tree is not
available anywhere else):

    python tests/golden/make_codec_golden.py

Only /root/reference/gaac/codec.py is loaded, by file path and on the CPU (importing the package would pull in
its Triton/CUDA modules).  The fixture pins the one thing closed forms do not pin cheaply: the exact byte
placement of sign/mantissa bytes, code bytes and escape bytes inside a reference page.
"""
import importlib.util, os, sys
import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from oracle import gaac_oracle as O   # noqa: E402  (only to pick bases for the inputs)

spec = importlib.util.spec_from_file_location("ref_codec", "/root/reference/gaac/codec.py")
ref = importlib.util.module_from_spec(spec)
sys.modules["ref_codec"] = ref      # dataclass creation looks the module up by name
spec.loader.exec_module(ref)


def make_input(H, S, seed):
    """Gaussian channels over ~8 binades + outliers (all three tiers) + a few special bit patterns."""
    scale = np.exp2(np.random.default_rng(7).random((1, 1, 128)) * 8 - 4)     # channel scales shared by calibration and data
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((H, S, 128)) * scale
    x = np.where(rng.random((H, S, 128)) < 4e-3, x * 1e4, x)
    x16 = O.f32_to_bf16_rne(x.astype(np.float32))
    special = np.array([0x0000, 0x8000, 0x0001, 0x807F, 0x7F80, 0xFF80, 0x7FC0, 0xFFFF, 0x7F7F, 0x0080], dtype=np.uint16)
    pos = rng.integers(0, x16.size, size=special.size * 3)
    x16.reshape(-1)[pos] = np.tile(special, 3)
    return x16


for kind in ("k", "v"):
    n_kv, H, S = 2, 4, 40
    calib16 = make_input(H, 256, seed=100 + (kind == "v"))
    x16 = make_input(H, S, seed=200 + (kind == "v"))
    b3, b4 = O.calibrate(calib16, n_kv)
    codec = ref.Codec(n_kv, device="cpu").set_bases(torch.from_numpy(b3), torch.from_numpy(b4))
    x = torch.from_numpy(x16.view(np.int16)).view(torch.bfloat16)
    page = codec.encode(x, kind)
    back = ref.Codec.decode(page).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(back, x16)
    np.savez_compressed(os.path.join(HERE, f"codec_{kind}.npz"),
                        x16=x16, base3=b3, base4=b4, n_kv=n_kv,
                        sm=page.sm.numpy(), codes=page.codes.numpy(), flags=page.flags.numpy(), ovf_off=page.ovf_off.numpy(),
                        ovf=page.ovf.numpy(), ovf_head_start=page.ovf_head_start.numpy(), tile_off=page.tile_off.numpy(),
                        nbytes=page.nbytes, decoded=back)
    print(kind, "nbytes", page.nbytes, "ratio", page.ratio, "esc", int(page.ovf_head_start[-1]))
