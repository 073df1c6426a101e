"""ctypes binding of gaac_amd/libgaac_hip.so (see include/gaac_hip.h).  There is no fallback: if the library is
missing, or a call is made without a GPU, the call raises."""
from __future__ import annotations
import ctypes, os
import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libgaac_hip.so")
_lib = None

c_int, c_long, c_float, c_void_p = ctypes.c_int, ctypes.c_long, ctypes.c_float, ctypes.c_void_p
P = c_void_p

_SIGNATURES = {
    "gaac_exponent_hist": [P, c_long, c_int, P, P],
    "gaac_bases_from_hist": [P, c_int, P, P, P],
    "gaac_encode_tiles": [c_int, P, c_long, c_long, c_int, c_int, c_int, P, P, c_int, P, P, P, P, P, P, P],
    "gaac_compact": [P, P, P, P, P, c_int, c_int, P],
    "gaac_row_offsets": [P, c_int, c_int, c_int, P, P, P],
    "gaac_decode_tiles": [c_int, P, P, P, P, P, P, P, P, c_int, P, c_int, c_int, c_int, P, c_long, c_long, P],
    "gaac_attn_split": [P] * 16 + [P, P, c_int, c_int, c_int, P, c_int, c_float, c_int, c_int, P, P, P, c_int, P, P, P, P],
    "gaac_attn_combine": [P, P, P, P, c_int, c_int, P],
    "gaac_cache_append": [P, c_int, c_int, P, P, P, P, c_int, c_int, c_int] + [P] * 18 + [P, P],
    "gaac_paged_store": [P, P, c_long, c_long, P, c_int, P, c_int, P, P, P, P, P, P, P, P, P, P, c_int, P],
    "gaac_paged_free": [P, c_int, P, P, P],
    "gaac_paged_release": [P, c_int, P, P, P, c_int, P],
    "gaac_paged_decode": [P, c_int, P, P, P, c_int, P, P, c_long, P, P, P, P, c_int, P],
    "gaac_paged_attn": [P, c_int, P, P, P, c_int, P, c_int, P, c_int, c_int, c_int, c_float, c_int, P, P, P, P, c_int, P, P, P, P, P, P, c_int, P, P, P],
    "gaac_bf16_attn": [P, P, c_int, P, c_long, P, c_int, c_int, c_int, c_float, c_int, P, P, P, P, P, P],
    "gaac_attn_fused": [P] * 16 + [P, P, c_int, c_int, c_int, P, c_int, c_float, c_int, c_int, P, P, P, c_int, c_int, P, P, P, P, P, P],
    "gaac_attn_fused_static": [P] * 16 + [P, P, c_int, c_int, c_int, P, c_int, c_float, c_int, c_int, P, P, P, c_int, c_int, P, P],
    "gaac_static_init": [],
    "gaac_static_reset": [P],
    "gaac_static_flags": [P, P],
    "gaac_attn_launch": [P] * 16 + [P, P, c_int, c_int, c_int, P, c_int, c_float, c_int, c_int, P, P, P, c_int, P, P, P, P, P],
}


def lib_path() -> str:
    """The library file: gaac_amd/libgaac_hip.so, or the instrumented build named by GAAC_HIP_LIB (read when the library is loaded)."""
    return os.environ.get("GAAC_HIP_LIB") or _LIB_PATH


def load():
    """The loaded library (ctypes.CDLL).  Raises if it has not been built (python -m gaac_amd.build)."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python -m gaac_amd.build` (hipcc, gfx950). "
                               "gaac_amd has no CPU or PyTorch fallback.")
        lib = ctypes.CDLL(path)
        lib.gaac_last_error.restype = ctypes.c_char_p
        lib.gaac_last_error.argtypes = []
        for name, args in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = c_int
            fn.argtypes = args
        _lib = lib
    return _lib


def exported_symbols() -> list[str]:
    return ["gaac_last_error", *_SIGNATURES]


def ptr(t: torch.Tensor | None):
    if t is None:
        return None
    if not t.is_cuda:
        raise RuntimeError("gaac_amd kernels need device tensors (got a CPU tensor): there is no CPU path")
    return t.data_ptr()


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def call(name: str, *args):
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed ({rc}): {lib.gaac_last_error().decode(errors='replace')}")
