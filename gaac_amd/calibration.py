"""Offline calibration of the per-(layer, kv head, channel) exponent bases on MI355X.

Same interface and file format as /root/reference/gaac/calibration.py:13-35: observe() the K/V a model produces during prefill,
bases() keeps per channel the start of the densest 8-wide (3-bit) and 16-wide (4-bit) exponent window, save() writes
{layer: {k3, k4, v3, v4}} with uint8 [n_kv, 128] CPU tables (4 KiB per layer) through torch.save, so files written by either
implementation load in the other.  Histograms live on the device and the histogram kernel adds into them in place."""
from __future__ import annotations
import torch
from . import _lib
from .codec import D, bases_from_hist


class BaseCollector:
    def __init__(self):
        self.hist = {}      # layer -> {'k': int64 [n_kv*D, 256], 'v': ..., 'n_kv': int}

    def _add(self, hist: torch.Tensor, x: torch.Tensor, n_kv: int):
        x = x.contiguous()
        _lib.call("gaac_exponent_hist", _lib.ptr(x), x.numel() // (n_kv * D), n_kv, _lib.ptr(hist), _lib.stream())

    def observe(self, layer: int, k: torch.Tensor, v: torch.Tensor):
        """k, v: [N, n_kv, D] bf16 of one prefill step."""
        n_kv = k.shape[1]
        h = self.hist.get(layer)
        if h is None:
            zeros = lambda: torch.zeros(n_kv * D, 256, dtype=torch.int64, device=k.device)
            h = self.hist[layer] = {"k": zeros(), "v": zeros(), "n_kv": n_kv}
        if h["n_kv"] != n_kv or k.shape[-1] != D or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
            raise RuntimeError(f"observe expects bf16 [N, {h['n_kv']}, {D}] for layer {layer}")
        self._add(h["k"], k, n_kv); self._add(h["v"], v, n_kv)

    def bases(self) -> dict:
        out = {}
        for layer in sorted(self.hist):
            h = self.hist[layer]
            k3, k4 = bases_from_hist(h["k"], h["n_kv"]); v3, v4 = bases_from_hist(h["v"], h["n_kv"])
            out[layer] = {"k3": k3.cpu(), "k4": k4.cpu(), "v3": v3.cpu(), "v4": v4.cpu()}
        return out

    def save(self, path: str) -> int:
        tables = self.bases()
        torch.save(tables, path)
        return len(tables)


def load_bases(path: str) -> dict:
    """Reads a bases file (written here or by the reference) without executing anything from it."""
    return torch.load(path, map_location="cpu", weights_only=True)
