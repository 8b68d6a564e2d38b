"""``Int8XLinear``: an ``nn.Linear`` stand-in backed by an INT8-X packed weight.

Mirrors the reference's ``ixrun/linear.py``: ``cache='full'`` decodes once at
construction and then runs a plain ``F.linear``; ``cache='none'`` decodes on
every forward.  ``deploy_model`` swaps every eligible ``nn.Linear`` of a model.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .config import MIN_LINEAR_ELEMS, SKIP_PATTERNS
from .quantize import int8x_quantize, portable_packed, quantize_for_deploy
from .triton_kernels import decode_weight_scatter, decode_weight_triton

__all__ = ["Int8XLinear", "deploy_model", "iter_quantizable_linears"]


def iter_quantizable_linears(model: nn.Module):
    """``(name, module)`` of the Linears to quantize: at least MIN_LINEAR_ELEMS
    weights and no SKIP_PATTERNS substring in the name (reference
    ``ixrun/linear.py:25-34``)."""
    for name, mod in model.named_modules():
        if isinstance(mod, nn.Linear) and mod.weight.numel() >= MIN_LINEAR_ELEMS \
                and not any(pat in name for pat in SKIP_PATTERNS):
            yield name, mod


def _set_parent_child(model: nn.Module, dotted_name: str, new_module: nn.Module):
    """Replace the submodule at ``dotted_name`` (reference ``ixrun/linear.py:37-42``)."""
    *path, leaf = dotted_name.split(".")
    parent = model
    for part in path:
        parent = getattr(parent, part)
    setattr(parent, leaf, new_module)


class Int8XLinear(nn.Module):
    """Linear layer over a packed dict (reference ``ixrun/linear.py:45-100``).

    ``cache='full'`` keeps the decoded bf16 weight in ``_w``; ``cache='none'``
    re-decodes on the input's device each forward.  ``use_triton`` keeps its
    name: True selects the device kernel (HIP here), False the torch decoder.
    """

    def __init__(self, packed: dict, bias=None, cache: str = "full", use_triton: bool = True):
        super().__init__()
        self.out_features = packed["out_f"]
        self.in_features = packed["in_f"]
        self.packed = packed
        self.use_triton = use_triton
        self._cache = cache
        if bias is not None:
            self.register_buffer("_bias_buf", bias.detach().clone())
        else:
            self._bias_buf = None
        self._w = None
        if cache == "full":
            self._w = self._decode(torch.device("cuda" if torch.cuda.is_available() else "cpu"))

    def _decode(self, device):
        if self.use_triton and torch.cuda.is_available():
            return decode_weight_triton(self.packed, device)
        return decode_weight_scatter(self.packed, device)

    def forward(self, x):
        w = self._w if self._cache == "full" else self._decode(x.device)
        bias = self._bias_buf.to(x.dtype) if self._bias_buf is not None else None
        return F.linear(x, w, bias)

    def extra_repr(self) -> str:
        return (f"in={self.in_features}, out={self.out_features}, "
                f"levels={self.packed['level_bits']}, bpw={self.packed['bits_per_weight']:.2f}")


@torch.no_grad()
def deploy_model(model: nn.Module, level_bits=(3, 5, 8), cache: str = "full", use_triton: bool = True,
                 verbose: bool = True) -> dict:
    """Swap every quantizable Linear for an Int8XLinear, in place, and return
    the statistics of the reference's ``deploy_model`` (``ixrun/linear.py:104-145``)."""
    n_layers = total_bytes = n_elems = 0
    counts = [0] * len(tuple(level_bits))
    for name, mod in list(iter_quantizable_linears(model)):
        packed = quantize_for_deploy(mod.weight.data, level_bits) if use_triton else int8x_quantize(mod.weight.data, level_bits)
        bias = mod.bias.data if mod.bias is not None else None
        layer = Int8XLinear(packed, bias=bias, cache=cache, use_triton=use_triton)
        if cache == "full":  # the decoded weight is what stays on the GPU; the packed form goes back to the host
            layer.packed = packed = portable_packed(packed)
        _set_parent_child(model, name, layer)
        n_layers += 1
        total_bytes += packed["total_bytes"]
        n_elems += packed["N"]
        counts = [a + b for a, b in zip(counts, packed["counts"])]
    stats = {
        "n_layers": n_layers,
        "total_bytes": total_bytes,
        "n_elems": n_elems,
        "counts": counts,
        "bits_per_weight": (total_bytes * 8) / max(n_elems, 1),
        "compression_vs_bf16": (n_elems * 2) / max(total_bytes, 1),
    }
    if verbose:
        tot = max(sum(counts), 1)
        shares = " ".join(f"L{i + 1}={c / tot * 100:.1f}%" for i, c in enumerate(counts))
        print(f"[deploy] {n_layers} layers | {total_bytes / 1e6:.0f}MB packed "
              f"({stats['compression_vs_bf16']:.2f}x vs bf16) | bpw={stats['bits_per_weight']:.2f} | {shares}",
              flush=True)
    return stats
