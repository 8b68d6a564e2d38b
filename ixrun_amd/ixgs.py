"""Group-scale INT8-X ("ixgs"): the (3,5,8) nested-bitmap streams with one fp16 scale per group of weights.

Mirror of the reference's ``ixgs`` package for the GPU path of this build: same function names, arguments and
dictionary keys (``ixgs/__init__.py``), the decode done by ``ixh_decode_gs`` of the HIP library instead of the
Triton kernel plus its three per-element rank tensors (``ixgs/kernels.py:30-142``).

Format (``ixgs/quantize.py:36-111``): the flat weights are cut into groups of ``group_size``; a group's scale is
``fp16(max(group max / 15, 1e-10))`` and its integers are ``clamp(round(w / scale), -127, 128)``.  Integers in
``[-3, 4]`` go to the 3-bit stream as ``v + 3``, those in ``[-15, 16]`` to the 5-bit stream as ``v + 15``, the rest
to the byte stream as ``v + 127``; ``b1`` marks tier 1 per element, ``b2`` marks tier 2 per element outside tier 1.
An empty ``b2`` / ``l3`` is stored as one zero element.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .bitpack import pack_bits_stream, unpack_bits_stream

__all__ = ["GROUP_SIZE", "SCALE_DIVISOR", "int8gs_quantize", "decode_weight_scatter", "decode_weight_triton",
           "has_triton", "per_tensor_int8_reference", "Int8GSLinear", "deploy_model_gs", "iter_quantizable_linears"]

GROUP_SIZE = 64
SCALE_DIVISOR = 15.0
TIER1 = (-3, 4)
TIER2 = (-15, 16)
SKIP_PATTERNS = ("lm_head", "embed", "shared", "wte")
MIN_LINEAR_ELEMS = 1000


@torch.no_grad()
def int8gs_quantize(weight: torch.Tensor, group_size: int = GROUP_SIZE) -> dict:
    """2-D weight -> packed dictionary with the reference's keys (``ixgs/quantize.py:97-111``).

    One deliberate difference: a group whose fp16 scale is zero (an all-zero group, or a group maximum below
    4.5e-7) makes the reference divide by zero and cast NaN to an integer; here such a group's integers are 0,
    which decodes to the zeros the group holds (to within 4.5e-7).
    """
    if weight.dim() != 2:
        raise ValueError(f"expected 2-D weight, got {list(weight.shape)}")
    out_f, in_f = weight.shape
    n = out_f * in_f
    n_groups = -(-n // group_size)
    w = weight.detach().float().reshape(-1).cpu()
    padded = torch.zeros(n_groups * group_size)
    padded[:n] = w
    group_max = padded.view(n_groups, group_size).abs().amax(dim=1)
    # the scale is rounded to fp16 before it divides, so that encoder and decoder use the same number
    scales16 = (group_max / SCALE_DIVISOR).clamp(min=1e-10).to(torch.float16)
    s_elem = scales16.float().repeat_interleave(group_size)[:n]
    live = s_elem > 0
    q = torch.where(live, (w / torch.where(live, s_elem, torch.ones_like(s_elem))).round().clamp(-127, 128),
                    torch.zeros_like(w)).to(torch.int32)

    in1 = (q >= TIER1[0]) & (q <= TIER1[1])
    rest = q[~in1]
    in2 = (rest >= TIER2[0]) & (rest <= TIER2[1])
    n1, n2 = int(in1.sum()), int(in2.sum())
    n3 = n - n1 - n2
    l1 = pack_bits_stream(q[in1] - TIER1[0], 3)
    l2 = pack_bits_stream(rest[in2] - TIER2[0], 5)
    l3 = (rest[~in2] + 127).to(torch.uint8) if n3 else torch.zeros(1, dtype=torch.uint8)
    b1 = pack_bits_stream(in1.to(torch.int32), 1)
    b2 = pack_bits_stream(in2.to(torch.int32), 1) if n2 + n3 else torch.zeros(1, dtype=torch.int32)
    total = 4 * (l1.numel() + l2.numel() + b1.numel() + b2.numel()) + max(n3, 1) + 2 * n_groups
    return {
        "out_f": out_f, "in_f": in_f, "N": n, "group_size": group_size,
        "group_scales": scales16,
        "b1": b1, "b2": b2, "l1": l1, "l2": l2, "l3": l3,
        "counts": [n1, n2, n3],
        "total_bytes": total,
        "bits_per_weight": (total * 8) / n,
        "compression_vs_bf16": (n * 2) / total,
    }


@torch.no_grad()
def decode_weight_scatter(packed: dict, device=None, dtype=torch.bfloat16) -> torch.Tensor:
    """Decode with torch ops only (``ixgs/quantize.py:113-151``): positions of each tier from the bitmaps, codes
    unpacked per stream and scattered, then ``dtype(f32(v) * f32(group scale))``."""
    if device is None:
        device = torch.device("cuda" if torch.cuda.is_available() else "cpu")
    n, gs = packed["N"], packed["group_size"]
    n1, n2, n3 = packed["counts"]
    tier1 = unpack_bits_stream(packed["b1"].cpu(), n, 1).bool()
    outside = (~tier1).nonzero(as_tuple=True)[0]
    q = torch.zeros(n, dtype=torch.int32)
    if n1:
        q[tier1] = unpack_bits_stream(packed["l1"].cpu(), n1, 3) + TIER1[0]
    if outside.numel():
        tier2 = unpack_bits_stream(packed["b2"].cpu(), outside.numel(), 1).bool()
        if n2:
            q[outside[tier2]] = unpack_bits_stream(packed["l2"].cpu(), n2, 5) + TIER2[0]
        if n3:
            q[outside[~tier2]] = packed["l3"].cpu()[:n3].to(torch.int32) - 127
    s_elem = packed["group_scales"].float().cpu().repeat_interleave(gs)[:n]
    return (q.float() * s_elem).to(dtype).view(packed["out_f"], packed["in_f"]).to(device)


def has_triton() -> bool:
    """The reference's name for "the device decoder can run" (``ixgs/kernels.py:24-25``): here, a GPU and the
    built HIP library."""
    if not torch.cuda.is_available():
        return False
    from . import _lib

    try:
        _lib.lib()
    except RuntimeError:
        return False
    return True


@torch.no_grad()
def decode_weight_triton(packed: dict, device=None, dtype=torch.bfloat16) -> torch.Tensor:
    """Device decode (``ixgs/kernels.py:121-142``) through ``ixh_decode_gs``.  Needs the GPU and the library;
    there is no fallback inside this function."""
    from . import _lib

    assert torch.cuda.is_available(), "the device decoder needs the GPU"
    device = torch.device(device) if device is not None else torch.device("cuda")
    mv = lambda t: t.to(device).contiguous()
    dp = _lib.DevicePacked((3, 5, 8), packed["out_f"], packed["in_f"], [mv(packed["b1"]), mv(packed["b2"])],
                           [mv(packed["l1"]), mv(packed["l2"]), mv(packed["l3"])], None)
    scales = mv(packed["group_scales"].to(torch.float16))
    out = torch.empty(packed["N"], dtype=torch.bfloat16, device=device)
    if packed["N"]:
        table = dp.prefix_build(512)
        dp.decode_gs(table, 512, scales, packed["group_size"], out)
    return out.view(packed["out_f"], packed["in_f"]).to(dtype)


@torch.no_grad()
def per_tensor_int8_reference(weight: torch.Tensor) -> torch.Tensor:
    """What per-tensor int8 makes of the weight (``ixgs/quantize.py:154-158``), for comparisons."""
    scale = weight.abs().max().clamp(min=1e-8) / 127.0
    return ((weight.float() / scale).round().clamp(-127, 127) * scale).to(weight.dtype)


def iter_quantizable_linears(model: nn.Module):
    """Linear layers the deploy replaces (``ixgs/linear.py:18-26``)."""
    for name, mod in model.named_modules():
        if isinstance(mod, nn.Linear) and mod.weight.numel() >= MIN_LINEAR_ELEMS \
                and not any(s in name for s in SKIP_PATTERNS):
            yield name, mod


def _decode(packed: dict, device, use_triton: bool = True) -> torch.Tensor:
    if use_triton and has_triton():
        return decode_weight_triton(packed, device)
    return decode_weight_scatter(packed, device)


class Int8GSLinear(nn.Module):
    """Linear layer over a group-scale packed weight (``ixgs/linear.py:35-73``): ``cache='full'`` decodes once,
    ``cache='none'`` decodes in every forward."""

    def __init__(self, packed: dict, bias=None, cache: str = "full", use_triton: bool = True):
        super().__init__()
        self.out_features, self.in_features = packed["out_f"], packed["in_f"]
        self.packed = packed
        self._cache, self._use_triton = cache, use_triton
        if bias is not None:
            self.register_buffer("_bias_buf", bias.detach().clone())
        else:
            self._bias_buf = None
        self._w = None
        if cache == "full":
            self._w = _decode(packed, torch.device("cuda" if torch.cuda.is_available() else "cpu"), use_triton)

    def forward(self, x):
        w = self._w if self._cache == "full" else _decode(self.packed, x.device, self._use_triton)
        bias = self._bias_buf.to(x.dtype) if self._bias_buf is not None else None
        return F.linear(x, w, bias)

    def extra_repr(self) -> str:
        p = self.packed
        return (f"in={self.in_features}, out={self.out_features}, gs={p['group_size']}, counts={p['counts']}, "
                f"bpw={p['bits_per_weight']:.2f}")


@torch.no_grad()
def deploy_model_gs(model: nn.Module, group_size: int = GROUP_SIZE, cache: str = "full", use_triton: bool = True,
                    verbose: bool = True) -> dict:
    """Swap every quantizable Linear for an Int8GSLinear in place; statistics as ``ixgs/linear.py:76-114``."""
    total_bytes = n_elems = n_layers = 0
    counts = [0, 0, 0]
    for name, mod in list(iter_quantizable_linears(model)):
        packed = int8gs_quantize(mod.weight.data, group_size)
        bias = mod.bias.data if mod.bias is not None else None
        parent = model
        *path, leaf = name.split(".")
        for part in path:
            parent = getattr(parent, part)
        setattr(parent, leaf, Int8GSLinear(packed, bias=bias, cache=cache, use_triton=use_triton))
        n_layers += 1
        total_bytes += packed["total_bytes"]
        n_elems += packed["N"]
        counts = [a + b for a, b in zip(counts, packed["counts"])]
    stats = {"n_layers": n_layers, "total_bytes": total_bytes, "n_elems": n_elems, "counts": counts,
             "bits_per_weight": (total_bytes * 8) / max(n_elems, 1),
             "compression_vs_bf16": (n_elems * 2) / max(total_bytes, 1)}
    if verbose and n_elems:
        shares = " ".join(f"L{i + 1}={c / n_elems * 100:.1f}%" for i, c in enumerate(counts))
        print(f"[deploy-gs] {n_layers} layers | {total_bytes / 1e6:.0f}MB ({stats['compression_vs_bf16']:.2f}x vs bf16) | "
              f"bpw={stats['bits_per_weight']:.2f} | {shares}", flush=True)
    return stats
