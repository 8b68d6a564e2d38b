"""INT8-X encoder and host-side (torch) decoder.

A weight matrix is first reduced to per-tensor int8 (``scale = max|w| / 127``)
and the int8 values are then stored losslessly by magnitude level.  With
``level_bits = (b_0 < b_1 < ... < 8)`` and ``T_b = 2**(b-1) - 1``, level ``i``
holds the values with ``T_{b_{i-1}} < |v| <= T_{b_i}`` as ``b_i``-bit codes
``v + T_{b_i}`` in flat (row-major) order.  Bitmap ``i`` has one bit for every
element that is not in a level below ``i``; the bit says whether the element
is in level ``i``.  The last level needs no bitmap and is kept as raw bytes.

This module follows the reference's ``ixrun/quantize.py`` (encoder ``:41-122``,
position rebuild ``:126-150``, scatter decoder ``:154-183``) so that the
dictionaries it writes are the ones the reference writes; the device decoders
live in :mod:`ixrun_amd.triton_kernels` and :mod:`ixrun_amd.fused`.
"""
from __future__ import annotations

import torch

from .bitpack import pack_bits_stream, pack_bitmap, unpack_bits_stream
from .config import BIT_TO_THRESHOLD, DEFAULT_LEVELS

__all__ = ["int8x_quantize", "int8x_quantize_device", "quantize_for_deploy", "portable_packed", "compute_positions", "decode_to_weight", "DEFAULT_LEVELS"]


def _level_ids(abs_v: torch.Tensor, level_bits: tuple) -> torch.Tensor:
    """Level index of every |v|: the first level whose threshold covers it
    (reference ``ixrun/quantize.py:25-37``)."""
    edges = torch.tensor([BIT_TO_THRESHOLD[b] for b in level_bits[:-1]], dtype=abs_v.dtype)
    return torch.bucketize(abs_v, edges, right=False)


@torch.no_grad()
def int8x_quantize(weight: torch.Tensor, level_bits: tuple = DEFAULT_LEVELS) -> dict:
    """Quantize a 2-D weight to the INT8-X packed dictionary.

    Keys, order and tensor types are those of the reference's
    ``int8x_quantize`` (``ixrun/quantize.py:110-122``): ``level_bits, out_f,
    in_f, N, scale`` (0-dim bf16), ``bitmaps`` (int32 words), ``streams``
    (int32 words, last one uint8), ``counts, total_bytes, bits_per_weight,
    compression_vs_bf16``.  ``level_bits`` is sorted; a last level other than
    8 raises ``ValueError`` (``:56-58``).
    """
    level_bits = tuple(sorted(level_bits))
    if level_bits[-1] != 8:
        raise ValueError("last level must be 8-bit to cover the full int8 range")
    out_f, in_f = weight.shape
    n = out_f * in_f

    # The scale is formed in the weight's own dtype (a bf16 weight gives a
    # bf16-rounded divisor) and the division is done in fp32 with
    # round-half-even, as at ixrun/quantize.py:64-73.
    scale = weight.abs().max().clamp(min=1e-8) / 127.0
    q = (weight.float() / scale).round().clamp(-127, 127).to(torch.int8).reshape(-1).cpu()
    scale = scale.detach().cpu().bfloat16().reshape(())

    q16 = q.to(torch.int16)
    lvl = _level_ids(q16.abs(), level_bits)
    n_levels = len(level_bits)
    counts = torch.bincount(lvl, minlength=n_levels).tolist()

    streams, bitmaps = [], []
    alive = None  # indices of elements not claimed by a lower level
    for i, b in enumerate(level_bits):
        member = lvl == i
        codes = (q16[member] + BIT_TO_THRESHOLD[b]).to(torch.int32)
        if i == n_levels - 1:
            streams.append(codes.to(torch.uint8))
        else:
            streams.append(pack_bits_stream(codes, b))
            bitmaps.append(pack_bitmap(member if alive is None else member[alive]))
            alive = (lvl > i).nonzero(as_tuple=True)[0]

    # byte accounting of ixrun/quantize.py:99-108: 2 bytes of scale, 4 per word
    total = 2 + streams[-1].numel()
    total += 4 * sum(s.numel() for s in streams[:-1])
    total += 4 * sum(bm.numel() for bm in bitmaps)

    return {
        "level_bits": level_bits,
        "out_f": out_f,
        "in_f": in_f,
        "N": n,
        "scale": scale,
        "bitmaps": bitmaps,
        "streams": streams,
        "counts": counts,
        "total_bytes": total,
        "bits_per_weight": (total * 8) / n,
        "compression_vs_bf16": (n * 2) / total,
    }


@torch.no_grad()
def int8x_quantize_device(weight: torch.Tensor, level_bits: tuple = DEFAULT_LEVELS) -> dict:
    """``int8x_quantize`` for a bf16 weight that lives on the GPU, done by the library's encoder kernels.

    The dictionary has the reference's keys (``ixrun/quantize.py:110-122``) with the same bytes in every
    tensor as the CPU writer produces for this weight, but the tensors stay on the weight's device.  Two
    extra keys carry what the encoder computes on the way and the modules would otherwise rebuild:
    ``table512`` (the rank table at unit 512) and ``device_packed`` (the library's view of the tensors).
    There is no CPU path behind this function: a CPU tensor or a missing library raises.
    """
    from ._lib import encode_device

    level_bits = tuple(sorted(level_bits))
    if level_bits[-1] != 8:
        raise ValueError("last level must be 8-bit to cover the full int8 range")
    out_f, in_f = weight.shape
    n = out_f * in_f
    if n == 0:
        raise RuntimeError("max(): cannot quantize an empty weight")
    dp, table, counts = encode_device(weight.detach().contiguous(), level_bits)
    n_lv = len(level_bits)
    bitmaps, streams = dp.tensors[: n_lv - 1], dp.tensors[n_lv - 1 : 2 * n_lv - 1]
    total = 2 + streams[-1].numel()
    total += 4 * sum(s.numel() for s in streams[:-1])
    total += 4 * sum(bm.numel() for bm in bitmaps)
    return {
        "level_bits": level_bits,
        "out_f": out_f,
        "in_f": in_f,
        "N": n,
        "scale": dp.tensors[-1].reshape(()),
        "bitmaps": list(bitmaps),
        "streams": list(streams),
        "counts": counts,
        "total_bytes": total,
        "bits_per_weight": (total * 8) / n,
        "compression_vs_bf16": (n * 2) / total,
        "table512": table,
        "device_packed": dp,
    }


REFERENCE_KEYS = ("level_bits", "out_f", "in_f", "N", "scale", "bitmaps", "streams", "counts", "total_bytes",
                  "bits_per_weight", "compression_vs_bf16")


def portable_packed(packed: dict) -> dict:
    """The dictionary with the reference's keys only and every tensor on the CPU: what ``int8x_quantize``
    returns and what the packed-cache file holds (``ixrun/quantize.py:110-122``, ``ixrun/engine.py:383``)."""
    out = {k: packed[k] for k in REFERENCE_KEYS}
    out["scale"] = packed["scale"].detach().cpu().reshape(())
    out["bitmaps"] = [t.detach().cpu() for t in packed["bitmaps"]]
    out["streams"] = [t.detach().cpu() for t in packed["streams"]]
    return out


@torch.no_grad()
def quantize_for_deploy(weight: torch.Tensor, level_bits: tuple = DEFAULT_LEVELS) -> dict:
    """What the deploy paths call per layer: with a GPU in the process a bf16 weight is moved there (if it is
    not there already) and encoded by the device kernels, so the packed tensors are born where the modules
    keep them; any other weight goes through the CPU writer.  Same bytes either way."""
    if torch.cuda.is_available() and weight.dtype == torch.bfloat16 and weight.dim() == 2 and weight.numel() > 0:
        return int8x_quantize_device(weight.cuda(), level_bits)
    return int8x_quantize(weight, level_bits)


@torch.no_grad()
def compute_positions(packed: dict) -> list:
    """Flat positions (int64, CPU, ascending) of the elements of each level.

    Same result as the reference's ``compute_positions``
    (``ixrun/quantize.py:126-150``): peel the bitmaps one by one, each indexed
    over the elements the earlier ones left over.
    """
    left = torch.arange(packed["N"], dtype=torch.int64)
    per_level = []
    for bm in packed["bitmaps"]:
        flag = unpack_bits_stream(bm.cpu(), left.numel(), 1).bool()
        per_level.append(left[flag])
        left = left[~flag]
    per_level.append(left)
    return per_level


@torch.no_grad()
def decode_to_weight(packed: dict, device=None, dtype=torch.bfloat16) -> torch.Tensor:
    """Scatter decode on ``device`` with torch ops only
    (reference ``ixrun/quantize.py:154-183``): every level's codes are unpacked
    and written to their positions, then ``w = dtype(f32(v) * f32(scale))``."""
    level_bits = packed["level_bits"]
    n = packed["N"]
    positions = compute_positions(packed)
    q = torch.zeros(n, dtype=torch.int32, device=device)
    for i, (b, cnt) in enumerate(zip(level_bits, packed["counts"])):
        if cnt == 0:
            continue
        stream = packed["streams"][i].to(device)
        if i == len(level_bits) - 1:
            codes = stream[:cnt].to(torch.int32)
        else:
            codes = unpack_bits_stream(stream, cnt, b, device=device)
        q[positions[i].to(device)] = codes - BIT_TO_THRESHOLD[b]
    scale = packed["scale"].to(device)
    return (q.float() * scale.float()).to(dtype).view(packed["out_f"], packed["in_f"])
