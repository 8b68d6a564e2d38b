"""Full-matrix decode of INT8-X packed weights.

The module keeps the name and the functions of the reference's
``ixrun/triton_kernels.py`` so that ``from ixrun.triton_kernels import ...``
style imports carry over, but nothing here is Triton: the device decode is the
gfx950 HIP kernel of ``libixhip.so`` (any level scheme, any size), and
``decode_weight_scatter`` is the plain torch decoder the reference keeps as its
portable path (``ixrun/triton_kernels.py:36-59``).
"""
from __future__ import annotations

import torch

from . import _lib
from .config import TRITON_BLOCK
from .quantize import decode_to_weight

__all__ = ["decode_weight_triton", "decode_weight_scatter", "precompute_block_offsets"]


@torch.no_grad()
def decode_weight_scatter(packed: dict, device=None, dtype=torch.bfloat16) -> torch.Tensor:
    """Torch-only decode (unpack every level, scatter to its positions); the
    default device is the GPU when there is one, as in the reference."""
    if device is None:
        device = torch.device("cuda") if torch.cuda.is_available() else torch.device("cpu")
    return decode_to_weight(packed, device=device, dtype=dtype)


def precompute_block_offsets(packed: dict, blk: int = TRITON_BLOCK, device=None) -> tuple:
    """``(b1_blk, b2_blk)``: level-1 / level-2 elements in the flat blocks before
    block ``k``, int32 on the device (reference ``ixrun/triton_kernels.py:180-220``).

    Counted on the GPU from the bitmaps by ``ixh_prefix_build``; unlike the
    reference this also takes ``N % blk != 0`` (the last block is short).
    """
    if device is None:
        device = torch.device("cuda")
    dp = _lib.DevicePacked.from_dict(packed, device)
    table = dp.prefix_build(blk)
    n_blk = table.shape[1] - 1
    b1 = table[0, :n_blk].contiguous()
    b2 = table[1, :n_blk].contiguous() if table.shape[0] > 1 else torch.zeros_like(b1)
    return b1, b2


@torch.no_grad()
def decode_weight_triton(packed: dict, device=None, dtype=torch.bfloat16) -> torch.Tensor:
    """Decode a packed dict to a ``[out_f, in_f]`` weight on the GPU.

    Same call as the reference's ``decode_weight_triton`` (``ixrun/triton_kernels.py:224-259``), with two
    differences: every level scheme goes through the kernel, not only (3,5,8), and there is no silent
    fallback.  The reference switches to its torch scatter decoder when Triton or the GPU is missing; here a
    process without a GPU or without the built ``libixhip.so`` gets an error, and ``decode_weight_scatter`` is
    the CPU decoder to call by name (``Int8XLinear`` does so in a process that has no GPU at all, as the
    reference's does at ``ixrun/linear.py:84-86``).
    """
    if not torch.cuda.is_available():
        raise RuntimeError("decode_weight_triton runs the HIP kernel and needs the GPU; "
                           "decode_weight_scatter is the CPU decoder")
    device = torch.device(device) if device is not None else torch.device("cuda")
    dp = _lib.DevicePacked.from_dict(packed, device)
    out = torch.empty(packed["N"], dtype=torch.bfloat16, device=device)
    if packed["N"]:
        table = dp.prefix_build(TRITON_BLOCK)
        dp.decode(table, TRITON_BLOCK, out_bf16=out)
    return out.view(packed["out_f"], packed["in_f"]).to(dtype)


@torch.no_grad()
def decode_int8(packed: dict, device=None) -> torch.Tensor:
    """The int8 values themselves, ``[out_f, in_f]`` on the GPU (no reference
    counterpart; used to show the decode is bit-exact before any scaling)."""
    device = torch.device(device) if device is not None else torch.device("cuda")
    dp = _lib.DevicePacked.from_dict(packed, device)
    out = torch.empty(packed["N"], dtype=torch.int8, device=device)
    if packed["N"]:
        table = dp.prefix_build(TRITON_BLOCK)
        dp.decode(table, TRITON_BLOCK, out_i8=out)
    return out.view(packed["out_f"], packed["in_f"])
