"""Bit-stream layout of the INT8-X packed tensors (host side).

A stream of ``bits``-wide unsigned codes is the little-endian bit string
``code[0] | code[1] << bits | code[2] << 2*bits | ...`` cut into 32-bit words
and stored as ``torch.int32`` (word 0 holds string bits 0..31, bit 0 is the
LSB).  The tail of the last word is zero.  This is the layout defined by the
reference's ``ixrun/bitpack.py:13-61`` (packer), ``:64-84`` (unpacker) and
``:87-89`` (bitmap = 1-bit stream), and it is what the gfx950 kernels read.

The packer works on groups of 32 codes, which always fill exactly ``bits``
whole words, so no per-bit expansion is materialised.
"""
from __future__ import annotations

import numpy as np
import torch

__all__ = ["pack_bits_stream", "unpack_bits_stream", "pack_bitmap"]

_GROUP = 32  # 32 codes of any width end on a word boundary


def pack_bits_stream(vals: torch.Tensor, bits: int, chunk_vals: int = 1 << 21) -> torch.Tensor:
    """Pack integer codes (low ``bits`` bits of each value) into int32 words.

    Same contract as the reference's ``pack_bits_stream``
    (``ixrun/bitpack.py:13-61``): ``bits <= 0`` raises ``ValueError``; an empty
    input gives an empty int32 tensor; the result is a 1-D CPU ``torch.int32``
    tensor of ``ceil(n * bits / 32)`` words.  ``chunk_vals`` only bounds the
    size of the temporaries; it does not change the output.
    """
    if bits <= 0:
        raise ValueError("bits must be positive")
    if bits > 32:
        raise ValueError("bits must be at most 32")
    flat = vals.detach().reshape(-1).to("cpu", torch.int64).numpy()
    n = flat.size
    if n == 0:
        return torch.zeros(0, dtype=torch.int32)

    total_words = (n * bits + 31) // 32
    if bits == 1:
        # one bit per code: numpy's little-endian bit packer gives the same bytes
        packed = np.packbits((flat & 1).astype(np.uint8), bitorder="little")
        raw = np.zeros(total_words * 4, dtype=np.uint8)
        raw[: packed.size] = packed
        return torch.from_numpy(raw.view("<u4").astype(np.uint32).view(np.int32))
    out = np.empty(total_words, dtype=np.uint32)
    step = max(int(chunk_vals), _GROUP)
    step = (step + _GROUP - 1) // _GROUP * _GROUP
    code_mask = np.uint64((1 << bits) - 1)
    word_mask = np.uint64(0xFFFFFFFF)

    for start in range(0, n, step):
        piece = flat[start : start + step].astype(np.uint64) & code_mask
        groups = (piece.size + _GROUP - 1) // _GROUP
        if groups * _GROUP != piece.size:
            piece = np.concatenate([piece, np.zeros(groups * _GROUP - piece.size, np.uint64)])
        piece = piece.reshape(groups, _GROUP)
        words = np.zeros((groups, bits), dtype=np.uint64)
        for i in range(_GROUP):
            off = i * bits
            j, s = off >> 5, off & 31
            col = piece[:, i]
            words[:, j] |= (col << np.uint64(s)) & word_mask
            if s + bits > 32:
                words[:, j + 1] |= col >> np.uint64(32 - s)
        w0 = start * bits // 32
        take = min(groups * bits, total_words - w0)
        out[w0 : w0 + take] = words.reshape(-1)[:take].astype(np.uint32)
    return torch.from_numpy(out.view(np.int32))


def unpack_bits_stream(packed: torch.Tensor, n_elements: int, bits: int, device=None) -> torch.Tensor:
    """Inverse of :func:`pack_bits_stream`: the first ``n_elements`` codes.

    Same contract as the reference's ``unpack_bits_stream``
    (``ixrun/bitpack.py:64-84``): returns a 1-D int32 tensor on ``device``
    (default: where ``packed`` lives); ``n_elements == 0`` gives an empty one.
    """
    dev = torch.device(device) if device is not None else packed.device
    if n_elements == 0:
        return torch.zeros(0, dtype=torch.int32, device=dev)
    words = packed.to(dev).reshape(-1).to(torch.int64) & 0xFFFFFFFF
    last = words.numel() - 1
    out = torch.empty(n_elements, dtype=torch.int32, device=dev)
    code_mask = (1 << bits) - 1
    step = 1 << 22
    for start in range(0, n_elements, step):
        stop = min(start + step, n_elements)
        bitpos = torch.arange(start, stop, device=dev, dtype=torch.int64) * bits
        j = bitpos >> 5
        s = bitpos & 31
        lo = words[j] >> s
        hi = words[torch.clamp(j + 1, max=last)] << (32 - s)
        out[start:stop] = ((lo | hi) & code_mask).to(torch.int32)
    return out


def pack_bitmap(mask: torch.Tensor) -> torch.Tensor:
    """A boolean mask as a 1-bit stream (reference ``ixrun/bitpack.py:87-89``)."""
    return pack_bits_stream(mask.to(torch.int32), 1)
