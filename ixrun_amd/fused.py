"""Fused decode+GEMV: the single-token (and small-batch) hot path.

``y[n] = sum_k x[k] * W[n, k]`` with ``W`` decoded from the packed streams
inside the kernel, so the bf16 weight never exists in memory.  This module
keeps the names and call signatures of the reference's ``ixrun/fused.py``
(``fused_gemv`` ``:297-347``, ``compute_row_prefixes`` ``:35-78``,
``_pick_config`` ``:182-193``, ``_pick_split`` ``:196-203``, ``FUSED_TILE``
``:24``); the kernels behind it are the gfx950 HIP kernels of ``libixhip.so``.
"""
from __future__ import annotations

import weakref

import numpy as np
import torch

from . import _lib

__all__ = ["fused_gemv", "compute_row_prefixes", "FUSED_TILE"]

FUSED_TILE = 512  # flat elements per rank-table unit of the specialised kernel


# --------------------------------------------------------------------------- #
#  host-side rank tables
# --------------------------------------------------------------------------- #
_POP8 = np.array([bin(i).count("1") for i in range(256)], dtype=np.uint8)


class _Rank1:
    """rank1(pos) = number of set bits below bit ``pos`` of a packed bitmap."""

    def __init__(self, words: torch.Tensor):
        self.w = np.ascontiguousarray(words.detach().cpu().numpy()).view(np.uint32)
        per_word = _POP8[self.w.view(np.uint8)].reshape(-1, 4).sum(axis=1, dtype=np.int64)
        self.before = np.concatenate([[0], np.cumsum(per_word)])  # set bits in words [0, j)

    def __call__(self, pos: np.ndarray) -> np.ndarray:
        pos = np.asarray(pos, dtype=np.int64)
        j = np.minimum(pos >> 5, self.w.size)
        inside = np.where(j < self.w.size, self.w[np.minimum(j, max(self.w.size - 1, 0))] if self.w.size else 0, 0)
        low = inside.astype(np.uint64) & ((np.uint64(1) << (pos & 31).astype(np.uint64)) - np.uint64(1))
        low32 = low.astype(np.uint32)
        return self.before[j] + _POP8[low32.view(np.uint8).reshape(-1, 4)].sum(axis=1, dtype=np.int64)


def rank_prefixes_at(packed: dict, positions: np.ndarray) -> list:
    """For every level but the last: how many of its elements precede each flat position."""
    space = np.asarray(positions, dtype=np.int64)
    out = []
    for bm in packed["bitmaps"]:
        c = _Rank1(bm)(space) if bm.numel() else np.zeros_like(space)
        out.append(c)
        space = space - c  # the same positions, in the next bitmap's index space
    return out


def compute_row_prefixes(packed: dict, chunk: int | None = None) -> tuple:
    """Global stream ranks at row (or row-chunk) starts, as CPU int32 tensors.

    ``chunk=None``: one entry per row, the number of level-1 / level-2 elements
    strictly before the row (reference ``ixrun/fused.py:60-65``).  ``chunk=C``:
    one entry per ``(row, c*C)`` boundary, ``in_f // C`` per row (``:67-78``).
    One array is returned per bitmap, i.e. ``(q1, q2)`` for a three-level
    scheme.  Ranks come from word popcounts; no per-element array is built.
    """
    out_f, in_f = packed["out_f"], packed["in_f"]
    rows = np.arange(out_f, dtype=np.int64)[:, None] * in_f
    if chunk is None:
        pos = rows.reshape(-1)
    else:
        pos = (rows + np.arange(in_f // chunk, dtype=np.int64)[None, :] * chunk).reshape(-1)
    return tuple(torch.from_numpy(c.astype(np.int32)) for c in rank_prefixes_at(packed, pos))


def _pick_config(out_f: int, in_f: int) -> tuple:
    """(waves, tile) the reference would launch with (``ixrun/fused.py:182-193``).

    Kept for callers that import it; the HIP kernels size their own launches.
    """
    if out_f < in_f and in_f % 1024 == 0:
        return 2, 1024
    if out_f > in_f:
        return 2, 512
    return 4, 512


def _pick_split(in_f: int) -> int:
    """Split factor of the reference's split-K path (``ixrun/fused.py:196-203``):
    the first of 2, 4 whose chunk is a whole number of 512-tiles, else 1."""
    for s in (2, 4):
        if in_f % s == 0 and (in_f // s) % FUSED_TILE == 0:
            return s
    return 1


# --------------------------------------------------------------------------- #
#  device tables for tensors handed in loose (the reference's calling style)
# --------------------------------------------------------------------------- #
def pick_unit(in_f: int) -> int:
    """Rank-table unit for a layer: 512 when rows are whole 512-tiles (the
    specialised kernel), else the largest divisor of in_f up to 1024."""
    if in_f % FUSED_TILE == 0:
        return FUSED_TILE
    for c in range(min(in_f, 1024), 0, -1):
        if in_f % c == 0:
            return c
    return max(in_f, 1)


_loose_cache: dict = {}  # id(b1) -> (weakref to b1, signature, rank table, unit); the entry dies with b1


def _tables_for(b1, b2, l1, l2, l3, scale, out_f, in_f):
    """DevicePacked + rank table for loose (3,5,8) tensors.  The table is remembered for as long as ``b1`` lives
    (a weak reference: the cache keeps no packed tensor alive); the argument struct is rebuilt from the live
    tensors on every call."""
    dp = _lib.DevicePacked((3, 5, 8), out_f, in_f, [b1, b2], [l1, l2, l3], scale.reshape(1))
    key = id(b1)
    sig = (b1.data_ptr(), b2.data_ptr(), l1.data_ptr(), l2.data_ptr(), l3.data_ptr(), scale.data_ptr(),
           b1._version, b2._version, out_f, in_f)
    hit = _loose_cache.get(key)
    if hit is not None and hit[0]() is b1 and hit[1] == sig:
        return dp, hit[2], hit[3]
    unit = pick_unit(in_f)
    table = dp.prefix_build(unit)
    _loose_cache[key] = (weakref.ref(b1, lambda _ref, _key=key: _loose_cache.pop(_key, None)), sig, table, unit)
    return dp, table, unit


_workspaces: dict = {}  # device -> the scratch in use
_retired: list = []     # replaced scratches: graphs captured earlier still write their partial sums there


def shared_workspace(device, nbytes: int) -> torch.Tensor | None:
    """One fp32 scratch per device for the partial sums of the kernels that combine pieces of a row.

    Layers run one after another on the device's stream and every kernel pair writes its partial sums before it
    reads them, so the layers share it (callers that run layers on several streams of one device at once must give
    ``gemv`` / ``gemm`` workspaces of their own).  It only grows, to at least twice its size, and a replaced buffer
    is never freed: a hipGraph captured earlier holds its address and goes on using it.  ``StreamingLinear`` asks
    for the size of its widest fused call when it is built, so a deployed model does not grow it afterwards."""
    if nbytes == 0:
        return None
    device = torch.device(device)
    ws = _workspaces.get(device)
    if ws is None or ws.numel() * 4 < nbytes:
        if ws is not None:
            _retired.append(ws)
            nbytes = max(nbytes, ws.numel() * 8)
        ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=device)
        _workspaces[device] = ws
    return ws


def fused_gemv(x, b1, b2, l1, l2, l3, q1, q2, scale, out_f: int, in_f: int,
               chunk: int = 0, y32: torch.Tensor | None = None):
    """``y = x @ W.T`` for one token with ``W`` decoded on the fly.

    Signature and results of the reference's ``fused_gemv``
    (``ixrun/fused.py:297-347``): ``x`` is bf16 with ``in_f`` elements;
    ``chunk == 0`` returns a new bf16 ``[out_f]``; ``chunk > 0`` adds the fp32
    dot products into the caller-zeroed ``y32`` with atomics and returns it.
    ``q1``/``q2`` are the reference's row (or half-row) rank tables; the HIP
    kernels work from a finer table of their own, derived from the bitmaps on
    first use and remembered for as long as ``b1`` lives, so ``q1``/``q2`` are
    only checked for shape.  Empty levels need no dummy tensors.
    """
    if x.dtype != torch.bfloat16:
        raise TypeError("fused_gemv takes bf16 activations")
    if x.numel() != in_f:
        raise ValueError(f"x has {x.numel()} elements, in_f is {in_f}")
    want = out_f * (in_f // chunk if chunk > 0 else 1)
    if q1.numel() != want or q2.numel() != want:
        raise ValueError(f"rank tables have {q1.numel()}/{q2.numel()} entries, expected {want}")
    dp, table, unit = _tables_for(b1, b2, l1, l2, l3, scale, out_f, in_f)
    xf = x.reshape(1, in_f)
    if chunk > 0:
        if y32 is None or y32.dtype != torch.float32 or y32.numel() != out_f:
            raise ValueError("the split path needs a fp32 y32 of out_f elements")
        dp.gemv(table, unit, xf, y32=y32, flags=_lib.IXH_GEMV_ATOMIC)
        return y32
    y = torch.empty(out_f, dtype=torch.bfloat16, device=x.device)
    ws = shared_workspace(x.device, dp.gemv_workspace_bytes(unit, 1))
    dp.gemv(table, unit, xf, y=y, workspace=ws)
    return y
