"""Seeded inputs shared by the tests (torch only carries the arrays)."""
from __future__ import annotations

import numpy as np
import torch


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> uint16 bit patterns (numpy has no bf16)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bits_to_bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint16).view(np.int16)).view(torch.bfloat16)


def student_t_weight(out_f: int, in_f: int, seed: int = 0) -> torch.Tensor:
    """Student-t(nu=4) scaled to std 0.02, CPU generator: the benchmark's weight recipe."""
    g = torch.Generator("cpu").manual_seed(seed)
    z = torch.randn(out_f, in_f, generator=g)
    chi = sum(torch.randn(out_f, in_f, generator=g) ** 2 for _ in range(4))
    return (z / torch.sqrt(chi / 4) * (0.02 / 2 ** 0.5)).bfloat16()


def outlier_weight(out_f: int, in_f: int, seed: int = 0) -> torch.Tensor:
    """The reference tests' recipe (tests/test_fused.py:17-22): N(0, 0.005) with a
    random 4 % of entries overwritten by N(0, 0.05)."""
    g = torch.Generator("cpu").manual_seed(seed)
    base = torch.randn(out_f, in_f, generator=g) * 0.005
    flat = base.view(-1)
    n_out = int(flat.numel() * 0.04)
    idx = torch.randperm(flat.numel(), generator=g)[:n_out]
    flat[idx] = torch.randn(n_out, generator=g) * 0.05
    return base.bfloat16()


def calibrated_weight(out_f: int, in_f: int, seed: int = 0, fractions=(0.55, 0.40, 0.05),
                      scale: float = 2.0 ** -9) -> tuple:
    """Weights whose int8 values fall into the (3,5,8) levels with the given
    fractions: levels drawn categorically, magnitudes uniform inside the level,
    random sign, one +-127 forced so that max|w|/127 gives back ``scale``.
    Returns (bf16 weight, int8 values).  ``scale`` must be a bf16 value; with a
    power of two every v*scale is exact in bf16, with any other bf16 scale the
    dequantisation rounds."""
    rng = np.random.default_rng(seed)
    n = out_f * in_f
    lvl = rng.choice(3, size=n, p=list(fractions))
    lo = np.array([0, 4, 16])[lvl]
    hi = np.array([3, 15, 127])[lvl]
    mag = rng.integers(lo, hi + 1)
    sign = rng.integers(0, 2, size=n) * 2 - 1
    v = (mag * sign).astype(np.int8)
    v[rng.integers(0, n)] = 127
    w = (torch.from_numpy(v.astype(np.float32)) * scale).bfloat16().view(out_f, in_f)
    return w, v


def activations(m: int, in_f: int, seed: int = 1) -> torch.Tensor:
    g = torch.Generator("cpu").manual_seed(seed)
    return torch.randn(m, in_f, generator=g).bfloat16()


def rel_l2(a: np.ndarray, b: np.ndarray) -> float:
    a = np.asarray(a, dtype=np.float64).reshape(-1)
    b = np.asarray(b, dtype=np.float64).reshape(-1)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def packed_from_int8(v: np.ndarray, out_f: int, in_f: int, scale: float = 0.0123046875, level_bits=(3, 5, 8)) -> dict:
    """A packed dictionary built straight from int8 values (through the oracle's
    encoder), for level mixes no quantized weight can have, e.g. no value above 3."""
    from oracle import ix_oracle

    e = ix_oracle.encode(np.asarray(v, dtype=np.int8).reshape(-1), level_bits)
    as_i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int32).copy())
    n = out_f * in_f
    return {
        "level_bits": tuple(level_bits), "out_f": out_f, "in_f": in_f, "N": n,
        "scale": torch.tensor(scale, dtype=torch.float32).bfloat16().reshape(()),
        "bitmaps": [as_i32(b) for b in e["bitmaps"]],
        "streams": [as_i32(s) for s in e["streams"]] + [torch.from_numpy(e["last"].copy())],
        "counts": e["counts"], "total_bytes": e["total_bytes"],
        "bits_per_weight": e["total_bytes"] * 8 / max(n, 1), "compression_vs_bf16": n * 2 / max(e["total_bytes"], 1),
    }


def int8_mix(kind: str, n: int, seed: int = 0) -> np.ndarray:
    """int8 values with a chosen level mix."""
    rng = np.random.default_rng(seed)
    sign = rng.integers(0, 2, size=n) * 2 - 1
    if kind == "only_l1":
        return rng.integers(-3, 4, size=n).astype(np.int8)
    if kind == "no_l3":
        return rng.integers(-15, 16, size=n).astype(np.int8)
    if kind == "no_l2":
        return np.where(rng.random(n) < 0.6, rng.integers(-3, 4, size=n), rng.integers(16, 128, size=n) * sign).astype(np.int8)
    if kind == "only_l3":
        return (rng.integers(16, 128, size=n) * sign).astype(np.int8)
    if kind == "rare_other":  # 99.8 % level 1, the rest split between levels 2 and 3
        v = rng.integers(-3, 4, size=n)
        hit = rng.random(n) < 0.002
        v[hit] = (np.where(rng.random(hit.sum()) < 0.7, rng.integers(4, 16, size=hit.sum()),
                           rng.integers(16, 128, size=hit.sum())) * sign[hit])
        return v.astype(np.int8)
    if kind == "five_dense":  # every level of (3,4,5,6,8) well populated: 40 / 25 / 20 / 10 / 5 %
        u = rng.random(n)
        mag = np.where(u < 0.40, rng.integers(0, 4, size=n),
              np.where(u < 0.65, rng.integers(4, 8, size=n),
              np.where(u < 0.85, rng.integers(8, 16, size=n),
              np.where(u < 0.95, rng.integers(16, 32, size=n), rng.integers(32, 128, size=n)))))
        return (mag * sign).astype(np.int8)
    raise KeyError(kind)
