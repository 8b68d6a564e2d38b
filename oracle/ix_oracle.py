"""ctypes front end of the C oracle (``ix_oracle.c``) with numpy in and out.

TEST INFRASTRUCTURE ONLY.  Imported by ``tests/``, by the smoke check and by
the CPU-baseline leg of ``bench.py``; the package never imports it.  The C file
lists which reference lines each function restates and what pins it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libixoracle.so")
_lib = None

_u32p = C.POINTER(C.c_uint32)
_pp = C.POINTER(_u32p)


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a second or two)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libixoracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.ixo_encode.restype = C.c_int64
        _lib.ixo_f32_to_bf16.restype = C.c_uint16
        _lib.ixo_f32_to_bf16.argtypes = [C.c_float]
        _lib.ixo_bf16_to_f32.restype = C.c_float
        _lib.ixo_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.ixo_f32_to_f16.restype = C.c_uint16
        _lib.ixo_f32_to_f16.argtypes = [C.c_float]
        _lib.ixo_f16_to_f32.restype = C.c_float
        _lib.ixo_f16_to_f32.argtypes = [C.c_uint16]
    return _lib


def _ptr(a, ty):
    return a.ctypes.data_as(C.POINTER(ty))


def _ptr_array(arrs):
    holder = (_u32p * 8)()
    for i, a in enumerate(arrs):
        holder[i] = _ptr(a, C.c_uint32)
    return holder


def _threshold(bits: int) -> int:
    return (1 << (bits - 1)) - 1


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even bf16 bit patterns of an fp32 array (numpy twin of the C helper)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def bf16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def pack_bits(codes: np.ndarray, bits: int) -> np.ndarray:
    codes = np.ascontiguousarray(codes, dtype=np.uint32)
    words = np.zeros((codes.size * bits + 31) // 32 + 1, dtype=np.uint32)
    lib().ixo_pack_bits(_ptr(codes, C.c_uint32), C.c_int64(codes.size), C.c_int(bits), _ptr(words, C.c_uint32))
    return words[:-1]


def unpack_bits(words: np.ndarray, n: int, bits: int) -> np.ndarray:
    words = np.concatenate([np.ascontiguousarray(words, dtype=np.uint32), np.zeros(1, np.uint32)])
    out = np.zeros(n, dtype=np.uint32)
    lib().ixo_unpack_bits(_ptr(words, C.c_uint32), C.c_int64(n), C.c_int(bits), _ptr(out, C.c_uint32))
    return out


def quantize_bf16(w_bits: np.ndarray):
    """bf16 bit patterns (uint16, any shape) -> (scale bf16 bits, int8 flat)."""
    w = np.ascontiguousarray(w_bits, dtype=np.uint16).reshape(-1)
    q = np.zeros(w.size, dtype=np.int8)
    scale = C.c_uint16(0)
    lib().ixo_quantize_bf16(_ptr(w, C.c_uint16), C.c_int64(w.size), C.byref(scale), _ptr(q, C.c_int8))
    return int(scale.value), q


def encode(q: np.ndarray, level_bits=(3, 5, 8)) -> dict:
    """int8 flat -> dict(bitmaps=[u32], streams=[u32...], last=u8, counts, total_bytes)."""
    q = np.ascontiguousarray(q, dtype=np.int8).reshape(-1)
    level_bits = tuple(level_bits)
    nl = len(level_bits)
    lb = (C.c_int * nl)(*level_bits)
    counts = (C.c_int64 * nl)()
    lib().ixo_count_levels(_ptr(q, C.c_int8), C.c_int64(q.size), lb, C.c_int(nl), counts)
    counts = list(counts)
    bitmaps, streams = [], []
    remaining = q.size
    for i in range(nl - 1):
        bitmaps.append(np.zeros((remaining + 31) // 32, dtype=np.uint32))
        # one spare word: a code that ends exactly on the last word boundary
        # never touches it, and the C walker may OR a zero into it
        streams.append(np.zeros((counts[i] * level_bits[i] + 31) // 32 + 1, dtype=np.uint32))
        remaining -= counts[i]
    last = np.zeros(counts[-1], dtype=np.uint8)
    cnt_arr = (C.c_int64 * nl)(*counts)
    total = lib().ixo_encode(
        _ptr(q, C.c_int8), C.c_int64(q.size), lb, C.c_int(nl),
        _ptr_array(bitmaps), _ptr_array(streams), _ptr(last, C.c_uint8), cnt_arr,
    )
    streams = [s[:-1] for s in streams]
    return {
        "level_bits": level_bits, "N": int(q.size), "bitmaps": bitmaps, "streams": streams,
        "last": last, "counts": counts, "total_bytes": int(total),
    }


def _as_u32(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if a.dtype == np.int32:
        a = a.view(np.uint32)
    return np.ascontiguousarray(a, dtype=np.uint32)


def _padded(arrs):
    # readers look one word past a code that straddles the final boundary only
    # when it does straddle; one zero word of slack keeps every read in bounds
    return [np.concatenate([_as_u32(a), np.zeros(1, np.uint32)]) for a in arrs]


def decode_i8(n: int, level_bits, bitmaps, streams, last) -> np.ndarray:
    nl = len(level_bits)
    lb = (C.c_int * nl)(*level_bits)
    bms, sts = _padded(bitmaps), _padded(streams)
    last = np.ascontiguousarray(last, dtype=np.uint8)
    q = np.zeros(n, dtype=np.int8)
    lib().ixo_decode_i8(C.c_int64(n), lb, C.c_int(nl), _ptr_array(bms), _ptr_array(sts),
                        _ptr(last, C.c_uint8), _ptr(q, C.c_int8))
    return q


def dequant_bf16(q: np.ndarray, scale_bits: int) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.int8).reshape(-1)
    w = np.zeros(q.size, dtype=np.uint16)
    lib().ixo_dequant_bf16(_ptr(q, C.c_int8), C.c_int64(q.size), C.c_uint16(scale_bits), _ptr(w, C.c_uint16))
    return w


def prefix(n: int, n_levels: int, bitmaps, chunk: int) -> np.ndarray:
    """int32 [n_levels-1, ceil(n/chunk)+1] exclusive level counts at flat positions u*chunk."""
    n_units = (n + chunk - 1) // chunk
    out = np.zeros((n_levels - 1, n_units + 1), dtype=np.int32)
    bms = _padded(bitmaps)
    lib().ixo_prefix(C.c_int64(n), C.c_int(n_levels), _ptr_array(bms), C.c_int64(chunk), _ptr(out, C.c_int32))
    return out


def gemm_f64(w_bits: np.ndarray, x_bits: np.ndarray) -> np.ndarray:
    """w bf16 bits [out_f,in_f], x bf16 bits [M,in_f] -> float64 [M,out_f]."""
    w = np.ascontiguousarray(w_bits, dtype=np.uint16)
    x = np.ascontiguousarray(x_bits, dtype=np.uint16).reshape(-1, w.shape[1])
    y = np.zeros((x.shape[0], w.shape[0]), dtype=np.float64)
    lib().ixo_gemm_f64(_ptr(w, C.c_uint16), C.c_int64(w.shape[0]), C.c_int64(w.shape[1]),
                       _ptr(x, C.c_uint16), C.c_int64(x.shape[0]), _ptr(y, C.c_double))
    return y


def gemm_f32(w_bits: np.ndarray, x_bits: np.ndarray) -> np.ndarray:
    w = np.ascontiguousarray(w_bits, dtype=np.uint16)
    x = np.ascontiguousarray(x_bits, dtype=np.uint16).reshape(-1, w.shape[1])
    y = np.zeros((x.shape[0], w.shape[0]), dtype=np.uint16)
    lib().ixo_gemm_f32(_ptr(w, C.c_uint16), C.c_int64(w.shape[0]), C.c_int64(w.shape[1]),
                       _ptr(x, C.c_uint16), C.c_int64(x.shape[0]), _ptr(y, C.c_uint16))
    return y


def fused_gemv_f32(out_f, in_f, level_bits, bitmaps, streams, last, scale_bits, x_bits) -> np.ndarray:
    nl = len(level_bits)
    lb = (C.c_int * nl)(*level_bits)
    bms, sts = _padded(bitmaps), _padded(streams)
    last = np.ascontiguousarray(last, dtype=np.uint8)
    x = np.ascontiguousarray(x_bits, dtype=np.uint16).reshape(-1)
    y = np.zeros(out_f, dtype=np.uint16)
    lib().ixo_fused_gemv_f32(C.c_int64(out_f), C.c_int64(in_f), lb, C.c_int(nl), _ptr_array(bms),
                             _ptr_array(sts), _ptr(last, C.c_uint8), C.c_uint16(scale_bits),
                             _ptr(x, C.c_uint16), _ptr(y, C.c_uint16))
    return y


# ---- torch conveniences for the tests (torch only carries the arrays) ----
def packed_to_numpy(packed: dict) -> dict:
    """A package/reference packed dict (torch tensors) as the oracle's numpy view."""
    import torch

    scale_bits = int(packed["scale"].reshape(1).view(torch.int16).item()) & 0xFFFF
    return {
        "level_bits": tuple(packed["level_bits"]), "N": packed["N"], "out_f": packed["out_f"],
        "in_f": packed["in_f"], "scale_bits": scale_bits,
        "bitmaps": [_as_u32(b.cpu().numpy()) for b in packed["bitmaps"]],
        "streams": [_as_u32(s.cpu().numpy()) for s in packed["streams"][:-1]],
        "last": packed["streams"][-1].cpu().numpy().astype(np.uint8),
        "counts": list(packed["counts"]),
    }


def decode_packed_i8(packed: dict) -> np.ndarray:
    p = packed_to_numpy(packed)
    return decode_i8(p["N"], p["level_bits"], p["bitmaps"], p["streams"], p["last"])


def decode_packed_bf16(packed: dict) -> np.ndarray:
    p = packed_to_numpy(packed)
    q = decode_i8(p["N"], p["level_bits"], p["bitmaps"], p["streams"], p["last"])
    return dequant_bf16(q, p["scale_bits"]).reshape(p["out_f"], p["in_f"])


# ---- group-scale sibling format (reference: ixgs/) ----

def gs_quantize(w_bits: np.ndarray, group: int = 64):
    """bf16 bit patterns -> (fp16 scale bits [ceil(n/group)], int16 values in [-127, 128])."""
    w = np.ascontiguousarray(w_bits, dtype=np.uint16).reshape(-1)
    scales = np.zeros((w.size + group - 1) // group, dtype=np.uint16)
    q = np.zeros(w.size, dtype=np.int16)
    lib().ixo_gs_quantize(_ptr(w, C.c_uint16), C.c_int64(w.size), C.c_int64(group), _ptr(scales, C.c_uint16),
                          _ptr(q, C.c_int16))
    return scales, q


def gs_encode(q: np.ndarray) -> dict:
    """int16 values -> dict(b1, b2, l1, l2 as uint32 words, l3 bytes, counts), unpadded."""
    q = np.ascontiguousarray(q, dtype=np.int16).reshape(-1)
    in1 = (q >= -3) & (q <= 4)
    in2 = ~in1 & (q >= -15) & (q <= 16)
    n1, n2 = int(in1.sum()), int(in2.sum())
    n3 = q.size - n1 - n2
    b1 = np.zeros((q.size + 31) // 32, dtype=np.uint32)
    b2 = np.zeros((n2 + n3 + 31) // 32 + 1, dtype=np.uint32)
    l1 = np.zeros((n1 * 3 + 31) // 32 + 1, dtype=np.uint32)
    l2 = np.zeros((n2 * 5 + 31) // 32 + 1, dtype=np.uint32)
    l3 = np.zeros(max(n3, 1), dtype=np.uint8)
    counts = (C.c_int64 * 3)()
    lib().ixo_gs_encode(_ptr(q, C.c_int16), C.c_int64(q.size), _ptr(b1, C.c_uint32), _ptr(b2, C.c_uint32),
                        _ptr(l1, C.c_uint32), _ptr(l2, C.c_uint32), _ptr(l3, C.c_uint8), counts)
    assert list(counts) == [n1, n2, n3]
    return {"N": int(q.size), "b1": b1, "b2": b2[:-1], "l1": l1[:-1], "l2": l2[:-1], "l3": l3[:n3],
            "counts": [n1, n2, n3]}


def gs_decode_i16(n: int, b1, b2, l1, l2, l3) -> np.ndarray:
    pad = lambda a: np.concatenate([_as_u32(a), np.zeros(1, np.uint32)])
    l3 = np.concatenate([np.ascontiguousarray(l3, dtype=np.uint8), np.zeros(1, np.uint8)])
    q = np.zeros(n, dtype=np.int16)
    b1, b2, l1, l2 = pad(b1), pad(b2), pad(l1), pad(l2)
    lib().ixo_gs_decode_i16(C.c_int64(n), _ptr(b1, C.c_uint32), _ptr(b2, C.c_uint32), _ptr(l1, C.c_uint32),
                            _ptr(l2, C.c_uint32), _ptr(l3, C.c_uint8), _ptr(q, C.c_int16))
    return q


def gs_dequant_bf16(q: np.ndarray, scales: np.ndarray, group: int = 64) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.int16).reshape(-1)
    scales = np.ascontiguousarray(scales, dtype=np.uint16)
    w = np.zeros(q.size, dtype=np.uint16)
    lib().ixo_gs_dequant_bf16(_ptr(q, C.c_int16), C.c_int64(q.size), C.c_int64(group), _ptr(scales, C.c_uint16),
                              _ptr(w, C.c_uint16))
    return w
