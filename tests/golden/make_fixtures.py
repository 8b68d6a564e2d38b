"""Writes tests/golden/codec_fixtures.npz: small known-answer tensors of the INT8-X codec.

Run from the repository root:  python tests/golden/make_fixtures.py

For each of the schemes (3,5,8) and (3,4,5,6,8): an 8 x 512 int8 tensor that holds every boundary value of every
level (0, +-3, +-4, +-7, +-8, +-15, +-16, +-31, +-32, +-127) and a fixed pseudo-random filling, its packed form
(bitmaps, code streams, last-level bytes, level counts), the rank table at unit 512, the decoded bf16 weights for the
scale 0.0123046875, three activation rows and their fp64 products.  The values come from this file's own integer
generator (no library RNG), the packed bytes from the CPU oracle; the tests compare the oracle, the package's host
codec and the HIP kernels against the stored arrays, so a change of any of them that alters a byte shows up here.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import ix_oracle  # noqa: E402

OUT_F, IN_F, ROWS = 8, 512, 3
SCALE_BITS = 0x3C4A  # bf16 0.0123046875
BOUNDARY = [0, 3, -3, 4, -4, 7, -7, 8, -8, 15, -15, 16, -16, 31, -31, 32, -32, 127, -127, 1, -1, 2, -2]


def lcg(seed):
    state = seed
    while True:
        state = (state * 1103515245 + 12345) % (1 << 31)
        yield state >> 8


def values(seed):
    g = lcg(seed)
    n = OUT_F * IN_F
    q = np.zeros(n, dtype=np.int64)
    for i in range(n):
        r = next(g) % 1000
        # about 60 % within +-3, 25 % within +-15, 10 % within +-31, the rest up to +-127
        span = 3 if r < 600 else (15 if r < 850 else (31 if r < 950 else 127))
        q[i] = next(g) % (2 * span + 1) - span
    for j, v in enumerate(BOUNDARY):  # boundary values at word starts, word ends and across unit borders
        q[j * 37 % n] = v
        q[(n - 1 - j * 41) % n] = v
        if j < OUT_F:
            q[(j + 1) * IN_F - 1] = v  # the last element of a row
    return q.astype(np.int8)


def activations(seed):
    g = lcg(seed)
    x = np.zeros(ROWS * IN_F, dtype=np.float32)
    for i in range(x.size):
        x[i] = (next(g) % 2001 - 1000) / 512.0
    return ix_oracle.f32_to_bf16_bits(x).reshape(ROWS, IN_F)


def main():
    out = {"scale_bits": np.array([SCALE_BITS], dtype=np.uint16)}
    for name, bits in (("s358", (3, 5, 8)), ("s34568", (3, 4, 5, 6, 8))):
        q = values(len(bits))
        e = ix_oracle.encode(q, bits)
        assert np.array_equal(ix_oracle.decode_i8(q.size, bits, e["bitmaps"], e["streams"], e["last"]), q)
        w = ix_oracle.dequant_bf16(q, SCALE_BITS).reshape(OUT_F, IN_F)
        x = activations(7 + len(bits))
        out[f"{name}_bits"] = np.array(bits, dtype=np.int32)
        out[f"{name}_q"] = q.reshape(OUT_F, IN_F)
        for i, b in enumerate(e["bitmaps"]):
            out[f"{name}_bitmap{i}"] = b
        for i, s in enumerate(e["streams"]):
            out[f"{name}_stream{i}"] = s
        out[f"{name}_last"] = e["last"]
        out[f"{name}_counts"] = np.array(e["counts"], dtype=np.int64)
        out[f"{name}_table512"] = ix_oracle.prefix(q.size, len(bits), e["bitmaps"], 512)
        out[f"{name}_w_bf16"] = w
        out[f"{name}_x_bf16"] = x
        out[f"{name}_y_f64"] = ix_oracle.gemm_f64(w, x)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "codec_fixtures.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
