"""Pins the CPU oracle (oracle/ix_oracle.c) and the package's host codec.

Three independent statements of the codec are compared: the C oracle (a single
forward walk), the package's vectorised torch/numpy encoder, and brute-force
Python written here from the definition.  Known answers come from the
reference's own tests and from a hand-derived 2x5 tensor.
"""
import numpy as np
import pytest
import torch

from ixrun_amd.bitpack import pack_bits_stream, unpack_bits_stream, pack_bitmap
from ixrun_amd.config import BIT_TO_THRESHOLD
from ixrun_amd.fused import compute_row_prefixes
from ixrun_amd.quantize import int8x_quantize, decode_to_weight, compute_positions
from ixrun_amd.triton_kernels import decode_weight_scatter

from helpers import bf16_bits, bits_to_bf16, student_t_weight, outlier_weight, calibrated_weight


def u32(t: torch.Tensor) -> np.ndarray:
    return t.numpy().view(np.uint32)


# ---------------------------------------------------------------- bit packing
def closed_form_words(codes, bits):
    """word[j] = sum_i code_i << (i*bits - 32 j), via one Python big integer."""
    big = 0
    for i, c in enumerate(codes):
        big |= int(c) << (i * bits)
    n_words = (len(codes) * bits + 31) // 32
    return np.array([(big >> (32 * j)) & 0xFFFFFFFF for j in range(n_words)], dtype=np.uint32)


def test_pack_known_answer(oracle):
    # 0..7 in 3 bits: 0 | 1<<3 | 2<<6 | ... | 7<<21
    assert oracle.pack_bits(np.arange(8), 3).tolist() == [0x00FAC688]
    assert u32(pack_bits_stream(torch.arange(8), 3)).tolist() == [0x00FAC688]


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("n", [1, 31, 32, 33, 64, 777, 1000])
def test_pack_closed_form(oracle, bits, n):
    rng = np.random.default_rng(bits * 1000 + n)
    codes = rng.integers(0, 1 << bits, size=n)
    want = closed_form_words(codes, bits)
    assert np.array_equal(oracle.pack_bits(codes, bits), want)
    assert np.array_equal(u32(pack_bits_stream(torch.from_numpy(codes), bits)), want)
    assert np.array_equal(oracle.unpack_bits(want, n, bits), codes)
    assert np.array_equal(unpack_bits_stream(torch.from_numpy(want.view(np.int32)), n, bits).numpy(), codes)


def test_pack_round_trips_of_reference_tests(oracle):
    # sizes of the reference's tests/test_core.py:15-35, incl. the multi-chunk 3-bit case
    g = torch.Generator().manual_seed(0)
    for bits, n in [(3, 1000), (5, 777), (3, 2_500_003)]:
        vals = torch.randint(0, 1 << bits, (n,), dtype=torch.int32, generator=g)
        packed = pack_bits_stream(vals, bits)
        assert packed.dtype == torch.int32 and packed.numel() == (n * bits + 31) // 32
        assert torch.equal(unpack_bits_stream(packed, n, bits), vals)
        assert np.array_equal(oracle.pack_bits(vals.numpy(), bits), u32(packed))
    # chunking must not change the result
    vals = torch.randint(0, 8, (100_003,), dtype=torch.int32, generator=g)
    assert torch.equal(pack_bits_stream(vals, 3, chunk_vals=64), pack_bits_stream(vals, 3))


def test_pack_errors_and_empty():
    with pytest.raises(ValueError):
        pack_bits_stream(torch.arange(4), 0)
    assert pack_bits_stream(torch.zeros(0, dtype=torch.int32), 3).numel() == 0
    assert unpack_bits_stream(torch.zeros(0, dtype=torch.int32), 0, 3).numel() == 0
    assert u32(pack_bitmap(torch.tensor([True, True, True, False, False, False, False, False, True, False]))).tolist() == [0x107]


# ---------------------------------------------------------------- hand-derived known answer
KAT_V = np.array([[0, 1, -3, 4, -15], [16, 127, -127, 3, 5]], dtype=np.int8)


def test_hand_known_answer(oracle):
    w = (torch.from_numpy(KAT_V.astype(np.float32)) * 2.0 ** -7).bfloat16()
    p = int8x_quantize(w)
    assert float(p["scale"]) == 2.0 ** -7 and p["scale"].dtype == torch.bfloat16 and p["scale"].dim() == 0
    assert u32(p["bitmaps"][0]).tolist() == [0x00000107]
    assert u32(p["bitmaps"][1]).tolist() == [0x00000023]
    assert u32(p["streams"][0]).tolist() == [0x00000C23]
    assert u32(p["streams"][1]).tolist() == [0x00005013]
    assert p["streams"][2].dtype == torch.uint8 and p["streams"][2].tolist() == [143, 254, 0]
    assert p["counts"] == [4, 3, 3] and p["total_bytes"] == 21 and p["N"] == 10
    assert p["bits_per_weight"] == 21 * 8 / 10 and p["compression_vs_bf16"] == 20 / 21
    assert list(p.keys()) == ["level_bits", "out_f", "in_f", "N", "scale", "bitmaps", "streams", "counts",
                              "total_bytes", "bits_per_weight", "compression_vs_bf16"]
    q1, q2 = compute_row_prefixes(p)
    assert q1.tolist() == [0, 3] and q2.tolist() == [0, 2] and q1.dtype == torch.int32

    # the C oracle from the int8 values alone
    scale_bits, q = oracle.quantize_bf16(bf16_bits(w))
    assert scale_bits == 0x3C00 and np.array_equal(q, KAT_V.reshape(-1))
    e = oracle.encode(q)
    assert [b.tolist() for b in e["bitmaps"]] == [[0x107], [0x23]]
    assert [s.tolist() for s in e["streams"]] == [[0xC23], [0x5013]]
    assert e["last"].tolist() == [143, 254, 0] and e["counts"] == [4, 3, 3] and e["total_bytes"] == 21
    assert np.array_equal(oracle.decode_i8(10, (3, 5, 8), e["bitmaps"], e["streams"], e["last"]), KAT_V.reshape(-1))
    assert oracle.prefix(10, 3, e["bitmaps"], 5).tolist() == [[0, 3, 4], [0, 2, 3]]


# ---------------------------------------------------------------- quantizer
def naive_int8(w: torch.Tensor):
    """Ground truth of the reference tests (tests/test_core.py:46-50,
    tests/test_int8_equivalence.py:29-33): plain per-tensor int8 and its dequantisation."""
    scale = w.abs().max().clamp(min=1e-8) / 127.0
    i8 = (w.float() / scale).round().clamp(-127, 127).to(torch.int8)
    return i8, (i8.float() * scale.bfloat16().float()).to(torch.bfloat16)


@pytest.mark.parametrize("maker,shape", [
    (lambda: (torch.randn(128, 256, generator=torch.Generator().manual_seed(42)) * 0.03).bfloat16(), (128, 256)),
    (lambda: student_t_weight(256, 512, seed=0), (256, 512)),
    (lambda: outlier_weight(192, 320, seed=3), (192, 320)),
    (lambda: torch.zeros(8, 40, dtype=torch.bfloat16), (8, 40)),
])
def test_quantize_matches_plain_int8(oracle, maker, shape):
    w = maker()
    i8_gt, w_gt = naive_int8(w)
    scale_bits, q = oracle.quantize_bf16(bf16_bits(w))
    assert np.array_equal(q, i8_gt.reshape(-1).numpy())
    assert np.array_equal(oracle.dequant_bf16(q, scale_bits), bf16_bits(w_gt).reshape(-1))
    p = int8x_quantize(w)
    assert bf16_bits(p["scale"].reshape(1))[0] == scale_bits
    for dec in (decode_to_weight(p), decode_weight_scatter(p, device="cpu")):
        assert dec.dtype == torch.bfloat16 and dec.shape == shape and torch.equal(dec, w_gt)
    assert np.array_equal(oracle.decode_packed_bf16(p), bf16_bits(w_gt))


def test_quantize_ties_and_clamp(oracle):
    # v*scale with scale 2^-7: x.5 ties must go to even, |v| > 127 cannot occur, -127 is kept
    vals = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.0, -127.0, 63.5], dtype=np.float32)
    w = (torch.from_numpy(vals) * 2.0 ** -7).bfloat16().reshape(1, -1)
    _, q = oracle.quantize_bf16(bf16_bits(w))
    i8_gt, _ = naive_int8(w)
    assert np.array_equal(q, i8_gt.reshape(-1).numpy())
    assert q[:6].tolist() == [0, 2, 2, 0, -2, -2]


def test_last_level_must_be_8():
    with pytest.raises(ValueError):
        int8x_quantize(torch.zeros(4, 4, dtype=torch.bfloat16), (3, 5))
    assert int8x_quantize(torch.zeros(4, 4, dtype=torch.bfloat16), (8, 5, 3))["level_bits"] == (3, 5, 8)


# ---------------------------------------------------------------- encoder / decoder
def brute_force_encode(q, level_bits):
    """Straight from the definition, one element at a time."""
    T = [BIT_TO_THRESHOLD[b] for b in level_bits]
    L = len(level_bits)
    bm_bits = [[] for _ in range(L - 1)]
    codes = [[] for _ in range(L)]
    for v in q.tolist():
        lv = next((i for i in range(L - 1) if abs(v) <= T[i]), L - 1)
        for i in range(min(lv + 1, L - 1)):
            bm_bits[i].append(1 if i == lv else 0)
        codes[lv].append(v + T[lv])
    return bm_bits, codes


def brute_force_decode_element(p, bm_bits, codes, level_bits):
    """Rank by linear scan: r_0 = p, c_i = ones of bitmap i below r_i, r_{i+1} = r_i - c_i."""
    r = p
    L = len(level_bits)
    for i in range(L - 1):
        c = sum(bm_bits[i][:r])
        if bm_bits[i][r]:
            return codes[i][c] - BIT_TO_THRESHOLD[level_bits[i]]
        r -= c
    return codes[L - 1][r] - 127


CORNER_VALUES = {
    "mixed": lambda rng, n: rng.integers(-127, 128, size=n),
    "small": lambda rng, n: rng.integers(-3, 4, size=n),          # no level 2, no level 3
    "no_l3": lambda rng, n: rng.integers(-15, 16, size=n),
    "no_l2": lambda rng, n: np.where(rng.random(n) < 0.5, rng.integers(-3, 4, size=n), rng.integers(16, 128, size=n)),
    "only_l3": lambda rng, n: rng.integers(16, 128, size=n) * (rng.integers(0, 2, size=n) * 2 - 1),
}


@pytest.mark.parametrize("kind", list(CORNER_VALUES))
@pytest.mark.parametrize("n", [1, 2, 31, 32, 33, 63, 64, 65, 96, 1000, 1024, 1025, 4096])
@pytest.mark.parametrize("level_bits", [(3, 5, 8), (3, 4, 5, 6, 8), (2, 8)])
def test_encode_decode_brute_force(oracle, kind, n, level_bits):
    rng = np.random.default_rng(hash((kind, n, level_bits)) % 2**32)
    q = CORNER_VALUES[kind](rng, n).astype(np.int8)
    e = oracle.encode(q, level_bits)
    bm_bits, codes = brute_force_encode(q, level_bits)
    L = len(level_bits)
    assert e["counts"] == [len(c) for c in codes] and sum(e["counts"]) == n
    for i in range(L - 1):
        assert np.array_equal(e["bitmaps"][i], closed_form_words(bm_bits[i], 1))
        assert np.array_equal(e["streams"][i], closed_form_words(codes[i], level_bits[i]))
    assert e["last"].tolist() == codes[L - 1]
    # byte accounting of quantize.py:99-108
    want_bytes = 2 + len(codes[L - 1]) + sum(4 * len(e["bitmaps"][i]) + 4 * len(e["streams"][i]) for i in range(L - 1))
    assert e["total_bytes"] == want_bytes
    dec = oracle.decode_i8(n, level_bits, e["bitmaps"], e["streams"], e["last"])
    assert np.array_equal(dec, q)
    if n <= 100:
        assert [brute_force_decode_element(p, bm_bits, codes, level_bits) for p in range(n)] == q.tolist()


@pytest.mark.parametrize("shape,level_bits", [((128, 256), (3, 5, 8)), ((64, 96), (3, 4, 5, 6, 8)), ((7, 33), (3, 5, 8)),
                                              ((5, 1024), (4, 8)), ((300, 17), (3, 5, 8))])
def test_package_encoder_equals_oracle(oracle, shape, level_bits):
    w = outlier_weight(*shape, seed=shape[0])
    p = int8x_quantize(w, level_bits)
    scale_bits, q = oracle.quantize_bf16(bf16_bits(w))
    e = oracle.encode(q, level_bits)
    assert p["counts"] == e["counts"] and p["total_bytes"] == e["total_bytes"]
    for a, b in zip(p["bitmaps"], e["bitmaps"]):
        assert np.array_equal(u32(a), b)
    for a, b in zip(p["streams"][:-1], e["streams"]):
        assert np.array_equal(u32(a), b)
    assert np.array_equal(p["streams"][-1].numpy(), e["last"])
    assert np.array_equal(oracle.decode_packed_i8(p), q)
    # positions partition 0..N-1 (reference tests/test_core.py:84-94)
    pos = compute_positions(p)
    assert [len(x) for x in pos] == p["counts"]
    allpos = torch.cat(pos)
    assert allpos.numel() == p["N"] and allpos.unique().numel() == p["N"]


def test_bits_per_weight_closed_form():
    # bpw = flag + data with flag = sum of the fractions still unassigned at each bitmap
    # (reference ixrun/search.py:74-83); packing adds at most one word per stream and 2 bytes of scale
    w, v = calibrated_weight(256, 1024, seed=5)
    p = int8x_quantize(w)
    n = p["N"]
    frac = [c / n for c in p["counts"]]
    data = sum(f * b for f, b in zip(frac, (3, 5, 8)))
    flag = 1.0 + (1.0 - frac[0])
    assert abs(p["bits_per_weight"] - (flag + data)) <= (2 + 4 * 4) * 8 / n
    assert np.array_equal(decode_to_weight(p).float().numpy().reshape(-1) * 512, v.astype(np.float32))
    # reference tests/test_core.py:67-81: >2x on the 4 % outlier mix
    p2 = int8x_quantize(outlier_weight(256, 512, seed=1))
    assert p2["compression_vs_bf16"] > 2.0 and p2["bits_per_weight"] < 8.0


# ---------------------------------------------------------------- prefix tables
@pytest.mark.parametrize("shape,level_bits,chunk", [
    ((64, 1024), (3, 5, 8), 512), ((96, 1024), (3, 5, 8), None), ((33, 96), (3, 4, 5, 6, 8), 32),
    ((5, 7), (3, 5, 8), None), ((32, 2048), (3, 5, 8), 1024), ((17, 100), (3, 5, 8), 50)])
def test_prefix_tables(oracle, shape, level_bits, chunk):
    w = outlier_weight(*shape, seed=11)
    p = int8x_quantize(w, level_bits)
    _, q = oracle.quantize_bf16(bf16_bits(w))
    c = chunk or shape[1]
    # brute force: running counts of each level over the int8 values
    T = [BIT_TO_THRESHOLD[b] for b in level_bits[:-1]]
    lvl = np.searchsorted(np.array(T), np.abs(q.astype(np.int32)), side="left")
    pn = oracle.packed_to_numpy(p)
    table = oracle.prefix(p["N"], len(level_bits), pn["bitmaps"], c)
    starts = np.arange(0, p["N"], c)
    for i in range(len(level_bits) - 1):
        cum = np.concatenate([[0], np.cumsum(lvl == i)])
        assert np.array_equal(table[i, :-1], cum[starts])
        assert table[i, -1] == p["counts"][i]
    got = compute_row_prefixes(p, chunk)
    assert len(got) == len(level_bits) - 1
    for i, g in enumerate(got):
        assert g.dtype == torch.int32 and np.array_equal(g.numpy(), table[i, :-1])


def test_pick_split_values():
    from ixrun_amd.fused import _pick_split, _pick_config, FUSED_TILE
    # expectations held by the reference's tests/test_peakq.py:172-217 and fused.py:182-203
    assert FUSED_TILE == 512
    assert [_pick_split(k) for k in (512, 1024, 2048, 17408, 5120, 6144, 1536, 4608)] == [1, 2, 2, 2, 2, 2, 1, 1]
    assert _pick_config(17408, 5120) == (2, 512) and _pick_config(5120, 17408) == (2, 1024)
    assert _pick_config(5120, 5120) == (4, 512)


# ---------------------------------------------------------------- contraction oracle
def test_gemm_oracle_special_cases(oracle):
    w = outlier_weight(48, 96, seed=2)
    p = int8x_quantize(w)
    wd = oracle.decode_packed_bf16(p)  # uint16 [48, 96]
    wf = (wd.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    # one-hot x picks a column exactly
    for k in (0, 17, 95):
        x = np.zeros((1, 96), dtype=np.uint16)
        x[0, k] = 0x3F80  # bf16 1.0
        assert np.array_equal(oracle.gemm_f64(wd, x)[0], wf[:, k])
        assert np.array_equal(oracle.gemm_f32(wd, x)[0], wd[:, k])
    ones = np.full((1, 96), 0x3F80, dtype=np.uint16)
    assert np.allclose(oracle.gemm_f64(wd, ones)[0], wf.sum(axis=1), rtol=1e-14, atol=0)
    # against numpy's own f64 matmul, several activation rows
    g = torch.Generator().manual_seed(1)
    xb = bf16_bits(torch.randn(3, 96, generator=g).bfloat16())
    xf = (xb.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    assert np.allclose(oracle.gemm_f64(wd, xb), xf @ wf.T, rtol=1e-12, atol=1e-15)
    # the fused walk is the same arithmetic as decode -> dequant -> fp32 gemm
    pn = oracle.packed_to_numpy(p)
    y_fused = oracle.fused_gemv_f32(48, 96, pn["level_bits"], pn["bitmaps"], pn["streams"], pn["last"],
                                    pn["scale_bits"], xb[0])
    assert np.array_equal(y_fused, oracle.gemm_f32(wd, xb[:1])[0])
