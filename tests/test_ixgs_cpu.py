"""Group-scale format on the CPU: the oracle's pins and the package's host-side mirror of the reference's ixgs/."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, bits_to_bf16


def heavy_tail(shape, seed):
    """The reference tests' recipe (ixgs/test_gs.py:24-34): N(0, 0.02) plus 0.05 % outliers of N(0, 1.5)."""
    g = torch.Generator("cpu").manual_seed(seed)
    w = torch.randn(shape, generator=g) * 0.02
    hit = (torch.rand(shape, generator=g) < 0.0005).float()
    return (w + hit * torch.randn(shape, generator=g) * 1.5).bfloat16()


def snr(a, b):
    mse = ((a.float() - b.float()) ** 2).mean().item()
    return float("inf") if mse == 0 else 10 * np.log10((b.float() ** 2).mean().item() / mse)


# ---------------------------------------------------------------- oracle pins
def test_fp16_conversion_matches_numpy(oracle):
    L = oracle.lib()
    every = np.arange(65536, dtype=np.uint16)
    as_f32 = every.view(np.float16).astype(np.float32)
    for h in range(0, 65536, 7):  # fp16 -> fp32, a seventh of all patterns plus the edges below
        f = L.ixo_f16_to_f32(int(h))
        assert (np.isnan(f) and np.isnan(as_f32[h])) or np.float32(f) == as_f32[h], hex(h)
    # fp32 -> fp16 on every fp16 value, on the midpoint between neighbours and one fp32 step either side of it
    finite = every[(every & 0x7C00) != 0x7C00]
    vals = finite.view(np.float16).astype(np.float32)
    pos = np.sort(vals[vals >= 0])
    mid = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    probes = np.concatenate([pos, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)),
                             np.float32([65504, 65519.99, 65520, 65536, 1e10, 2.0 ** -25, 2.9e-8, 3.0e-8, 1e-10, 0])])
    rng = np.random.default_rng(0)
    probes = np.concatenate([probes, np.abs(rng.standard_normal(20000)).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 5, 20000)])
    with np.errstate(over="ignore"):
        want = probes.astype(np.float16).view(np.uint16)
    step = max(1, probes.size // 30000)
    for f, wv in zip(probes[::step], want[::step]):
        assert L.ixo_f32_to_f16(float(f)) == int(wv), float(f)
        assert L.ixo_f32_to_f16(float(-f)) == (int(wv) | 0x8000), float(-f)


def test_encode_hand_known_answer(oracle):
    q = np.array([0, 4, -3, 5, 16, -15, 17, -127, 128, -16], dtype=np.int16)
    e = oracle.gs_encode(q)
    assert e["counts"] == [3, 3, 4]
    assert list(e["b1"]) == [0x007] and list(e["b2"]) == [0x07]
    assert list(e["l1"]) == [3 | 7 << 3 | 0 << 6] and list(e["l2"]) == [20 | 31 << 5 | 0 << 10]
    assert list(e["l3"]) == [144, 0, 255, 111]
    assert np.array_equal(oracle.gs_decode_i16(10, e["b1"], e["b2"], e["l1"], e["l2"], e["l3"]), q)


def test_quantize_hand_known_answer(oracle):
    """Two groups of four whose scales are exact: max 1.875 -> 0.125, max 0.46875 -> 0.03125."""
    w = torch.tensor([1.875, -0.375, 0.5, 0.625, -0.46875, 0.046875, 0.0, 0.140625]).bfloat16()
    scales, q = oracle.gs_quantize(bf16_bits(w), group=4)
    assert list(scales.view(np.float16)) == [0.125, 0.03125]
    assert list(q) == [15, -3, 4, 5, -15, 2, 0, 4]  # 1.5 and 4.5 round to the even neighbour
    back = oracle.gs_dequant_bf16(q, scales, group=4)
    assert np.array_equal(back, bf16_bits(torch.tensor([1.875, -0.375, 0.5, 0.625, -0.46875, 0.0625, 0.0, 0.125]).bfloat16()))


@pytest.mark.parametrize("n", [1, 31, 32, 33, 1000, 4099])
def test_encode_round_trip(oracle, n):
    rng = np.random.default_rng(n)
    q = rng.integers(-127, 129, size=n).astype(np.int16)
    small = rng.random(n) < 0.6
    q[small] = rng.integers(-3, 5, size=int(small.sum()))
    e = oracle.gs_encode(q)
    assert sum(e["counts"]) == n
    assert e["l1"].size == (e["counts"][0] * 3 + 31) // 32 and e["l2"].size == (e["counts"][1] * 5 + 31) // 32
    assert np.array_equal(oracle.gs_decode_i16(n, e["b1"], e["b2"], e["l1"], e["l2"], e["l3"]), q)
    # the streams are the bit packing pinned elsewhere in this suite
    assert np.array_equal(e["l1"], oracle.pack_bits((q[(q >= -3) & (q <= 4)] + 3).astype(np.uint32), 3))


@pytest.mark.parametrize("shape", [(512, 256), (1000, 640)])
def test_reference_roundtrip_property(oracle, shape):
    """ixgs/test_gs.py:38-58: the decoded weight is bf16(round(w / s) * s) with s the stored fp16 scale, and on
    heavy-tailed weights its SNR beats per-tensor int8."""
    from ixrun_amd import ixgs

    w = heavy_tail(shape, seed=0)
    scales, q = oracle.gs_quantize(bf16_bits(w), 64)
    e = oracle.gs_encode(q)
    assert e["counts"][2] == 0  # |v| <= 15 by construction
    got = bits_to_bf16(oracle.gs_dequant_bf16(oracle.gs_decode_i16(q.size, e["b1"], e["b2"], e["l1"], e["l2"], e["l3"]),
                                              scales, 64)).view(shape)
    s = torch.from_numpy(scales.view(np.float16).astype(np.float32)).repeat_interleave(64)[: q.size]
    want = ((w.float().reshape(-1) / s).round().clamp(-127, 128) * s).bfloat16().view(shape)
    assert torch.equal(got.float(), want.float())
    assert snr(got, w) > snr(ixgs.per_tensor_int8_reference(w), w)


# ---------------------------------------------------------------- host mirror
@pytest.mark.parametrize("shape,group", [((512, 256), 64), ((100, 130), 64), ((33, 77), 32), ((8, 200), 128), ((5, 7), 4)])
def test_quantize_matches_oracle(oracle, shape, group):
    from ixrun_amd import ixgs

    w = heavy_tail(shape, seed=3)
    p = ixgs.int8gs_quantize(w, group)
    scales, q = oracle.gs_quantize(bf16_bits(w), group)
    e = oracle.gs_encode(q)
    assert np.array_equal(p["group_scales"].numpy().view(np.uint16), scales)
    assert p["counts"] == e["counts"]
    u32 = lambda t: t.numpy().view(np.uint32)
    assert np.array_equal(u32(p["b1"]), e["b1"]) and np.array_equal(u32(p["l1"]), e["l1"]) and np.array_equal(u32(p["l2"]), e["l2"])
    if e["counts"][1] + e["counts"][2]:
        assert np.array_equal(u32(p["b2"]), e["b2"])
    else:
        assert p["b2"].tolist() == [0]
    assert p["l3"].tolist() == [0]  # empty tier 3 is stored as one zero byte
    n_groups = -(-p["N"] // group)
    assert p["total_bytes"] == 4 * (p["l1"].numel() + p["l2"].numel() + p["b1"].numel() + p["b2"].numel()) + 1 + 2 * n_groups
    got = ixgs.decode_weight_scatter(p, device="cpu")
    assert np.array_equal(bf16_bits(got).reshape(-1), oracle.gs_dequant_bf16(q, scales, group))


def test_zero_groups_decode_to_zero(oracle):
    from ixrun_amd import ixgs

    w = heavy_tail((16, 64), seed=1)
    w[3] = 0
    w[7] = 1e-9
    p = ixgs.int8gs_quantize(w)
    assert p["group_scales"][3] == 0 and p["group_scales"][7] == 0
    got = ixgs.decode_weight_scatter(p, device="cpu")
    assert torch.all(got[3] == 0) and torch.all(got[7] == 0)
    scales, q = oracle.gs_quantize(bf16_bits(w), 64)
    assert np.array_equal(bf16_bits(got).reshape(-1), oracle.gs_dequant_bf16(q, scales, 64))


def test_forward_equivalence():
    """ixgs/test_gs.py:78-95."""
    from ixrun_amd import ixgs

    w = heavy_tail((256, 128), seed=2)
    x = torch.randn(8, 128, generator=torch.Generator("cpu").manual_seed(2)).bfloat16()
    w_rec = ixgs.decode_weight_scatter(ixgs.int8gs_quantize(w), device="cpu")
    corr = lambda a, b: torch.corrcoef(torch.stack([a.float().flatten(), b.float().flatten()]))[0, 1]
    y_ref = torch.nn.functional.linear(x, w)
    c_gs = corr(y_ref, torch.nn.functional.linear(x, w_rec))
    c_pt = corr(y_ref, torch.nn.functional.linear(x, ixgs.per_tensor_int8_reference(w)))
    assert c_gs > 0.99 and c_gs > c_pt


def test_rejects_bad_input():
    from ixrun_amd import ixgs

    with pytest.raises(ValueError):
        ixgs.int8gs_quantize(torch.zeros(4, 4, 4))
