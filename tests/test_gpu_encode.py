"""The device encoder against the CPU oracle and the CPU writer, through the C ABI.

Everything here is integer / byte work and must be bit-exact: the bf16 scale, the
per-level counts, every word of every bitmap and code stream, the last level's bytes and
the rank table at unit 512 (reference: ixrun/quantize.py:41-122, ixrun/bitpack.py:13-61,
ixrun/fused.py:67-78).
"""
import numpy as np
import pytest
import torch

from helpers import bf16_bits, calibrated_weight, outlier_weight, student_t_weight

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from ixrun_amd import _lib

    assert _lib.lib().ixh_version() >= 100
    return torch.device("cuda:0")


def make_weight(kind, out_f, in_f):
    g = torch.Generator("cpu").manual_seed(5)
    if kind == "student_t":
        return student_t_weight(out_f, in_f, seed=0)
    if kind == "outlier":
        return outlier_weight(out_f, in_f, seed=0)
    if kind == "calibrated_pow2":
        return calibrated_weight(out_f, in_f, seed=0)[0]
    if kind == "calibrated_odd_scale":
        return calibrated_weight(out_f, in_f, seed=0, scale=0.0123046875)[0]
    if kind == "zeros":  # the scale falls back to its floor, every value is 0
        return torch.zeros(out_f, in_f, dtype=torch.bfloat16)
    if kind == "all_extreme":  # every element +-max: only the last level is used
        sign = torch.randint(0, 2, (out_f, in_f), generator=g) * 2 - 1
        return (sign * 0.75).bfloat16()
    if kind == "wide_range":  # magnitudes over many binades: quotients near every rounding boundary
        e = torch.randint(-20, 1, (out_f, in_f), generator=g).float()
        return (torch.randn(out_f, in_f, generator=g) * torch.exp2(e)).bfloat16()
    if kind == "tiny":  # near the scale's floor, quotients with subnormal divisors' neighbours
        return (torch.randn(out_f, in_f, generator=g) * 3e-8).bfloat16()
    if kind == "half_steps":  # exact ties k + 0.5 of the quotient: round-half-even decides
        k = torch.randint(-253, 254, (out_f, in_f), generator=g).float() * 0.5
        w = (k * 2.0 ** -7).bfloat16()
        w.view(-1)[0] = 127 * 2.0 ** -7
        return w
    raise KeyError(kind)


KINDS = ["student_t", "outlier", "calibrated_pow2", "calibrated_odd_scale", "zeros", "all_extreme", "wide_range", "tiny",
         "half_steps"]


def oracle_encode(oracle, w, level_bits):
    scale_bits, q = oracle.quantize_bf16(bf16_bits(w))
    e = oracle.encode(q, level_bits)
    table = oracle.prefix(q.size, len(level_bits), e["bitmaps"], 512)
    return scale_bits, q, e, table


def check_against_oracle(oracle, dev, w, level_bits):
    from ixrun_amd.quantize import int8x_quantize_device

    scale_bits, q, e, table = oracle_encode(oracle, w, level_bits)
    p = int8x_quantize_device(w.to(dev), level_bits)
    torch.cuda.synchronize()
    what = f"{tuple(w.shape)} {level_bits}"
    assert int(bf16_bits(p["scale"].reshape(1))[0]) == scale_bits, f"{what}: scale"
    assert p["counts"] == [int(c) for c in e["counts"]], f"{what}: counts"
    assert p["total_bytes"] == e["total_bytes"], f"{what}: total_bytes"
    for i in range(len(level_bits) - 1):
        got_bm = p["bitmaps"][i].cpu().numpy().view(np.uint32)
        got_st = p["streams"][i].cpu().numpy().view(np.uint32)
        assert got_bm.shape == e["bitmaps"][i].shape and np.array_equal(got_bm, e["bitmaps"][i]), f"{what}: bitmap {i}"
        assert got_st.shape == e["streams"][i].shape and np.array_equal(got_st, e["streams"][i]), f"{what}: stream {i}"
    assert np.array_equal(p["streams"][-1].cpu().numpy(), e["last"]), f"{what}: last level"
    assert np.array_equal(p["table512"].cpu().numpy(), table), f"{what}: rank table"
    return p, q


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("shape", [(1, 1), (2, 5), (3, 11), (7, 33), (1, 512), (1, 513), (33, 1000), (128, 256),
                                   (300, 1031), (64, 1536), (256, 4608)])
def test_encode_bit_exact(oracle, dev, kind, shape):
    check_against_oracle(oracle, dev, make_weight(kind, *shape), (3, 5, 8))


@pytest.mark.parametrize("level_bits", [(3, 4, 5, 6, 8), (2, 8), (4, 8), (7, 8), (1, 2, 3, 4, 5, 6, 7, 8), (3, 3, 8),
                                        (1, 7, 8)])
@pytest.mark.parametrize("kind", ["student_t", "calibrated_odd_scale", "wide_range"])
def test_encode_other_level_schemes(oracle, dev, kind, level_bits):
    check_against_oracle(oracle, dev, make_weight(kind, 300, 1031), level_bits)


def test_encode_hand_known_answer(dev):
    """The 2x5 tensor worked out by hand from the reference's code: v = [0,1,-3,4,-15 | 16,127,-127,3,5], s = 2^-7."""
    from ixrun_amd.quantize import int8x_quantize_device

    v = torch.tensor([0, 1, -3, 4, -15, 16, 127, -127, 3, 5], dtype=torch.float32)
    w = (v * 2.0 ** -7).bfloat16().view(2, 5)
    p = int8x_quantize_device(w.to(dev), (3, 5, 8))
    u32 = lambda t: [int(x) for x in t.cpu().numpy().view(np.uint32)]
    assert u32(p["bitmaps"][0]) == [0x00000107] and u32(p["bitmaps"][1]) == [0x00000023]
    assert u32(p["streams"][0]) == [0x00000C23] and u32(p["streams"][1]) == [0x00005013]
    assert p["streams"][2].cpu().tolist() == [143, 254, 0]
    assert p["counts"] == [4, 3, 3] and p["total_bytes"] == 21
    assert float(p["scale"]) == 2.0 ** -7


def test_encode_matches_cpu_writer(dev):
    """Same dictionary as the package's CPU writer (which follows the reference's writer line by line)."""
    from ixrun_amd.quantize import int8x_quantize, int8x_quantize_device

    w = outlier_weight(96, 1000, seed=3)
    for level_bits in [(3, 5, 8), (3, 4, 5, 6, 8)]:
        a = int8x_quantize(w, level_bits)
        b = int8x_quantize_device(w.to(dev), level_bits)
        for key in ("level_bits", "out_f", "in_f", "N", "counts", "total_bytes", "bits_per_weight", "compression_vs_bf16"):
            assert a[key] == b[key], key
        assert torch.equal(a["scale"], b["scale"].cpu())
        for x, y in zip(a["bitmaps"] + a["streams"], b["bitmaps"] + b["streams"]):
            assert x.dtype == y.dtype and torch.equal(x, y.cpu())


def test_encode_unaligned_weight(oracle, dev):
    """A weight that starts 2 bytes past a 16-byte boundary takes the scalar load path."""
    from ixrun_amd import _lib

    w = student_t_weight(40, 520, seed=2)
    scale_bits, q, e, table = oracle_encode(oracle, w, (3, 5, 8))
    buf = torch.empty(w.numel() + 8, dtype=torch.bfloat16, device=dev)
    view = buf[1 : 1 + w.numel()].view(40, 520)
    view.copy_(w)
    assert view.data_ptr() % 16 == 2
    dp, tab, counts = _lib.encode_device(view, (3, 5, 8))
    assert counts == [int(c) for c in e["counts"]]
    assert np.array_equal(dp.tensors[0].cpu().numpy().view(np.uint32), e["bitmaps"][0])
    assert np.array_equal(dp.tensors[2].cpu().numpy().view(np.uint32), e["streams"][0])
    assert np.array_equal(tab.cpu().numpy(), table)


def test_encode_rejects_bad_arguments(dev):
    from ixrun_amd import _lib
    from ixrun_amd.quantize import int8x_quantize_device

    w = torch.zeros(4, 8, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        int8x_quantize_device(w, (3, 5, 7))
    with pytest.raises(RuntimeError):
        int8x_quantize_device(w.cpu(), (3, 5, 8))
    with pytest.raises(RuntimeError):
        int8x_quantize_device(torch.zeros(0, 8, dtype=torch.bfloat16, device=dev), (3, 5, 8))
    with pytest.raises(_lib.IxhError):
        _lib.encode_device(w, (3, 9, 8))


def test_encoded_layer_runs(oracle, dev):
    """Encoder output straight into the module: decode gives back the int8, the fused product matches."""
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize_device

    w = student_t_weight(192, 2048, seed=4)
    p, q = check_against_oracle(oracle, dev, w, (3, 5, 8))
    layer = StreamingLinear(p)
    q_dev = torch.empty(p["N"], dtype=torch.int8, device=dev)
    layer._dp.decode(layer._table, layer._unit, out_i8=q_dev)
    assert np.array_equal(q_dev.cpu().numpy(), q)
    x = torch.randn(1, 2048, generator=torch.Generator("cpu").manual_seed(1)).bfloat16()
    y = layer(x.to(dev))
    w_deq = (torch.from_numpy(q.astype(np.float32)) * p["scale"].float().cpu()).bfloat16().view(192, 2048)
    want = torch.nn.functional.linear(x.float(), w_deq.float())
    assert (y.float().cpu() - want).norm() / want.norm() < 4e-3


def test_encode_full_size_layer(oracle, dev):
    """5120x17408 Student-t: every stream equal to the oracle's, and the round trip through the device decoder."""
    from ixrun_amd.triton_kernels import decode_int8

    w = student_t_weight(5120, 17408, seed=0)
    p, q = check_against_oracle(oracle, dev, w, (3, 5, 8))
    assert np.array_equal(decode_int8(p, device=dev).cpu().numpy().reshape(-1), q)
