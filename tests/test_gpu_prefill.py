"""Parity of the fused decode + matrix-core GEMM (many activation rows) with the CPU oracle.

Outputs are bf16; they are compared with the fp64 oracle GEMM over the oracle's decoded
bf16 weight, rounded to bf16: relative L2 <= 1e-3 and max|dy| / max|y| < 5e-3 (the
reference's own acceptance metric, tests/test_fused.py:34-37).  With one-hot activation
rows the products are exact, so the outputs must equal decoded weight columns bit for bit.
"""
import numpy as np
import pytest
import torch

from helpers import activations, bf16_bits, int8_mix, packed_from_int8, student_t_weight
from test_gpu_parity import check_outputs, dev, device_packed, make_packed, quantize  # noqa: F401

pytestmark = pytest.mark.gpu


def run_gemm(dp, x, dev):
    table = dp.prefix_build(512)
    m = x.shape[0]
    y = torch.full((m, dp.out_f), float("nan"), dtype=torch.bfloat16, device=dev)
    ws = torch.empty(max(dp.gemm_workspace_bytes(m) // 4, 1), dtype=torch.float32, device=dev)
    dp.gemm(table, x.to(dev), y, ws)
    return bf16_bits(y)


@pytest.mark.parametrize("kind", ["student_t", "calibrated_odd_scale", "rare_other", "only_l1", "only_l3", "no_l2"])
@pytest.mark.parametrize("shape", [(64, 512), (100, 4608), (130, 8192)])
@pytest.mark.parametrize("level_bits", [(3, 5, 8), (3, 4, 5, 6, 8)])
def test_gemm_matches_oracle(oracle, dev, kind, shape, level_bits):
    out_f, in_f = shape
    p = make_packed(kind, out_f, in_f, level_bits)
    dp = device_packed(p, dev)
    w_bits = oracle.decode_packed_bf16(p)
    for m in (17, 64, 130, 512, 600):
        x = activations(m, in_f, seed=m)
        y64 = oracle.gemm_f64(w_bits, bf16_bits(x))
        check_outputs(run_gemm(dp, x, dev), y64, f"{kind} {shape} {level_bits} m={m}")


@pytest.mark.parametrize("level_bits", [(2, 8), (4, 8), (3, 5, 8), (2, 3, 4, 5, 6, 7, 8)])
def test_gemm_other_schemes(oracle, dev, level_bits):
    p = quantize(student_t_weight(96, 4096, seed=3), level_bits)
    dp = device_packed(p, dev)
    x = activations(33, 4096, seed=7)
    y64 = oracle.gemm_f64(oracle.decode_packed_bf16(p), bf16_bits(x))
    check_outputs(run_gemm(dp, x, dev), y64, f"{level_bits}")


@pytest.mark.parametrize("kind", ["student_t", "calibrated_odd_scale"])
@pytest.mark.parametrize("level_bits", [(3, 5, 8), (3, 4, 5, 6, 8)])
def test_gemm_one_hot_rows_are_exact(oracle, dev, kind, level_bits):
    """Row j of x is e_k(j): y[j] is then column k(j) of the decoded weight, exactly."""
    out_f, in_f = 100, 4608
    p = make_packed(kind, out_f, in_f, level_bits)
    dp = device_packed(p, dev)
    w_want = oracle.decode_packed_bf16(p)
    cols = [0, 1, 63, 64, 511, 512, 575, 1024, 2303, 2304, 4095, 4096, 4607] + list(range(7, 4608, 97))
    x = torch.zeros(len(cols), in_f, dtype=torch.bfloat16)
    for j, k in enumerate(cols):
        x[j, k] = 1.0
    y = run_gemm(dp, x, dev)
    for j, k in enumerate(cols):
        assert np.array_equal(y[j], w_want[:, k]), (kind, level_bits, k)


def test_gemm_strided_rows_and_repeatability(oracle, dev):
    out_f, in_f, m = 70, 4096, 40
    p = make_packed("calibrated_odd_scale", out_f, in_f, (3, 4, 5, 6, 8))
    dp = device_packed(p, dev)
    table = dp.prefix_build(512)
    xw = activations(m, in_f + 64, seed=4)
    x = xw.to(dev)[:, :in_f]  # row stride in_f + 64
    yw = torch.zeros((m, out_f + 10), dtype=torch.bfloat16, device=dev)
    ws = torch.empty(dp.gemm_workspace_bytes(m) // 4, dtype=torch.float32, device=dev)
    dp.gemm(table, x, yw[:, :out_f], ws)
    y64 = oracle.gemm_f64(oracle.decode_packed_bf16(p), bf16_bits(xw[:, :in_f].contiguous()))
    first = bf16_bits(yw[:, :out_f].contiguous())
    check_outputs(first, y64, "strided")
    assert torch.all(yw[:, out_f:] == 0)
    for _ in range(3):
        dp.gemm(table, x, yw[:, :out_f], ws)
        assert np.array_equal(bf16_bits(yw[:, :out_f].contiguous()), first)


# ---- the 128-row tile kernel (tensors that are almost all level 1, 3-bit first level), forced onto every mix ----
# gemm_tiles = 1: wherever it fits; 2: the same with no value lists, every element above level 1 computed where it is
# needed (the path of a unit column with more than 2048 such elements in a workgroup's 128 rows)
@pytest.mark.parametrize("mode", [1, 2])
@pytest.mark.parametrize("kind", ["student_t", "calibrated_odd_scale", "rare_other", "only_l1", "only_l3", "no_l2"])
@pytest.mark.parametrize("shape", [(100, 4608), (130, 8192)])
@pytest.mark.parametrize("level_bits", [(3, 5, 8), (3, 4, 5, 6, 8)])
def test_gemm_tile_kernel_matches_oracle(oracle, dev, gemv_option, mode, kind, shape, level_bits):
    out_f, in_f = shape
    p = make_packed(kind, out_f, in_f, level_bits)
    dp = device_packed(p, dev)
    w_bits = oracle.decode_packed_bf16(p)
    gemv_option("gemm_tiles", mode)
    for m in (17, 130, 512, 600):
        x = activations(m, in_f, seed=m)
        y64 = oracle.gemm_f64(w_bits, bf16_bits(x))
        check_outputs(run_gemm(dp, x, dev), y64, f"tiles={mode} {kind} {shape} {level_bits} m={m}")


@pytest.mark.parametrize("mode", [-1, 1, 2])
@pytest.mark.parametrize("level_bits", [(3, 5, 8), (3, 4, 5, 6, 8), (3, 8)])
def test_gemm_kernels_decode_the_same_weight(oracle, dev, gemv_option, mode, level_bits):
    """One-hot activation rows through each kernel of ixh_gemm: the outputs are columns of the decoded weight, bit
    for bit.  The first 600 columns hold values of every size, the others are 99.8 % level 1: the first two unit
    columns of every 128-row tile then have more elements above level 1 than a value list takes (2048), the others
    far fewer, and both paths of the tile kernel run in one launch."""
    out_f, in_f = 200, 3072
    q = int8_mix("rare_other", out_f * in_f, seed=4).reshape(out_f, in_f)
    q[:, :600] = int8_mix("five_dense", out_f * 600, seed=5).reshape(out_f, 600)
    p = packed_from_int8(q, out_f, in_f, level_bits=level_bits)
    dp = device_packed(p, dev)
    w_want = oracle.decode_packed_bf16(p)
    gemv_option("gemm_tiles", mode)
    cols = [0, 1, 511, 512, 599, 600, 1023, 1024, 2047, 2048, 3071] + list(range(5, in_f, 61))
    x = torch.zeros(len(cols), in_f, dtype=torch.bfloat16)
    for j, k in enumerate(cols):
        x[j, k] = 1.0
    y = run_gemm(dp, x, dev)
    for j, k in enumerate(cols):
        assert np.array_equal(y[j], w_want[:, k]), (mode, level_bits, k)


def test_gemm_tile_kernel_leaves_long_rows_to_the_other(oracle, dev, gemv_option):
    """Rows of 120 units cannot be cut into at most 16 slices of at most 7 unit columns: with the tile kernel asked for
    wherever it fits, ixh_gemm still answers, through its other kernel."""
    out_f, in_f = 24, 61440
    p = make_packed("student_t", out_f, in_f, (3, 4, 5, 6, 8))
    dp = device_packed(p, dev)
    gemv_option("gemm_tiles", 1)
    x = activations(40, in_f, seed=3)
    y64 = oracle.gemm_f64(oracle.decode_packed_bf16(p), bf16_bits(x))
    check_outputs(run_gemm(dp, x, dev), y64, "120 units per row")


def test_streaming_linear_prefers_the_tile_kernel_where_it_wins(oracle, dev):
    """A layer of more than 2**24 elements, almost all level 1, with a decode buffer at hand: up to 512 rows (256 when it
    has more outputs than inputs) forward goes through ixh_gemm and leaves the buffer alone, beyond that it decodes."""
    from ixrun_amd.engine import StreamingLinear

    out_f, in_f = 4096, 4608
    q = int8_mix("rare_other", out_f * in_f, seed=2)  # 99.8 % level 1
    q[0] = 127
    p = quantize(torch.from_numpy(q.astype(np.float32) * 0.0123046875).reshape(out_f, in_f), (3, 4, 5, 6, 8))
    sl = StreamingLinear(p)
    buf = torch.zeros(p["N"], dtype=torch.bfloat16, device=dev)
    sl._set_shared_buf(buf)
    assert sl._fused_gemm_wins(512) and not sl._fused_gemm_wins(513)
    x = activations(300, in_f, seed=6)
    y = sl(x.to(dev))
    torch.cuda.synchronize()
    assert not buf.any(), "forward decoded into the buffer"
    w_bits = oracle.decode_packed_bf16(p)
    rows = np.r_[0:40, out_f - 40:out_f]
    y64 = oracle.gemm_f64(np.ascontiguousarray(w_bits[rows]), bf16_bits(x))
    check_outputs(np.ascontiguousarray(bf16_bits(y)[:, rows]), y64, "StreamingLinear m=300, tile kernel")
    sl(activations(600, in_f, seed=7).to(dev))
    torch.cuda.synchronize()
    assert buf.any(), "600 rows should have gone through decode + GEMM"


def test_gemm_rejects_what_it_cannot_take(oracle, dev):
    from ixrun_amd import _lib

    p = make_packed("student_t", 64, 1000)  # rows that are not whole 512-element units
    dp = device_packed(p, dev)
    x = activations(32, 1000, seed=1)
    with pytest.raises(_lib.IxhError) as e:
        run_gemm(dp, x, dev)
    assert e.value.code == _lib.IXH_EUNSUPPORTED
    p = make_packed("student_t", 64, 4096)
    dp = device_packed(p, dev)
    table = dp.prefix_build(512)
    y = torch.zeros((32, 64), dtype=torch.bfloat16, device=dev)
    with pytest.raises(_lib.IxhError) as e:
        dp.gemm(table, activations(32, 4096, seed=1).to(dev), y, None)
    assert e.value.code == -4


def test_streaming_linear_takes_the_fused_gemm(oracle, dev):
    """Five-level layer, 48 rows: StreamingLinear.forward must not touch the decode buffer."""
    from ixrun_amd.engine import StreamingLinear

    out_f, in_f = 192, 5120
    p = quantize(student_t_weight(out_f, in_f, seed=5), (3, 4, 5, 6, 8))
    sl = StreamingLinear(p)  # no shared buffer set: a decode would fail
    x = activations(48, in_f, seed=2)
    y = sl(x.to(dev).reshape(2, 24, in_f))
    assert y.shape == (2, 24, out_f) and y.dtype == torch.bfloat16
    y64 = oracle.gemm_f64(oracle.decode_packed_bf16(p), bf16_bits(x))
    check_outputs(bf16_bits(y.reshape(48, out_f)), y64, "StreamingLinear m=48")


def _full_size_prefill(oracle, dev, out_f, in_f, m, what):
    p = quantize(student_t_weight(out_f, in_f, seed=0), (3, 4, 5, 6, 8))
    dp = device_packed(p, dev)
    x = activations(m, in_f, seed=1)
    y = run_gemm(dp, x, dev)
    w_bits = oracle.decode_packed_bf16(p)
    rows = np.r_[0:64, 2500:2564, out_f - 64:out_f]
    y64 = oracle.gemm_f64(np.ascontiguousarray(w_bits[rows]), bf16_bits(x))
    check_outputs(np.ascontiguousarray(y[:, rows]), y64, what)


def test_full_size_prefill_square_layer(oracle, dev):
    """5120 x 5120 five-level, 512 rows through ixh_gemm; 192 sampled output columns against the oracle."""
    _full_size_prefill(oracle, dev, 5120, 5120, 512, "5120x5120 five-level m=512")


def test_full_size_prefill_config5(oracle, dev):
    """BASELINE config 5 as stated: W 5120 x 17408 in the five-level scheme (3,4,5,6,8), 512 activation rows, through
    ixh_gemm (decode into LDS tiles, bf16 MFMA, fp32 accumulate); 192 sampled output columns against the fp64 oracle."""
    _full_size_prefill(oracle, dev, 5120, 17408, 512, "config 5: 5120x17408 five-level m=512")
