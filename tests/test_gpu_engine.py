"""Deploy modes of the engine over a toy model (the reference needs a HF checkpoint here;
the deploy helpers take any nn.Module): cached, streaming with the packed-weight cache
file, graph.  Outputs are compared with the same model run on plain int8-dequantised
weights, the reference's own equivalence claim (tests/test_int8_equivalence.py:29-33)."""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

from helpers import outlier_weight

pytestmark = pytest.mark.gpu


def toy_model():
    torch.manual_seed(0)
    model = nn.Sequential()
    model.add_module("proj_in", nn.Linear(512, 1024, bias=True))
    model.add_module("act", nn.GELU())
    model.add_module("proj_out", nn.Linear(1024, 512, bias=False))
    model.add_module("lm_head", nn.Linear(512, 64, bias=False))  # skipped by name
    model.add_module("tiny", nn.Linear(64, 8))                   # skipped by size
    with torch.no_grad():
        model.proj_in.weight.copy_(outlier_weight(1024, 512, seed=1).float())
        model.proj_out.weight.copy_(outlier_weight(512, 1024, seed=2).float())
    return model.bfloat16()


def int8_reference(model):
    ref = copy.deepcopy(model)
    with torch.no_grad():
        for name in ("proj_in", "proj_out"):
            w = getattr(ref, name).weight
            scale = w.abs().max().clamp(min=1e-8) / 127.0
            i8 = (w.float() / scale).round().clamp(-127, 127)
            w.copy_((i8 * scale.bfloat16().float()).to(torch.bfloat16))
    return ref.cuda()


def close(a, b):
    return (a.float() - b.float()).abs().max() <= 2e-2 * b.float().abs().max()


@pytest.mark.parametrize("rows", [1, 3, 40])
def test_deploy_modes(tmp_path, rows):
    from ixrun_amd.engine import GraphLinear, Int8XEngine, StreamingLinear
    from ixrun_amd.linear import Int8XLinear

    x = torch.randn(rows, 512, generator=torch.Generator().manual_seed(5)).bfloat16().cuda()
    base = toy_model()
    want = int8_reference(base)(x)

    cached = copy.deepcopy(base).cuda()
    stats = Int8XEngine._deploy_cached(cached, (3, 5, 8), verbose=False)
    assert stats["n_layers"] == 2 and isinstance(cached.proj_in, Int8XLinear) and isinstance(cached.lm_head, nn.Linear)
    assert torch.equal(cached.proj_out._w.cpu(), int8_reference(base).proj_out.weight.cpu())  # bit-exact weights
    assert close(cached(x), want)

    cache = str(tmp_path / "packed.pt")
    streaming = copy.deepcopy(base)
    stats = Int8XEngine._deploy_streaming(streaming, (3, 5, 8), verbose=False, cache_path=cache)
    assert stats["mode"] == "streaming" and stats["n_layers"] == 2 and isinstance(streaming.proj_in, StreamingLinear)
    streaming = streaming.cuda()
    assert close(streaming(x), want)
    # the file holds what the CPU writer produces for these weights (the layers were encoded on the device)
    from ixrun_amd.quantize import int8x_quantize

    blob = torch.load(cache, map_location="cpu", weights_only=True)
    for name, packed, _ in blob["layers"]:
        ref = int8x_quantize(getattr(base, name).weight.data, (3, 5, 8))
        assert list(packed.keys()) == list(ref.keys()) and packed["counts"] == ref["counts"]
        assert torch.equal(packed["scale"], ref["scale"])
        assert all(torch.equal(a, b) for a, b in zip(packed["bitmaps"] + packed["streams"], ref["bitmaps"] + ref["streams"]))
    again = copy.deepcopy(base)
    Int8XEngine._deploy_streaming(again, (3, 5, 8), verbose=False, cache_path=cache)  # now read from the file
    assert torch.equal(again.cuda()(x), streaming(x))
    with pytest.raises(ValueError, match="level_bits"):
        Int8XEngine._deploy_streaming(copy.deepcopy(base), (3, 4, 5, 6, 8), verbose=False, cache_path=cache)
    other = nn.Sequential(nn.Linear(512, 1024))
    with pytest.raises(ValueError, match="mismatch"):
        Int8XEngine._deploy_streaming(other.bfloat16(), (3, 5, 8), verbose=False, cache_path=cache)

    graph_model = copy.deepcopy(base)
    stats, replay = Int8XEngine._deploy_graph(graph_model, (3, 5, 8), verbose=False)
    assert stats["mode"] == "graph" and isinstance(graph_model.proj_in, GraphLinear)
    graph_model = graph_model.cuda()
    for _ in range(3):
        replay()
        torch.cuda.synchronize()
        assert close(graph_model(x), want)


def test_five_level_streaming_linear():
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize, decode_to_weight

    w = outlier_weight(256, 768, seed=7)
    p = int8x_quantize(w, (3, 4, 5, 6, 8))
    sl = StreamingLinear(p)
    sl._set_shared_buf(torch.empty(p["N"], dtype=torch.bfloat16, device="cuda"))
    assert torch.equal(sl._decode().cpu(), decode_to_weight(p))
    for rows in (1, 5, 64):
        x = torch.randn(rows, 768, generator=torch.Generator().manual_seed(rows)).bfloat16().cuda()
        want = torch.nn.functional.linear(x.float().cpu(), decode_to_weight(p).float())
        assert close(sl(x).cpu(), want)


def test_tuned_library_gemm_on_the_many_row_path(oracle):
    """Decode + library GEMM with the GEMM kernel chosen by measurement: same result to the tolerance of the
    many-row path (rel-L2 <= 1e-3 against the fp64 product of the dequantised weights), signature remembered,
    tuning off again afterwards."""
    import torch.cuda.tunable as tunable
    from ixrun_amd import gemm_tuning
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize
    from helpers import student_t_weight

    dev = torch.device("cuda:0")
    w = student_t_weight(256, 1024, seed=11)
    p = int8x_quantize(w, (3, 5, 8))
    layer = StreamingLinear(p)
    layer._gemm_ok = False
    layer._set_shared_buf(torch.empty(p["N"], dtype=torch.bfloat16, device=dev))
    x = torch.randn(96, 1024, generator=torch.Generator("cpu").manual_seed(3)).bfloat16()
    w_deq = oracle.bf16_bits_to_f32(oracle.decode_packed_bf16(p)).astype(np.float64).reshape(256, 1024)
    want = torch.from_numpy(x.double().numpy() @ w_deq.T).bfloat16().double().numpy()  # the exact product, as bf16
    plain = layer(x.to(dev)).float().cpu().numpy()
    gemm_tuning.enable(max_ms=50)
    try:
        tuned = layer(x.to(dev)).float().cpu().numpy()
        again = layer(x.to(dev)).float().cpu().numpy()
        assert (96, 256, 1024, torch.bfloat16, False) in gemm_tuning.tuned_shapes()
        assert not tunable.tuning_is_enabled()
    finally:
        gemm_tuning.disable()
    for got in (plain, tuned, again):
        assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-3
    assert np.array_equal(tuned, again)


@pytest.mark.parametrize("rows,dense", [(8, False), (16, False), (17, False), (4, True), (16, True), (17, True)])
def test_row_count_policy_with_a_decode_buffer(oracle, rows, dense):
    """Up to 16 rows the fused kernels, for dense level mixes as well, beyond that decode + GEMM when the layer has a
    decode buffer: all within the many-row tolerance of the exact product."""
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize
    from helpers import student_t_weight

    dev = torch.device("cuda:0")
    from helpers import calibrated_weight, int8_mix, packed_from_int8

    if dense:  # 55 / 40 / 5 %
        p = int8x_quantize(calibrated_weight(128, 2048, seed=5)[0], (3, 5, 8))
    else:      # 99.8 % level 1
        p = packed_from_int8(int8_mix("rare_other", 128 * 2048, seed=5), 128, 2048)
    assert (p["counts"][0] * 100 >= p["N"] * 97) == (not dense)
    x = torch.randn(rows, 2048, generator=torch.Generator("cpu").manual_seed(rows)).bfloat16()
    w_deq = oracle.bf16_bits_to_f32(oracle.decode_packed_bf16(p)).astype(np.float64).reshape(128, 2048)
    want = torch.from_numpy(x.double().numpy() @ w_deq.T).bfloat16().double().numpy()
    plain = StreamingLinear(p)
    buffered = StreamingLinear(p)
    buf = torch.full((p["N"],), 9.0, dtype=torch.bfloat16, device=dev)
    buffered._set_shared_buf(buf)
    for layer in (plain, buffered):
        got = layer(x.to(dev)).float().cpu().numpy()
        assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-3
    decoded = bool((buf != 9.0).any())  # the buffer was written iff the pair path ran
    assert decoded == (rows > 16)


@pytest.mark.parametrize("rows", [16, 17, 24, 32, 33])
@pytest.mark.parametrize("buffered", [False, True])
def test_two_fused_calls_for_17_to_32_rows(oracle, monkeypatch, rows, buffered):
    """17 .. 32 rows on a large layer that is almost all level 1 go through the fused kernel in two calls (16 rows and
    the rest), with or without a decode buffer (which then stays untouched); 33 rows and small layers keep the
    many-row paths.  The size limit is lowered for the test so that a small layer counts as large."""
    from ixrun_amd import engine
    from helpers import int8_mix, packed_from_int8

    dev = torch.device("cuda:0")
    p = packed_from_int8(int8_mix("rare_other", 128 * 2048, seed=7), 128, 2048)
    assert p["counts"][0] * 100 >= p["N"] * 97
    x = torch.randn(rows, 2048, generator=torch.Generator("cpu").manual_seed(rows)).bfloat16()
    w_deq = oracle.bf16_bits_to_f32(oracle.decode_packed_bf16(p)).astype(np.float64).reshape(128, 2048)
    want = torch.from_numpy(x.double().numpy() @ w_deq.T).bfloat16().double().numpy()
    for limit, two_calls in ((0, 16 < rows <= 32), (engine.SPLIT_FUSED_MIN_WEIGHTS, False)):
        monkeypatch.setattr(engine, "SPLIT_FUSED_MIN_WEIGHTS", limit)
        layer = engine.StreamingLinear(p)
        buf = torch.full((p["N"],), 9.0, dtype=torch.bfloat16, device=dev)
        if buffered:
            layer._set_shared_buf(buf)
        calls = []
        real = layer._gemv_fn  # the bound ixh_gemv; its fifth argument is the row count of the call
        monkeypatch.setattr(layer, "_gemv_fn", lambda *a: (calls.append(a[4]), real(*a))[1])
        got = layer(x.to(dev)).float().cpu().numpy()
        assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-3
        if rows <= 16:
            assert calls == [rows]
        elif two_calls:
            assert calls == [16, rows - 16] and not bool((buf != 9.0).any())
        else:
            assert calls == [] and bool((buf != 9.0).any()) == buffered
