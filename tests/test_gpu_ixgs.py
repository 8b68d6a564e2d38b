"""Device decode of the group-scale format (ixh_decode_gs) against the CPU oracle: bf16 bit patterns must be equal.
Mirrors the reference's ixgs/test_gs.py on the GPU path."""
import numpy as np
import pytest
import torch

from helpers import bf16_bits
from test_ixgs_cpu import heavy_tail

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from ixrun_amd import _lib

    assert _lib.lib().ixh_version() >= 100
    return torch.device("cuda:0")


def packed_from_ints(oracle, q, scales, out_f, in_f, group):
    """A packed dictionary straight from integers, for values the quantizer never produces (tier 3, +128)."""
    e = oracle.gs_encode(q)
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int32).copy())
    n2, n3 = e["counts"][1], e["counts"][2]
    return {"out_f": out_f, "in_f": in_f, "N": out_f * in_f, "group_size": group,
            "group_scales": torch.from_numpy(scales.view(np.float16).copy()),
            "b1": i32(e["b1"]), "b2": i32(e["b2"]) if n2 + n3 else torch.zeros(1, dtype=torch.int32),
            "l1": i32(e["l1"]), "l2": i32(e["l2"]),
            "l3": torch.from_numpy(e["l3"].copy()) if n3 else torch.zeros(1, dtype=torch.uint8),
            "counts": e["counts"], "total_bytes": 0, "bits_per_weight": 0.0, "compression_vs_bf16": 0.0}


@pytest.fixture(params=["by_mix", "staged", "dense"])
def decoder(request, force_decoder):
    """Which of the two unit-512 decoders runs: chosen by the mix of tiers, or forced (level by level where the
    group size allows it, or the one that stages the streams)."""
    if request.param != "by_mix":
        force_decoder(request.param)
    return request.param


@pytest.mark.parametrize("shape,group", [((512, 256), 64), ((1000, 640), 64), ((1, 1), 64), ((3, 11), 64), ((33, 1000), 64),
                                         ((300, 1031), 64), ((256, 4608), 64), ((128, 512), 8), ((128, 512), 32),
                                         ((64, 1536), 128), ((40, 100), 20), ((7, 513), 3), ((2048, 2048), 64)])
def test_decode_matches_oracle(oracle, dev, decoder, shape, group):
    from ixrun_amd import ixgs

    w = heavy_tail(shape, seed=1)
    p = ixgs.int8gs_quantize(w, group)
    scales, q = oracle.gs_quantize(bf16_bits(w), group)
    want = oracle.gs_dequant_bf16(q, scales, group)
    got = ixgs.decode_weight_triton(p, dev)
    assert got.shape == tuple(shape) and got.dtype == torch.bfloat16
    assert np.array_equal(bf16_bits(got).reshape(-1), want)
    assert torch.equal(got.cpu(), ixgs.decode_weight_scatter(p, device="cpu"))  # ixgs/test_gs.py:61-75


@pytest.mark.parametrize("mix", ["all_tiers", "only_tier3", "only_tier2", "dense_mix"])
@pytest.mark.parametrize("shape,group", [((64, 1536), 64), ((37, 1000), 64), ((5, 100), 10)])
def test_decode_hand_built_tiers(oracle, dev, decoder, mix, shape, group):
    """Integers over the whole range [-127, 128], which the quantizer itself never emits."""
    from ixrun_amd import ixgs

    n = shape[0] * shape[1]
    rng = np.random.default_rng(7)
    if mix == "all_tiers":
        q = rng.integers(-3, 5, size=n)
        r = rng.random(n)
        q[r < 0.3] = rng.integers(-15, 17, size=int((r < 0.3).sum()))
        q[r < 0.05] = rng.integers(-127, 129, size=int((r < 0.05).sum()))
        q[:4] = [128, -127, 16, -15]
    elif mix == "only_tier3":
        q = rng.choice([-127, -100, -16, 17, 99, 128], size=n)
    elif mix == "only_tier2":
        q = rng.choice([-15, -4, 5, 16], size=n)
    else:
        q = rng.integers(-127, 129, size=n)
    q = q.astype(np.int16)
    scales = (rng.random(-(-n // group)).astype(np.float32) * 0.01 + 1e-4).astype(np.float16).view(np.uint16)
    p = packed_from_ints(oracle, q, scales, shape[0], shape[1], group)
    got = ixgs.decode_weight_triton(p, dev)
    assert np.array_equal(bf16_bits(got).reshape(-1), oracle.gs_dequant_bf16(q, scales, group))


def test_linear_and_deploy(oracle, dev):
    from ixrun_amd import ixgs

    w = heavy_tail((256, 128), seed=2)
    x = torch.randn(8, 128, generator=torch.Generator("cpu").manual_seed(2)).bfloat16().to(dev)
    p = ixgs.int8gs_quantize(w)
    for cache in ("full", "none"):
        layer = ixgs.Int8GSLinear(p, cache=cache)
        want = torch.nn.functional.linear(x, ixgs.decode_weight_scatter(p, dev))
        assert torch.equal(layer(x), want)
    model = torch.nn.Sequential(torch.nn.Linear(128, 256), torch.nn.GELU(), torch.nn.Linear(256, 64)).bfloat16()
    with torch.no_grad():
        model[0].weight.copy_(w)
    ref = model.to(dev)(x)
    import copy

    deployed = copy.deepcopy(model)
    stats = ixgs.deploy_model_gs(deployed, verbose=False)
    assert stats["n_layers"] == 2 and isinstance(deployed[0], ixgs.Int8GSLinear) and stats["counts"][2] == 0
    out = deployed.to(dev)(x)
    corr = torch.corrcoef(torch.stack([ref.float().flatten(), out.float().flatten()]))[0, 1]
    assert corr > 0.99


def test_rejects_bad_arguments(dev):
    from ixrun_amd import _lib, ixgs

    p = ixgs.int8gs_quantize(heavy_tail((8, 64), seed=0))
    mv = lambda t: t.to(dev)
    dp = _lib.DevicePacked((3, 5, 8), 8, 64, [mv(p["b1"]), mv(p["b2"])], [mv(p["l1"]), mv(p["l2"]), mv(p["l3"])], None)
    table = dp.prefix_build(512)
    out = torch.empty(512, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        dp.decode_gs(table, 512, mv(p["group_scales"])[:3], 64, out)
    with pytest.raises(_lib.IxhError):
        dp.decode_gs(table, 512, mv(p["group_scales"]), 0, out)
