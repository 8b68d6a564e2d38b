"""Seeded random configurations through every device entry point: shapes, level schemes, level mixes and row counts
drawn at random, each checked against the CPU oracle (integers bit-exact, products within the suite's tolerances).
The fixed cases of the other files name the corner cases; this file looks for interplay between them."""
import numpy as np
import pytest
import torch

from helpers import activations, bf16_bits, packed_from_int8
from test_gpu_parity import check_outputs, device_packed, run_gemv

pytestmark = pytest.mark.gpu

N_CASES = 40


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from ixrun_amd import _lib

    assert _lib.lib().ixh_version() >= 100
    return torch.device("cuda:0")


def draw_case(seed):
    rng = np.random.default_rng(1000 + seed)
    inner = sorted(rng.choice(np.arange(1, 8), size=rng.integers(1, 5), replace=False).tolist())
    level_bits = tuple(inner) + (8,)
    if rng.random() < 0.4:
        level_bits = (3, 5, 8)
    in_f = int(rng.choice([512, 1024, 1536, 2048, 4608, int(rng.integers(1, 700)), int(rng.integers(1, 3000))]))
    out_f = int(rng.integers(1, 160))
    n = out_f * in_f
    # a random level mix: level i holds magnitudes (T_{i-1}, T_i]
    edges = [0] + [(1 << (b - 1)) - 1 for b in level_bits]
    probs = rng.dirichlet(np.ones(len(level_bits)) * rng.choice([0.3, 1.0, 5.0]))
    if rng.random() < 0.3:
        probs = np.array([0.995] + [0.005 / (len(level_bits) - 1)] * (len(level_bits) - 1))
    lvl = rng.choice(len(level_bits), size=n, p=probs)
    lo = np.array([0 if i == 0 else edges[i] + 1 for i in range(len(level_bits))])
    hi = np.array(edges[1:])
    ok = hi >= lo  # repeated thresholds leave a level empty: send its elements to the first level
    lvl = np.where(ok[lvl], lvl, 0)
    mag = rng.integers(lo[lvl], hi[lvl] + 1)
    v = (mag * (rng.integers(0, 2, size=n) * 2 - 1)).astype(np.int8)
    m = int(rng.integers(1, 17))
    scale = float(torch.tensor(rng.uniform(1e-3, 5e-2), dtype=torch.float32).bfloat16())
    return level_bits, out_f, in_f, v, m, scale


@pytest.mark.parametrize("seed", range(N_CASES))
def test_random_configuration(oracle, dev, seed):
    from ixrun_amd import _lib

    level_bits, out_f, in_f, v, m, scale = draw_case(seed)
    what = f"seed {seed}: {out_f}x{in_f} {level_bits} m={m}"
    print(what, flush=True)
    p = packed_from_int8(v, out_f, in_f, scale=scale, level_bits=level_bits)
    dp = device_packed(p, dev)
    n = out_f * in_f
    want_bits = oracle.dequant_bf16(v, int(bf16_bits(p["scale"].reshape(1))[0]))
    pn = oracle.packed_to_numpy(p)
    for chunk in {512, 1024, in_f}:
        table = dp.prefix_build(chunk)
        assert np.array_equal(table.cpu().numpy(), oracle.prefix(n, len(level_bits), pn["bitmaps"], chunk)), what
        q = torch.empty(n, dtype=torch.int8, device=dev)
        w = torch.empty(n + 8, dtype=torch.bfloat16, device=dev)
        dp.decode(table, chunk, out_i8=q, out_bf16=w[:n])
        assert np.array_equal(q.cpu().numpy(), v), what
        assert np.array_equal(bf16_bits(w[:n]), want_bits), what
        w.zero_()
        dp.decode(table, chunk, out_bf16=w[:n])  # bf16 only: the staged kernel where it applies
        assert np.array_equal(bf16_bits(w[:n]), want_bits), what
    x = activations(m, in_f, seed=seed)
    y64 = oracle.gemm_f64(want_bits.reshape(out_f, in_f), bf16_bits(x))
    chunks = [in_f] + ([512] if in_f % 512 == 0 else [])
    for chunk in chunks:
        for flags in (0, _lib.IXH_GEMV_STAGED, _lib.IXH_GEMV_FORCE_GENERIC, _lib.IXH_GEMV_DENSE):
            check_outputs(run_gemv(dp, chunk, x, m, dev, flags=flags), y64, f"{what} chunk={chunk} flags={flags}")
        check_outputs(run_gemv(dp, chunk, x, m, dev, atomic=True), y64, f"{what} chunk={chunk} atomic")
    if in_f % 512 == 0:
        ws = torch.empty(max(dp.gemm_workspace_bytes(m), 4), dtype=torch.uint8, device=dev)
        y = torch.empty(m, out_f, dtype=torch.bfloat16, device=dev)
        dp.gemm(dp.prefix_build(512), x.to(dev), y, ws)
        check_outputs(bf16_bits(y), y64, f"{what} gemm")


@pytest.mark.parametrize("seed", range(12))
def test_random_encode(oracle, dev, seed):
    """Random weights (not integers): the device encoder against the oracle's quantiser + encoder."""
    from test_gpu_encode import check_against_oracle

    rng = np.random.default_rng(500 + seed)
    level_bits, out_f, in_f, v, m, scale = draw_case(100 + seed)
    g = torch.Generator("cpu").manual_seed(seed)
    spread = float(rng.choice([0.02, 1.0, 300.0]))
    w = (torch.randn(out_f, in_f, generator=g) * spread * torch.exp2(torch.randint(-6, 1, (out_f, in_f), generator=g).float())).bfloat16()
    print(f"seed {seed}: {out_f}x{in_f} {level_bits}", flush=True)
    check_against_oracle(oracle, dev, w, level_bits)
