"""The committed known-answer tensors (tests/golden/codec_fixtures.npz, written by tests/golden/make_fixtures.py)
against the CPU oracle and the package's host codec, and, on a GPU, against the HIP kernels through the C ABI."""
import os

import numpy as np
import pytest
import torch

from helpers import bf16_bits, bits_to_bf16, rel_l2

FIXTURES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "codec_fixtures.npz")
SCHEMES = ["s358", "s34568"]


@pytest.fixture(scope="module")
def golden():
    return np.load(FIXTURES, allow_pickle=False)


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from ixrun_amd import _lib

    assert _lib.lib().ixh_version() >= 100  # the HIP library itself, not a fallback
    return torch.device("cuda:0")


def stored(golden, name):
    bits = tuple(int(b) for b in golden[f"{name}_bits"])
    return {
        "bits": bits, "q": golden[f"{name}_q"], "counts": golden[f"{name}_counts"].tolist(),
        "bitmaps": [golden[f"{name}_bitmap{i}"] for i in range(len(bits) - 1)],
        "streams": [golden[f"{name}_stream{i}"] for i in range(len(bits) - 1)],
        "last": golden[f"{name}_last"], "table": golden[f"{name}_table512"], "w": golden[f"{name}_w_bf16"],
        "x": golden[f"{name}_x_bf16"], "y": golden[f"{name}_y_f64"], "scale_bits": int(golden["scale_bits"][0]),
    }


def as_packed(s):
    """The stored arrays as the package's packed dictionary."""
    out_f, in_f = s["q"].shape
    i32 = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.int32).copy())
    return {
        "level_bits": s["bits"], "out_f": out_f, "in_f": in_f, "N": out_f * in_f,
        "scale": bits_to_bf16(np.array([s["scale_bits"]], dtype=np.uint16)).reshape(()),
        "bitmaps": [i32(b) for b in s["bitmaps"]],
        "streams": [i32(t) for t in s["streams"]] + [torch.from_numpy(s["last"].copy())],
        "counts": s["counts"],
    }


@pytest.mark.parametrize("name", SCHEMES)
def test_every_boundary_value_is_there(golden, name):
    s = stored(golden, name)
    have = set(np.unique(s["q"]).tolist())
    assert {0, 3, -3, 4, -4, 7, -7, 8, -8, 15, -15, 16, -16, 31, -31, 32, -32, 127, -127} <= have
    assert sum(s["counts"]) == s["q"].size


@pytest.mark.parametrize("name", SCHEMES)
def test_oracle_reproduces_the_stored_bytes(oracle, golden, name):
    s = stored(golden, name)
    e = oracle.encode(s["q"].reshape(-1), s["bits"])
    assert e["counts"] == s["counts"]
    for got, want in zip(e["bitmaps"] + e["streams"] + [e["last"]], s["bitmaps"] + s["streams"] + [s["last"]]):
        assert np.array_equal(got, want)
    assert np.array_equal(oracle.decode_i8(s["q"].size, s["bits"], s["bitmaps"], s["streams"], s["last"]), s["q"].reshape(-1))
    assert np.array_equal(oracle.dequant_bf16(s["q"], s["scale_bits"]).reshape(s["w"].shape), s["w"])
    assert np.array_equal(oracle.prefix(s["q"].size, len(s["bits"]), s["bitmaps"], 512), s["table"])
    assert np.array_equal(oracle.gemm_f64(s["w"], s["x"]), s["y"])


@pytest.mark.parametrize("name", SCHEMES)
def test_host_codec_reproduces_the_stored_bytes(golden, name):
    """The package's own writer (torch, CPU) from the stored bf16 weights: same scale, same packed bytes; its scatter
    decoder gives the stored weights back."""
    from ixrun_amd.quantize import decode_to_weight, int8x_quantize

    s = stored(golden, name)
    p = int8x_quantize(bits_to_bf16(s["w"]), s["bits"])
    assert int(bf16_bits(p["scale"].reshape(1))[0]) == s["scale_bits"]
    assert list(p["counts"]) == s["counts"]
    for got, want in zip(p["bitmaps"] + p["streams"][:-1], s["bitmaps"] + s["streams"]):
        assert np.array_equal(got.numpy().view(np.uint32), want)
    assert np.array_equal(p["streams"][-1].numpy(), s["last"])
    assert np.array_equal(bf16_bits(decode_to_weight(p)), s["w"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", SCHEMES)
def test_kernels_reproduce_the_stored_answers(golden, dev, name):
    from ixrun_amd import _lib

    s = stored(golden, name)
    out_f, in_f = s["q"].shape
    dp = _lib.DevicePacked.from_dict(as_packed(s), dev)
    table = dp.prefix_build(512)
    assert np.array_equal(table.cpu().numpy(), s["table"])
    o8 = torch.empty(out_f * in_f, dtype=torch.int8, device=dev)
    o16 = torch.empty(out_f * in_f, dtype=torch.bfloat16, device=dev)
    dp.decode(table, 512, out_i8=o8, out_bf16=o16)
    assert np.array_equal(o8.cpu().numpy().reshape(out_f, in_f), s["q"])
    assert np.array_equal(bf16_bits(o16.cpu()).reshape(out_f, in_f), s["w"])
    # every product kernel that takes the tensor: the library's own choice and each forced one
    x = bits_to_bf16(s["x"]).to(dev)
    want = s["y"]
    flag_sets = [0, _lib.IXH_GEMV_FORCE_358, _lib.IXH_GEMV_DENSE, _lib.IXH_GEMV_STAGED, _lib.IXH_GEMV_FORCE_GENERIC]
    if s["bits"] == (3, 5, 8):
        flag_sets.append(_lib.IXH_GEMV_COLUMN_KERNEL)
    for m in (1, 3):
        for flags in flag_sets:
            y = torch.zeros((m, out_f), dtype=torch.bfloat16, device=dev)
            ws = torch.empty(max(dp.gemv_workspace_bytes(512, m, flags) // 4, 1), dtype=torch.float32, device=dev)
            dp.gemv(table, 512, x[:m].contiguous(), y=y, workspace=ws, flags=flags)
            rounded = bits_to_bf16(bf16_bits(torch.from_numpy(want[:m]).float().bfloat16())).double().numpy()
            assert rel_l2(y.float().cpu().double().numpy(), rounded) < 1e-3, (name, m, flags)
    # the device encoder from the stored weights: the stored bytes
    enc, table2, counts = _lib.encode_device(bits_to_bf16(s["w"]).to(dev), s["bits"])
    assert list(counts) == s["counts"]
    assert np.array_equal(table2.cpu().numpy(), s["table"])
    n_levels = len(s["bits"])
    got = [t.cpu().numpy() for t in enc.tensors[:-1]]  # bitmaps, then streams (the last one bytes); the scale is last
    for g, w in zip(got[: 2 * n_levels - 2], s["bitmaps"] + s["streams"]):
        assert np.array_equal(g.view(np.uint32), w)
    assert np.array_equal(got[2 * n_levels - 2], s["last"])
    assert int(bf16_bits(enc.tensors[-1].cpu())[0]) == s["scale_bits"]
