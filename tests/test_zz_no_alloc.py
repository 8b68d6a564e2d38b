"""The entry point that allocates nothing (ixh_gemv_noalloc) against ixh_gemv, through the C ABI.

Both run the same kernels; the only difference is where the partial sums of the kernels that need a workspace
live (the library's built-in buffer instead of a caller's tensor), so the outputs must be equal bit for bit.  The
calls must not change the device's free memory and must replay correctly from a hipGraph.  Each
case calls twice in a row, the second time with a smaller tensor, so that what the first call left in the shared
buffer would show.
"""
import numpy as np
import pytest
import torch

from helpers import activations, bf16_bits, calibrated_weight, outlier_weight, student_t_weight

pytestmark = pytest.mark.gpu

LIMIT = 16 << 20


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from ixrun_amd import _lib

    assert _lib.lib().ixh_version() >= 100
    return torch.device("cuda:0")


def _layer(recipe, out_f, in_f, dev, level_bits=(3, 5, 8)):
    from ixrun_amd import _lib
    from ixrun_amd.quantize import int8x_quantize

    w = {"student_t": lambda: student_t_weight(out_f, in_f, seed=2),
         "outlier": lambda: outlier_weight(out_f, in_f, seed=2),
         "calibrated": lambda: calibrated_weight(out_f, in_f, seed=2, scale=0.0123046875)[0]}[recipe]()
    dp = _lib.DevicePacked.from_dict(int8x_quantize(w, level_bits), dev)
    return dp, dp.prefix_build(512)


def _both(dp, table, x, flags, dev):
    m = x.shape[0]
    need = dp.gemv_workspace_bytes(512, m, flags)
    ws = torch.empty(max(need // 4, 1), dtype=torch.float32, device=dev)
    y_ref = torch.zeros((m, dp.out_f), dtype=torch.bfloat16, device=dev)
    dp.gemv(table, 512, x, y=y_ref, workspace=ws, flags=flags)
    y_new = torch.full((m, dp.out_f), 7.0, dtype=torch.bfloat16, device=dev)
    dp.gemv_noalloc(table, 512, x, y_new, flags=flags)
    torch.cuda.synchronize()
    return bf16_bits(y_ref), bf16_bits(y_new), need


@pytest.mark.parametrize("recipe,level_bits", [("calibrated", (3, 5, 8)), ("outlier", (3, 5, 8)), ("student_t", (3, 5, 8)),
                                               ("outlier", (3, 4, 5, 6, 8))])
@pytest.mark.parametrize("m", [1, 3, 8, 16])
def test_noalloc_equals_gemv_twice_in_a_row(dev, recipe, level_bits, m):
    """Big tensor first, then a smaller one: the second call's partial sums cover only a part of what the first left
    in the buffer.  Flags: the library's own choice, the column-block kernel and the staged kernel (both always go
    through the workspace), the wave-per-unit kernel."""
    from ixrun_amd import _lib

    big, big_t = _layer(recipe, 640, 4608, dev, level_bits)
    small, small_t = _layer(recipe, 96, 1536, dev, level_bits)
    used = 0
    for flags in (0, _lib.IXH_GEMV_COLUMN_KERNEL, _lib.IXH_GEMV_STAGED, _lib.IXH_GEMV_FORCE_GENERIC):
        for dp, table in ((big, big_t), (small, small_t)):
            x = activations(m, dp.in_f, seed=3 + m).to(dev)
            y_ref, y_new, need = _both(dp, table, x, flags, dev)
            assert need <= LIMIT
            used = max(used, need)
            assert np.array_equal(y_ref, y_new), (recipe, level_bits, m, flags, dp.out_f)
    assert used > 0  # at least one of the routes really went through the buffer


@pytest.mark.parametrize("level_bits", [(3, 5, 8), (3, 4, 5, 6, 8)])
@pytest.mark.parametrize("m", [3, 8, 16])
def test_noalloc_with_row_blocks_shared_by_workgroups(dev, gemv_option, level_bits, m):
    """The tile kernel with two and three workgroups to a block of rows: their partial sums meet in the built-in
    buffer and a second launch adds them.  Twice in a row, the smaller tensor second."""
    from ixrun_amd import _lib

    big, big_t = _layer("student_t", 640, 4608, dev, level_bits)
    small, small_t = _layer("student_t", 96, 1536, dev, level_bits)
    gemv_option("gemv_tiles", 1)
    gemv_option("gemv_tile_cus", 4)
    for split in (2, 3):
        gemv_option("gemv_tile_split", split)
        for dp, table in ((big, big_t), (small, small_t)):
            x = activations(m, dp.in_f, seed=5 + m).to(dev)
            y_ref, y_new, need = _both(dp, table, x, _lib.IXH_GEMV_FORCE_358, dev)
            assert 0 < need <= LIMIT
            assert np.array_equal(y_ref, y_new), (level_bits, m, split, dp.out_f)


def test_noalloc_rejects_what_does_not_fit(dev):
    """A request whose partial sums exceed the built-in buffer fails with IXH_EWORKSPACE before anything is launched
    (the table handed in is a real one for that chunk, so even a wrongly accepted call would run validly); the
    atomic mode, which has no workspace, is refused too."""
    from ixrun_amd import _lib
    from ixrun_amd.quantize import int8x_quantize

    dp = _lib.DevicePacked.from_dict(int8x_quantize(outlier_weight(2048, 2048, seed=1)), dev)
    table = dp.prefix_build(1)
    assert dp.gemv_workspace_bytes(1, 2) == 2 * 2048 * 2048 * 4 > LIMIT
    x = activations(2, 2048, seed=1).to(dev)
    y = torch.full((2, 2048), 7.0, dtype=torch.bfloat16, device=dev)
    with pytest.raises(_lib.IxhError) as e:
        dp.gemv_noalloc(table, 1, x, y)
    assert e.value.code == -4 and "built-in buffer" in str(e.value)
    with pytest.raises(_lib.IxhError) as e:
        dp.gemv_noalloc(table, 1, x, y, flags=_lib.IXH_GEMV_ATOMIC)
    assert e.value.code == -1
    torch.cuda.synchronize()
    assert torch.all(y == 7.0)  # nothing ran


def test_noalloc_allocates_nothing_and_replays_in_a_graph(dev, gemv_option):
    """The device's free memory does not move over a run of calls (outputs allocated beforehand; the first call on a
    device, which looks the buffer's address up, is made before the measurement), and a call captured into a
    hipGraph replays correctly: three replays with new activations each time, eager work and a synchronisation
    between them, every replay equal to the eager ixh_gemv result.  The routes: row-block kernel (no workspace), the
    tile kernel with two workgroups to a block of rows (their pieces meet in the buffer and a second launch adds them),
    the staged and the column-block kernel (one piece per 512 columns in the buffer)."""
    from ixrun_amd import _lib

    gemv_option("gemv_tiles", 1)
    gemv_option("gemv_tile_cus", 4)
    gemv_option("gemv_tile_split", 2)
    cases = []
    for recipe, out_f, in_f, m, flags in (("student_t", 640, 4608, 1, 0), ("student_t", 640, 4608, 16, _lib.IXH_GEMV_FORCE_358),
                                          ("outlier", 96, 1536, 3, _lib.IXH_GEMV_STAGED),
                                          ("calibrated", 640, 4608, 2, _lib.IXH_GEMV_COLUMN_KERNEL)):
        dp, table = _layer(recipe, out_f, in_f, dev)
        x = activations(m, in_f, seed=11 + m).to(dev)
        y = torch.empty((m, out_f), dtype=torch.bfloat16, device=dev)
        cases.append((dp, table, x, y, flags))
    assert cases[1][0].gemv_workspace_bytes(512, 16, _lib.IXH_GEMV_FORCE_358) > 0
    for dp, table, x, y, flags in cases:  # warm: code object loaded, buffer address known, plans cached
        dp.gemv_noalloc(table, 512, x, y, flags=flags)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(dev)
    for _ in range(20):
        for dp, table, x, y, flags in cases:
            dp.gemv_noalloc(table, 512, x, y, flags=flags)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before

    for dp, table, x, y, flags in cases:
        m = x.shape[0]
        need = dp.gemv_workspace_bytes(512, m, flags)
        ws = torch.empty(max(need // 4, 1), dtype=torch.float32, device=dev)
        y_ref = torch.empty_like(y)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            dp.gemv_noalloc(table, 512, x, y, flags=flags)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            dp.gemv_noalloc(table, 512, x, y, flags=flags)
        for replay in range(3):
            x.copy_(activations(m, dp.in_f, seed=100 + replay).to(dev))
            y.fill_(7.0)
            dp.gemv(table, 512, x, y=y_ref, workspace=ws, flags=flags)  # eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert np.array_equal(bf16_bits(y), bf16_bits(y_ref)), (dp.out_f, m, flags, replay)


def test_noalloc_takes_a_large_layer_whose_kernels_fit(dev):
    """A layer whose full set of partial sums (one piece per 512 columns) is larger than the built-in buffer: the
    row-block kernels need none of it and the tile kernel divides a block of rows among at most eight workgroups, so
    the call runs and equals ixh_gemv with a full workspace; only the kernels with one piece per 512 columns are
    refused.  Weights made and encoded on the device (normal with a few large elements: 99 % level 1)."""
    from ixrun_amd import _lib

    out_f, in_f = 8320, 16384
    g = torch.Generator(device=dev).manual_seed(5)
    w = (torch.randn((out_f, in_f), generator=g, device=dev) * 0.008).bfloat16()
    w[::97, ::89] = 1.0
    dp, table, counts = _lib.encode_device(w, (3, 5, 8))
    del w
    assert counts[0] * 100 >= dp.N * 97
    for m in (1, 16):
        need = dp.gemv_workspace_bytes(512, m)
        x = activations(m, in_f, seed=21 + m).to(dev)
        ws = torch.empty(need // 4, dtype=torch.float32, device=dev)
        y_ref = torch.zeros((m, out_f), dtype=torch.bfloat16, device=dev)
        dp.gemv(table, 512, x, y=y_ref, workspace=ws)
        y_new = torch.full((m, out_f), 7.0, dtype=torch.bfloat16, device=dev)
        if m == 16:
            assert need > LIMIT
        dp.gemv_noalloc(table, 512, x, y_new)
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(y_ref), bf16_bits(y_new)), m
    x = activations(16, in_f, seed=3).to(dev)
    y = torch.full((16, out_f), 7.0, dtype=torch.bfloat16, device=dev)
    for flags in (_lib.IXH_GEMV_STAGED, _lib.IXH_GEMV_COLUMN_KERNEL):
        with pytest.raises(_lib.IxhError) as e:
            dp.gemv_noalloc(table, 512, x, y, flags=flags)
        assert e.value.code == -4 and "built-in buffer" in str(e.value)
    torch.cuda.synchronize()
    assert torch.all(y == 7.0)  # nothing ran
