"""hipGraph capture of the per-layer launches: a chain of packed layers is
captured once and replayed; every replay must reproduce the eager result bit
for bit, also with other work and synchronisations between replays."""
import numpy as np
import pytest
import torch

from helpers import activations, bf16_bits, outlier_weight, student_t_weight

pytestmark = pytest.mark.gpu


def build_chain(n_layers, width, dev, maker, level_bits=(3, 5, 8)):
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize

    layers = []
    for k in range(n_layers):
        sl = StreamingLinear(int8x_quantize(maker(width, width, seed=k), level_bits))
        layers.append(sl)
    return layers


def dense_weight(out_f, in_f, seed=0):
    """Weights whose every level is well populated, in (3,5,8) and in (3,4,5,6,8)."""
    from helpers import calibrated_weight

    return calibrated_weight(out_f, in_f, seed=seed, scale=0.0123046875)[0]


def run_chain(layers, x):
    h = x
    for sl in layers:
        h = sl(h) * 4.0  # keep the activations from shrinking to nothing down the chain
    return h


@pytest.mark.parametrize("maker,m,level_bits", [
    (student_t_weight, 1, (3, 5, 8)), (outlier_weight, 1, (3, 5, 8)), (student_t_weight, 4, (3, 5, 8)),
    (outlier_weight, 16, (3, 5, 8)), (dense_weight, 1, (3, 4, 5, 6, 8)), (student_t_weight, 16, (3, 4, 5, 6, 8)),
    (dense_weight, 2, (3, 5, 8)), (dense_weight, 8, (3, 5, 8)), (dense_weight, 16, (3, 5, 8)), (student_t_weight, 8, (3, 5, 8)),
    (student_t_weight, -8, (3, 5, 8)), (student_t_weight, -16, (3, 4, 5, 6, 8))])
def test_graph_replay_matches_eager(maker, m, level_bits, gemv_option):
    dev = torch.device("cuda:0")
    if m < 0:  # the tile kernel with two workgroups to a block of rows: two launches a layer, pieces in the shared scratch
        m = -m
        gemv_option("gemv_tiles", 1)
        gemv_option("gemv_tile_cus", 8)
        gemv_option("gemv_tile_split", 2)
    layers = build_chain(6, 1024, dev, maker, level_bits)
    x = activations(m, 1024, seed=3).to(dev)
    eager = run_chain(layers, x).clone()
    torch.cuda.synchronize()

    static_x = x.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_chain(layers, static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = run_chain(layers, static_x)
    for rep in range(4):
        # unrelated eager work and a sync between replays
        junk = torch.randn(1 << 16, device=dev).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager), f"replay {rep} differs from the eager result"
        del junk
    # new input through the same graph
    x2 = activations(m, 1024, seed=4).to(dev)
    static_x.copy_(x2)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(static_y, run_chain(layers, x2))


@pytest.mark.parametrize("shared_buffer", [False, True])
def test_graph_replay_many_rows(shared_buffer):
    """48 activation rows: the fused decode + MFMA GEMM (no decode buffer) and the bf16 decode + library GEMM
    (with one), captured and replayed; five-level and dense (3,5,8) layers alternate down the chain."""
    from helpers import calibrated_weight
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize

    dev = torch.device("cuda:0")
    width, m = 1024, 48
    layers = []
    for k in range(4):
        if k % 2 == 0:
            packed = int8x_quantize(student_t_weight(width, width, seed=k), (3, 4, 5, 6, 8))
        else:
            packed = int8x_quantize(calibrated_weight(width, width, seed=k, scale=0.0123046875)[0])
        layers.append(StreamingLinear(packed))
    if shared_buffer:
        shared = torch.empty(width * width, dtype=torch.bfloat16, device=dev)
        for sl in layers:
            sl._set_shared_buf(shared)
    x = activations(m, width, seed=3).to(dev)
    eager = run_chain(layers, x).clone()
    torch.cuda.synchronize()

    static_x = x.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_chain(layers, static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = run_chain(layers, static_x)
    for rep in range(3):
        junk = torch.randn(1 << 16, device=dev).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager), f"replay {rep} differs from the eager result"
        del junk


def _capture(fn, static_x):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn(static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = fn(static_x)
    return graph, static_y


def test_graph_64_layers_of_5120x5120():
    """BASELINE config 5b as stated: a sequence of 64 packed 5120 x 5120 layers (64 distinct device copies, 0.85 GB
    of packed bytes), every per-layer launch captured in one hipGraph.  Replays equal the eager pass bit for bit; the
    first and the last layer's outputs are checked against the fp64 oracle on the inputs they really saw."""
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize
    from oracle import ix_oracle
    from test_gpu_parity import check_outputs

    dev = torch.device("cuda:0")
    width, n_layers, n_distinct = 5120, 64, 4
    packed = [int8x_quantize(student_t_weight(width, width, seed=k)) for k in range(n_distinct)]
    layers = [StreamingLinear(packed[k % n_distinct]) for k in range(n_layers)]

    def chain(x, keep=None):
        h = x
        for k, sl in enumerate(layers):
            if keep is not None and k == n_layers - 1:
                keep["last_in"] = h.clone()
            h = sl(h) * 0.7  # output std is 1.43 x input std at this width: keep the chain in range
            if keep is not None and k == 0:
                keep["first_out"] = h.clone()
        return h

    x = activations(1, width, seed=3).to(dev)
    seen = {}
    eager = chain(x, seen).clone()
    torch.cuda.synchronize()
    assert torch.isfinite(eager.float()).all() and eager.float().abs().max() > 0

    # layer outputs against the oracle (the 0.7 is a bf16 multiply: applied to the oracle's bf16-rounded result)
    for w, xin, got in ((packed[0], x, seen["first_out"]), (packed[(n_layers - 1) % n_distinct], seen["last_in"], eager)):
        y64 = ix_oracle.gemm_f64(ix_oracle.decode_packed_bf16(w), bf16_bits(xin))
        y_layer = torch.from_numpy(ix_oracle.bf16_bits_to_f32(ix_oracle.f32_to_bf16_bits(y64.astype(np.float32))))
        want = (y_layer.bfloat16() * 0.7).double().numpy()
        err = np.linalg.norm(got.double().cpu().numpy() - want) / np.linalg.norm(want)
        assert err <= 1e-3, err

    static_x = x.clone()
    graph, static_y = _capture(chain, static_x)
    for rep in range(3):
        junk = torch.randn(1 << 16, device=dev).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager), f"replay {rep} differs from the eager pass"
        del junk
    x2 = activations(1, width, seed=4).to(dev)
    static_x.copy_(x2)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(static_y, chain(x2))


def test_graph_survives_a_larger_workspace_request():
    """A graph captured while the shared scratch was small keeps working after a bigger layer made the scratch grow:
    the replaced buffer stays alive, so the replay neither reads freed memory nor writes into tensors allocated
    afterwards."""
    from ixrun_amd import fused
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize

    dev = torch.device("cuda:0")
    fused._workspaces.pop(dev, None)  # start from no scratch, whatever earlier tests left
    # five-level layers with a dense mix: the staged kernel, whose pieces of a row meet in the workspace
    layers = [StreamingLinear(int8x_quantize(outlier_weight(256, 2048, seed=k), (3, 4, 5, 6, 8))) for k in range(2)]
    layers.append(StreamingLinear(int8x_quantize(outlier_weight(2048, 256, seed=9), (3, 4, 5, 6, 8))))

    def chain(x):
        return layers[1](layers[2](layers[0](x)))

    x = activations(3, 2048, seed=3).to(dev)
    eager = chain(x).clone()
    small = fused._workspaces[dev]
    static_x = x.clone()
    graph, static_y = _capture(chain, static_x)
    assert fused._workspaces[dev] is small  # the capture itself did not grow it

    big = StreamingLinear(int8x_quantize(outlier_weight(4096, 8192, seed=5), (3, 4, 5, 6, 8)))
    big(activations(16, 8192, seed=1).to(dev))
    assert fused._workspaces[dev] is not small and any(t is small for t in fused._retired)
    del small
    torch.cuda.synchronize()
    canaries = [torch.full((1 << 18,), 3.0, device=dev) for _ in range(16)]  # what a freed scratch would be given to
    for rep in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager), f"replay {rep} after the scratch grew"
        assert all(bool((c == 3.0).all()) for c in canaries)
