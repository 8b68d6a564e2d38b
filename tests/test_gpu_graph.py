"""hipGraph capture of the per-layer launches: a chain of packed layers is
captured once and replayed; every replay must reproduce the eager result bit
for bit, also with other work and synchronisations between replays."""
import numpy as np
import pytest
import torch

from helpers import activations, bf16_bits, outlier_weight, student_t_weight

pytestmark = pytest.mark.gpu


def build_chain(n_layers, width, dev, maker):
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize

    layers = []
    for k in range(n_layers):
        sl = StreamingLinear(int8x_quantize(maker(width, width, seed=k)))
        layers.append(sl)
    return layers


def run_chain(layers, x):
    h = x
    for sl in layers:
        h = sl(h) * 4.0  # keep the activations from shrinking to nothing down the chain
    return h


@pytest.mark.parametrize("maker,m", [(student_t_weight, 1), (outlier_weight, 1), (student_t_weight, 4), (outlier_weight, 16)])
def test_graph_replay_matches_eager(maker, m):
    dev = torch.device("cuda:0")
    layers = build_chain(6, 1024, dev, maker)
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
