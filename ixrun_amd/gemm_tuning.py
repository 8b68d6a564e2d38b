"""Choice of the library GEMM behind the many-row path (decode to bf16, then ``F.linear``).

The many-row product ``Y[M, out_f] = X[M, in_f] W[out_f, in_f]^T`` is a plain bf16 GEMM
(reference ``ixrun/engine.py:171-173``) and stays with the BLAS libraries.  Their default
pick is poor at prefill shapes: M = 512, out_f = 5120, in_f = 17408 runs in 172 us on
MI355X, while the best kernel that the same libraries hold needs 92 us (only 40 output
tiles of 256 x 256, so the winner is one that also splits K).  ``torch.cuda.tunable`` times
the candidates of a GEMM signature once and uses the winner for the rest of the process;
this module switches that on for exactly the shapes the layers meet, one shape at a time,
and leaves tuning off otherwise, so that unrelated GEMMs of the host program are never
held up.

Off by default: ``enable()`` turns it on (nothing is read from the environment).  The first call of a
new (rows, out_f, in_f, dtype, bias) signature then takes up to ``max_ms`` longer.  Nothing
is tuned while a graph is being captured: run one eager forward of each shape first.
"""
from __future__ import annotations

import os

import torch
import torch.nn.functional as F

_state = {"on": False, "max_ms": 300, "seen": set()}


def enable(max_ms: int = 300, results_file: str | None = None) -> None:
    """Use tuned library GEMMs in ``linear`` from now on (per process).

    torch keeps the winners in a csv file; ``results_file`` names one to
    read now and extend, so that a later process starts with them; without it the file is
    a per-process one in the temporary directory."""
    import tempfile

    import torch.cuda.tunable as tunable

    tunable.enable(True)
    tunable.tuning_enable(False)
    if results_file:
        tunable.set_filename(results_file)
        if os.path.exists(results_file):
            tunable.read_file(results_file)
    else:
        tunable.set_filename(os.path.join(tempfile.gettempdir(), f"ixrun_gemm_choices_{os.getpid()}.csv"))
    _state["on"] = True
    _state["max_ms"] = int(max_ms)


def disable() -> None:
    import torch.cuda.tunable as tunable

    tunable.tuning_enable(False)
    tunable.enable(False)
    _state["on"] = False


def enabled() -> bool:
    return bool(_state["on"])


def tuned_shapes():
    """Signatures tuned so far: (rows, out_f, in_f, dtype, with_bias)."""
    return sorted(_state["seen"], key=str)


def linear(x, w, bias=None):
    """``F.linear`` with the library GEMM chosen by measurement when tuning is enabled."""
    if not enabled() or not x.is_cuda:
        return F.linear(x, w, bias)
    rows = x.numel() // x.shape[-1] if x.shape[-1] else 0
    key = (rows, w.shape[0], w.shape[1], x.dtype, bias is not None)
    if key in _state["seen"] or torch.cuda.is_current_stream_capturing():
        return F.linear(x, w, bias)
    import torch.cuda.tunable as tunable

    tunable.set_max_tuning_duration(_state["max_ms"])
    tunable.tuning_enable(True)
    try:
        y = F.linear(x, w, bias)
    finally:
        tunable.tuning_enable(False)
    _state["seen"].add(key)
    return y
