"""Deploy modules and engine of the INT8-X streaming path.

``StreamingLinear`` keeps a layer's packed streams resident on the GPU and
serves every forward from them: up to 16 activation rows go through the fused
decode+GEMV kernel (the bf16 weight never reaches memory), larger batches are
decoded into a shared bf16 buffer and multiplied with ``F.linear``.
``GraphLinear`` / ``Int8XEngine`` follow the reference's ``ixrun/engine.py``
(``StreamingLinear`` ``:40-173``, ``GraphLinear`` ``:179-196``,
``ResourceScheduler`` ``:202-235``, ``Int8XEngine`` ``:241-516``) and keep its
attribute names (``_b1 .. _l3, _scale, _b1_blk, _b2_blk, _q1, _q2,
_split_chunk, _use_fused, _w_buf``), which callers of ``fused_gemv`` read.
"""
from __future__ import annotations

import gc
import os

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib, gemm_tuning
from .config import TRITON_BLOCK
from .fused import FUSED_TILE, _pick_split, _workspaces, pick_unit, shared_workspace
from .linear import _set_parent_child, iter_quantizable_linears
from .quantize import int8x_quantize, portable_packed, quantize_for_deploy

__all__ = ["Int8XEngine", "StreamingLinear", "GraphLinear", "ResourceScheduler"]

try:  # the current stream's handle without building a Stream object (1 us less per forward)
    _raw_stream = torch._C._cuda_getCurrentRawStream
except AttributeError:  # pragma: no cover
    def _raw_stream(index):
        return torch.cuda.current_stream(index).cuda_stream

MAX_FUSED_ROWS = 16  # activation rows served by the fused decode+GEMV kernel
# With a decode buffer at hand, more rows than this go through decode + library GEMM.  Tensors that are almost all
# level 1, MI355X: the pair takes 72-75 us on 17408 x 5120 and 5120 x 17408 at any M up to 32 and 34-50 us on
# 5120 x 5120 (five levels: 73-74 and 38-39 us); the fused kernels take 25 / 27 us (17408 x 5120), 27 / 30 us
# (5120 x 17408) and 15 / 18 us (5120 x 5120) at M = 8 / 16 (five levels, measured before several workgroups could share
# a block of rows: 29 / 32, 39 / 51 and 23 / 31 us): every row count the fused kernels take.  Dense mixes (55 / 40 / 5 %): the pair takes
# 91-93 us on the large layers and 34-52 us on 5120 x 5120, the fused kernels 54-62 / 69-73 / 79-85 / 80-85 / 83-88 us
# (large layers) and 21 / 26 / 29 / 29 / 31 us (5120 x 5120) at M = 1 / 2 / 4 / 8 / 16: every row count as well.  Dense
# five-level mixes: one row 97-105 us fused against 120 us for the pair; two to sixteen rows 113-126 us fused (the
# decoder in its tile mode) against 119-123 us: the pair keeps those (the any-scheme kernel took 209-260 us).
MAX_FUSED_ROWS_WITH_BUFFER = 16
MAX_FUSED_ROWS_WITH_BUFFER_DENSE = 16
# 17 .. 32 rows on a large layer that is almost all level 1: two fused calls (16 rows and the rest) instead of the
# many-row paths.  MI355X, Student-t weights with 99.4 % of the elements in level 1, hipGraph replays over distinct
# layers: 5120 x 17408 at 17 / 24 / 32 rows 60 / 70 / 75 us in two calls against 118-120 us fused decode+GEMM and
# 137 us decode + library GEMM; 17408 x 5120 54 / 60 / 64 us against 120-122 and 87 us.  On 5120 x 5120 the two
# calls tie with the fused decode+GEMM (37-45 against 44-45 us) and lose to decode + library GEMM (34 us), and three
# calls for 33 .. 48 rows gain nothing on any shape: large layers and up to 32 rows only.
SPLIT_FUSED_MIN_WEIGHTS = 40_000_000
# More rows than that: with a shared decode buffer the layer decodes into it and calls the library GEMM
# (5120 x 5120 five-level on MI355X: 60 us at 32 rows, 84 us at 512); without one it runs the fused
# decode+GEMM, which keeps the bf16 weight out of HBM altogether but is slower (84 us and 194 us): its
# decode shares the CU with the matrix-core tiles at two waves per SIMD, the stand-alone decode runs at six.


class StreamingLinear(nn.Module):
    """GPU-resident packed weight, decoded inside every forward.

    Construction mirrors the reference (``ixrun/engine.py:49-104``): the packed
    tensors become buffers on the GPU and the rank tables are derived once.
    Here the tables are counted on the device from the bitmaps
    (``ixh_prefix_build``); ``_q1``/``_q2`` and ``_b1_blk``/``_b2_blk`` are the
    reference-shaped views of them.  Any level scheme is accepted; bitmaps and
    streams beyond the third level are registered as ``_b3``, ``_l4`` and so on.
    """

    def __init__(self, packed: dict, bias=None):
        super().__init__()
        self.out_features = packed["out_f"]
        self.in_features = packed["in_f"]
        self.N = packed["N"]
        self.level_bits = tuple(packed["level_bits"])
        self.counts = packed["counts"]

        n_levels = len(self.level_bits)
        for i in range(n_levels - 1):
            self.register_buffer(f"_b{i + 1}", packed["bitmaps"][i].cuda())
        for i in range(n_levels):
            self.register_buffer(f"_l{i + 1}", packed["streams"][i].cuda())
        self.register_buffer("_scale", packed["scale"].reshape(()).cuda())
        self._gemv_flags = 0  # extra IXH_GEMV_* flags of every fused call (comparisons: bench.py --gemv-flags)
        self._bind()

        # rank tables: the kernels' own (unit = 512 where rows allow it) and
        # the two the reference exposes
        self._unit = pick_unit(self.in_features)
        ready = packed.get("table512") if self._unit == 512 else None  # left by the device encoder
        self.register_buffer("_table", ready.cuda() if ready is not None else self._dp.prefix_build(self._unit))
        self._table_ptr = self._table.data_ptr()
        if self.N % TRITON_BLOCK == 0 and TRITON_BLOCK % self._unit == 0:
            blk_table = self._table[:, :: TRITON_BLOCK // self._unit][:, : self.N // TRITON_BLOCK]
        else:
            blk_table = self._dp.prefix_build(TRITON_BLOCK)[:, :-1]
        self.register_buffer("_b1_blk", blk_table[0].contiguous())
        self.register_buffer("_b2_blk", blk_table[1].contiguous() if n_levels > 2 else torch.zeros_like(blk_table[0]))
        self._use_triton = True

        self._use_fused = True
        self._gemm_ok = True
        self._split_chunk = 0
        per_row = self.in_features // self._unit
        split = _pick_split(self.in_features) if self.out_features < self.in_features else 1
        if split > 1 and self.in_features % FUSED_TILE == 0:
            self._split_chunk = self.in_features // split
            step = self._split_chunk // self._unit
        else:
            step = per_row
        q = self._table[:, : self.out_features * per_row : step]
        self.register_buffer("_q1", q[0].contiguous())
        self.register_buffer("_q2", q[1].contiguous() if n_levels > 2 else torch.zeros_like(q[0]))
        self._y32 = None

        if bias is not None:
            self.register_buffer("_bias", bias.detach().clone().cuda())
        else:
            self._bias = None
        self._w_buf = None  # set by the engine
        # the shared scratch takes its final size now, not inside some later forward (or graph capture)
        shared_workspace(self._scale.device, self._dp.gemv_workspace_bytes(self._unit, MAX_FUSED_ROWS))

    def _fused_gemm_wins(self, rows: int) -> bool:
        """Whether ``ixh_gemm`` beats decode + library GEMM when a decode buffer is at hand.

        Only its 128-row tile kernel does (3-bit first level, at least 97 % of the elements there, more
        than 2**24 elements), and only up to 512 activation rows, beyond which it decodes the weight once
        per 512 rows.  Measured on MI355X against the tuned library GEMM, 5120 x 17408: 70 / 77 / 111 us
        against 94 / 127 / 158 us at 128 / 256 / 512 rows; 4096 x 14336: 92 / 95 / 121 against
        105 / 113 / 142; 17408 x 5120: 82 / 95 / 142 against 80 / 96 / 126, which is why layers with more
        outputs than inputs go back to the library from 257 rows on."""
        return (self.level_bits[0] == 3 and self.N > (1 << 24) and self.counts[0] * 100 >= self.N * 97
                and (rows <= 256 or (rows <= 512 and self.in_features >= self.out_features)))

    def _bind(self):
        n_levels = len(self.level_bits)
        self._dp = _lib.DevicePacked(
            self.level_bits, self.out_features, self.in_features,
            [getattr(self, f"_b{i + 1}") for i in range(n_levels - 1)],
            [getattr(self, f"_l{i + 1}") for i in range(n_levels)],
            self._scale.reshape(1),
        )
        # what every fused call passes unchanged (the table follows the module when it moves: see _apply)
        import ctypes
        self._gemv_fn = _lib.lib().ixh_gemv
        self._struct_ref = ctypes.byref(self._dp.struct)
        self._table_ptr = self._table.data_ptr() if hasattr(self, "_table") else None
        self._plans = {}

    def _apply(self, fn, recurse=True):
        # .to()/.cuda() may move the buffers: point the kernel arguments at the new storage
        out = super()._apply(fn, recurse)
        if hasattr(self, "_scale") and self._scale.is_cuda:
            self._bind()
        return out

    def _set_shared_buf(self, w_buf):
        self._w_buf = w_buf
        self._plans = {}

    def _decode(self):
        """Decode into the shared buffer and return it as ``[out_f, in_f]``
        (reference ``ixrun/engine.py:109-133``)."""
        w_flat = self._w_buf[: self.N]
        self._dp.decode(self._table, self._unit, out_bf16=w_flat)
        return w_flat.view(self.out_features, self.in_features)

    def _fused_plan(self, rows):
        """How a forward of `rows` activation rows is served by the fused kernel: the row count of each call (one, or
        two for 17 .. 32 rows on a large layer that is almost all level 1) with the scratch it needs, or False where
        the many-row paths take over.  Worked out once per row count; ``_set_shared_buf`` and ``_bind`` forget the
        answers."""
        if self._w_buf is None:
            fused_rows = MAX_FUSED_ROWS
        elif self.counts[0] * 100 >= self.N * 97:
            fused_rows = MAX_FUSED_ROWS_WITH_BUFFER
        elif self.level_bits == (3, 5, 8):
            fused_rows = MAX_FUSED_ROWS_WITH_BUFFER_DENSE
        else:
            fused_rows = 1
        two_calls = (MAX_FUSED_ROWS < rows <= 2 * MAX_FUSED_ROWS and fused_rows == MAX_FUSED_ROWS
                     and self.N >= SPLIT_FUSED_MIN_WEIGHTS and self.counts[0] * 100 >= self.N * 97)
        plan = False
        if 1 <= rows <= fused_rows or two_calls:
            calls = []
            for r0 in range(0, rows, MAX_FUSED_ROWS):
                n = min(MAX_FUSED_ROWS, rows - r0)
                calls.append((r0, n, self._dp.gemv_workspace_bytes(self._unit, n, self._gemv_flags)))
            plan = tuple(calls)
        self._plans[rows] = plan
        return plan

    def forward(self, x):
        in_f = self.in_features
        if self._use_fused and x.dtype is torch.bfloat16 and x.is_cuda and in_f and x.shape[-1] == in_f:
            rows = x.numel() // in_f
            plan = self._plans.get(rows)
            if plan is None:
                plan = self._fused_plan(rows)
            if plan:
                # the hot path of token generation: one ctypes call with the arguments that never change kept bound
                out_f = self.out_features
                if not x.is_contiguous():
                    x = x.contiguous()
                dev = x.device
                y = torch.empty(x.shape[:-1] + (out_f,), dtype=torch.bfloat16, device=dev)
                x_ptr, y_ptr = x.data_ptr(), y.data_ptr()
                stream = _raw_stream(dev.index if dev.index is not None else torch.cuda.current_device())
                for r0, n, ws_bytes in plan:  # one call, or two on the same stream and workspace
                    ws = _workspaces.get(dev) if ws_bytes else None
                    if ws_bytes and (ws is None or ws.numel() * 4 < ws_bytes):
                        ws = shared_workspace(dev, ws_bytes)
                    rc = self._gemv_fn(self._struct_ref, self._table_ptr, self._unit, x_ptr + r0 * in_f * 2, n, in_f,
                                       y_ptr + r0 * out_f * 2, out_f, None, ws.data_ptr() if ws_bytes else None,
                                       ws_bytes, self._gemv_flags, stream)
                    if rc:
                        _lib.check(rc)
                if self._bias is not None:
                    y = y + self._bias.to(y.dtype)
                return y
        rows = x.numel() // in_f if in_f else 0
        if (self._use_fused and self._gemm_ok and x.dtype == torch.bfloat16 and x.is_cuda and rows > MAX_FUSED_ROWS
                and x.shape[-1] == self.in_features and self._unit == 512
                and (self._w_buf is None or self._fused_gemm_wins(rows))):
            # many rows: decode tiles on chip straight into the matrix-core GEMM, no bf16 weight in HBM
            x2 = x.reshape(rows, self.in_features)
            if x2.stride(1) != 1:
                x2 = x2.contiguous()
            y = torch.empty((rows, self.out_features), dtype=torch.bfloat16, device=x.device)
            ws = shared_workspace(x.device, self._dp.gemm_workspace_bytes(rows))
            try:
                self._dp.gemm(self._table, x2, y, ws)
            except _lib.IxhError as e:
                if e.code != _lib.IXH_EUNSUPPORTED:
                    raise
                self._gemm_ok = False  # shape the fused GEMM does not take: decode + GEMM from here on
            else:
                y = y.view(x.shape[:-1] + (self.out_features,))
                if self._bias is not None:
                    y = y + self._bias.to(y.dtype)
                return y
        w = self._decode()
        bias = self._bias.to(x.dtype) if self._bias is not None else None
        return gemm_tuning.linear(x, w.to(x.dtype) if w.dtype != x.dtype else w, bias)


class GraphLinear(nn.Module):
    """GEMM-only layer whose weight buffer is refreshed by a captured graph of
    decode launches (reference ``ixrun/engine.py:179-196``)."""

    def __init__(self, packed: dict, bias=None, decode_buf=None):
        super().__init__()
        self.out_features = packed["out_f"]
        self.in_features = packed["in_f"]
        self.N = packed["N"]
        self._w_buf = decode_buf
        if bias is not None:
            self.register_buffer("_bias", bias.detach().clone().cuda())
        else:
            self._bias = None

    def forward(self, x):
        w = self._w_buf[: self.N].view(self.out_features, self.in_features)
        bias = self._bias.to(x.dtype) if self._bias is not None else None
        return gemm_tuning.linear(x, w, bias)


class ResourceScheduler:
    """Memory estimates and a mode recommendation (reference ``ixrun/engine.py:202-235``)."""

    @staticmethod
    @torch.no_grad()
    def estimate(model: nn.Module, level_bits=(3, 5, 8)) -> dict:
        bf16_bytes = packed_bytes = n_elems = max_layer = 0
        for _, mod in iter_quantizable_linears(model):
            w = mod.weight.data
            packed_bytes += int8x_quantize(w, level_bits)["total_bytes"]
            bf16_bytes += w.numel() * 2
            n_elems += w.numel()
            max_layer = max(max_layer, w.numel())
        return {
            "bf16_weight_MB": bf16_bytes / 1e6,
            "packed_storage_MB": packed_bytes / 1e6,
            "compression": bf16_bytes / max(packed_bytes, 1),
            "max_layer_elems": max_layer,
            "shared_decode_buf_MB": max_layer * 2 / 1e6,
            "n_elems": n_elems,
        }

    @staticmethod
    def recommend(model: nn.Module, gpu_budget_GB: float, level_bits=(3, 5, 8)) -> str:
        est = ResourceScheduler.estimate(model, level_bits)
        return "cached" if est["bf16_weight_MB"] + 1500 <= gpu_budget_GB * 1000 else "streaming"


class Int8XEngine:
    """Load a model, deploy it on packed weights, generate.

    Same construction and deploy modes as the reference's ``Int8XEngine``
    (``ixrun/engine.py:241-516``).  The three ``_deploy_*`` helpers take any
    ``nn.Module``; ``from_pretrained`` needs ``transformers`` and a local
    checkpoint, as in the reference.
    """

    def __init__(self, model, tokenizer, stats=None, graph_replay=None):
        self.model = model
        self.tokenizer = tokenizer
        self.stats = stats or {}
        self._graph_replay = graph_replay
        self.model.eval()

    @classmethod
    def from_pretrained(cls, model_path: str, mode: str = "cached", level_bits=(3, 5, 8),
                        dtype=torch.bfloat16, verbose: bool = True, cache_path: str | None = None):
        from transformers import AutoModelForCausalLM, AutoTokenizer

        tokenizer = AutoTokenizer.from_pretrained(model_path, trust_remote_code=True)
        if tokenizer.pad_token is None:
            tokenizer.pad_token = tokenizer.eos_token
        big = mode in ("streaming", "graph")
        model = AutoModelForCausalLM.from_pretrained(model_path, dtype=dtype, low_cpu_mem_usage=True)
        if not big:
            model = model.cuda()
        if mode == "streaming":
            stats = cls._deploy_streaming(model, level_bits, verbose=verbose, cache_path=cache_path)
        elif mode == "graph":
            stats, replay = cls._deploy_graph(model, level_bits, verbose=verbose)
            return cls(model, tokenizer, stats, graph_replay=replay)
        else:
            stats = cls._deploy_cached(model, level_bits, verbose=verbose)
        eng = cls(model, tokenizer, stats)
        if big:
            eng._finalize_device()
        return eng

    # ----- deploy helpers ---------------------------------------------------
    @staticmethod
    def _deploy_cached(model, level_bits, verbose=True):
        from .linear import deploy_model

        return deploy_model(model, level_bits=level_bits, cache="full", verbose=verbose)

    @staticmethod
    @torch.no_grad()
    def _deploy_streaming(model, level_bits, verbose=True, cache_path=None):
        """Packed weights resident on the GPU plus one shared decode buffer
        (reference ``ixrun/engine.py:343-416``).  ``cache_path`` names a file of
        already packed layers, ``{"level_bits": ..., "layers": [(name, packed,
        bias), ...]}``, written on the first deploy and read on later ones; a
        cache built with other ``level_bits`` or for other layer names raises
        ``ValueError`` as in the reference (``:360-370``)."""
        targets = list(iter_quantizable_linears(model))
        layer_data = None
        if cache_path is not None and os.path.exists(cache_path):
            if verbose:
                print(f"[engine][cache] loading packed weights from {cache_path}", flush=True)
            # tuples, dicts, numbers and tensors only: the safe loader reads all of it
            blob = torch.load(cache_path, map_location="cpu", weights_only=True)
            if tuple(blob["level_bits"]) != tuple(level_bits):
                raise ValueError(
                    f"cache was built with level_bits={blob['level_bits']}, "
                    f"requested {tuple(level_bits)}; delete the cache or change level_bits")
            layer_data = blob["layers"]
            have = {n for n, _ in model.named_modules()}
            missing = [n for n, _, _ in layer_data if n not in have]
            if missing:
                raise ValueError(f"cache/model mismatch: {len(missing)} unknown layers")
            if verbose:
                print(f"[engine][cache] {len(layer_data)} layers loaded", flush=True)
        if layer_data is None:
            layer_data = []
            for name, mod in targets:
                bias = mod.bias.data if mod.bias is not None else None
                layer_data.append((name, quantize_for_deploy(mod.weight.data, level_bits), bias))
            if cache_path is not None:
                if verbose:
                    print(f"[engine][cache] saving packed weights to {cache_path}", flush=True)
                torch.save({"level_bits": tuple(level_bits),
                            "layers": [(n, portable_packed(p), b) for n, p, b in layer_data]}, cache_path)

        total_bytes = max_n = 0
        layers = []
        for name, packed, bias in layer_data:
            layers.append((name, StreamingLinear(packed, bias=bias)))
            total_bytes += packed["total_bytes"]
            max_n = max(max_n, packed["N"])
        shared_w = torch.empty(max_n, dtype=torch.bfloat16, device="cuda")
        for name, sl in layers:
            sl._set_shared_buf(shared_w)
            _set_parent_child(model, name, sl)
        gc.collect()
        torch.cuda.empty_cache()
        shared_mb = shared_w.numel() * 2 / 1e6
        if verbose:
            print(f"[engine][streaming] {len(layers)} layers | packed GPU-resident={total_bytes / 1e6:.0f}MB | "
                  f"shared decode buf={shared_mb:.1f}MB", flush=True)
        return {"mode": "streaming", "n_layers": len(layers), "total_bytes": total_bytes, "shared_gpu_MB": shared_mb}

    @staticmethod
    @torch.no_grad()
    def _deploy_graph(model, level_bits, verbose=True):
        """Streaming deploy with every layer's decode launch captured in one
        graph (reference ``ixrun/engine.py:420-487``): each layer gets its own
        decode buffer, the graph replays all decodes, forwards are GEMM-only."""
        targets = list(iter_quantizable_linears(model))
        total_params = sum(m.weight.numel() for _, m in targets)
        if total_params * 2 > torch.cuda.get_device_properties(0).total_memory * 0.9:
            raise RuntimeError(
                f"graph mode needs {total_params * 2 / 1e9:.1f}GB of per-layer decode buffers "
                f"- too large for this GPU; use mode='streaming'")
        total_bytes = 0
        specs = []
        for name, mod in targets:
            packed = quantize_for_deploy(mod.weight.data, level_bits)
            bias = mod.bias.data if mod.bias is not None else None
            sl = StreamingLinear(packed, bias=bias)
            buf = torch.empty(packed["N"], dtype=torch.bfloat16, device="cuda")
            sl._set_shared_buf(buf)
            specs.append((name, sl, buf))
            total_bytes += packed["total_bytes"]

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _, sl, _ in specs:
                sl._decode()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _, sl, _ in specs:
                sl._decode()
        torch.cuda.synchronize()
        if verbose:
            print(f"[engine][graph] captured {len(specs)} decode kernels", flush=True)
        for name, sl, buf in specs:
            meta = {"out_f": sl.out_features, "in_f": sl.in_features, "N": sl.N}
            _set_parent_child(model, name, GraphLinear(meta, bias=sl._bias, decode_buf=buf))

        def replay(_keep_alive=specs, _graph=graph):
            _graph.replay()

        if verbose:
            print(f"[engine][graph] {len(specs)} layers | packed={total_bytes / 1e6:.0f}MB | decode=graph.replay()",
                  flush=True)
        return {"mode": "graph", "n_layers": len(specs), "total_bytes": total_bytes}, replay

    # ----- inference --------------------------------------------------------
    def _finalize_device(self):
        """Move whatever the deploy left on the CPU (reference ``ixrun/engine.py:490-504``)."""
        for _, mod in self.model.named_modules():
            for p in mod.parameters(recurse=False):
                if p.data.device.type != "cuda":
                    p.data = p.data.cuda()
            for bname, b in mod.named_buffers(recurse=False):
                if b.device.type != "cuda":
                    setattr(mod, bname, b.cuda())
        gc.collect()
        torch.cuda.empty_cache()
        self.model.eval()

    def _pre_forward(self):
        if self._graph_replay is not None:
            self._graph_replay()

    @torch.no_grad()
    def generate(self, prompt, max_new_tokens: int = 64, **kw):
        """Greedy text generation through the wrapped model's own ``generate``."""
        self._pre_forward()
        ids = self.tokenizer(prompt, return_tensors="pt").to("cuda")
        out = self.model.generate(**ids, max_new_tokens=max_new_tokens, do_sample=False, **kw)
        return self.tokenizer.decode(out[0][ids["input_ids"].shape[1]:], skip_special_tokens=True)
