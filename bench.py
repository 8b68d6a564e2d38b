#!/usr/bin/env python3
"""Headline benchmark: fused (3,5,8) decode + GEMV on the 5120x17408 batch-1 layer.

One step = one fused decode+GEMV over one packed layer.  The timed region walks
round-robin over COPIES distinct packed copies of the layer (together larger
than the 256 MB last-level cache) so that every launch streams its packed bytes
from HBM.  Inputs are resident on the GPU before the clock starts.

Prints one JSON line.  Extra workloads (--workload) time the other shapes of the
hot path with the same harness; the many-row (prefill) workload runs the fused
decode + matrix-core GEMM and is priced against the bf16 MFMA peak.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK = 8.0e12  # B/s, MI355X published
MFMA_BF16_PEAK = 2.5e15  # FLOP/s dense bf16, MI355X published

# HBM bytes per launch of the dominant kernel, from two rocprofv3 --pmc runs of this script (FETCH_SIZE, then
# WRITE_SIZE, KiB per dispatch, scaled by what the same counters read for the 256 MiB copy of --calibrate-copy:
# x 2.0 and x 1.0); the counter summaries are kept under profiles/.  Each figure carries the hash of the kernel
# sources it was measured on (kernel_sources_sha16) and is reported only while the sources still hash to it;
# workloads without a counter run, or measured on other sources, report null.
# (bytes per launch, the sources the kernel is compiled from, their kernel_sources_sha16 at the counter run)
_ROWS = ("ixh_rows358.hip", "ixh_rows_common.h", "ixh_dev.h", "build.sh")
_TILES = ("ixh_tiles358.hip", "ixh_rows_common.h", "ixh_dev.h")
_DENSE = ("ixh_dense358.hip", "ixh_dense_tiles.h", "ixh_dev.h")
_DENSE5 = ("ixh_dense5.hip", "ixh_dense_tiles.h", "ixh_dev.h")
_PREFILL = ("ixh_prefill358.hip", "ixh_prefill358.h", "ixh_rows_common.h", "ixh_dev.h")
_DECODE_ROWS = ("ixh_decode_rows358.hip", "ixh_rows_common.h", "ixh_dev.h")
_OLD = ((), "measured-on-earlier-sources")  # figures kept for the record; reported as null
MEASURED_TRAFFIC_BYTES = {
    "down_proj_5120x17408_m1_student_t": (23032.0 * 2.0 * 1024 + 16.0 * 1024, _ROWS, "3e8407b518bc293b"),
    "gate_up_17408x5120_m1_student_t": (22936.0 * 2.0 * 1024 + 40.0 * 1024, _ROWS, "3e8407b518bc293b"),
    "attn_proj_5120x5120_m1_student_t": (7135.0 * 2.0 * 1024 + 16.0 * 1024, _ROWS, "3e8407b518bc293b"),
    "down_proj_5120x17408_m1_calibrated": (33825.0 * 2.0 * 1024 + 40.0 * 1024, _DENSE, "711eef94d053feb1"),
    "down_proj_5120x17408_m1_five_level_calibrated": (49708.0 * 2.0 * 1024 + 1338.0 * 1024, _DENSE5, "aaca19573f1ed2a1"),
    "gate_up_17408x5120_m4_student_t": (28740.0 * 2.0 * 1024 + 160.0 * 1024, _TILES, "21f9d013a3b417ff"),
    "gate_up_17408x5120_m16_student_t": (26687.0 * 2.0 * 1024 + 640.0 * 1024, _TILES, "21f9d013a3b417ff"),
    "attn_proj_5120x5120_m16_student_t": (8657.0 * 2.0 * 1024 + 640.0 * 1024, _TILES, "21f9d013a3b417ff"),
    "down_proj_5120x17408_m16_student_t": (27677.0 * 2.0 * 1024 + 960.0 * 1024, _TILES, "21f9d013a3b417ff"),
    "decode_5120x17408_five_level_calibrated": (49719.0 * 2.0 * 1024 + 174080.0 * 1024, _DENSE5, "aaca19573f1ed2a1"),
    "prefill_5120x5120_m512_five_level": (50297.9 * 2.0 * 1024 + 30720.0 * 1024,) + _OLD,
    # the three kernels of a step: k_prefill_xtile + k_prefill358 + k_prefill358_reduce
    "prefill_5120x17408_m512_five_level": ((8716.0 + 68452.0 + 30734.0) * 2.0 * 1024 + (17408.0 + 61606.0 + 5120.0) * 1024,
                                           _PREFILL, "55862ec6d8c72acd"),
    # k_decode358_rows<true> (x 2.0 / x 1.0 as above) + the operands and outputs of the library GEMM that
    # torch.cuda.tunable picked (bf16 weight, X, Y: its FETCH_SIZE, 158,001, is weighted for other request sizes than
    # our kernels' and fixes its reads only between 162 and 324 MB)
    "prefill_5120x17408_m512_five_level_unfused": (23101.0 * 2.0 * 1024 + 179854.0 * 1024
                                                   + 2.0 * (5120 * 17408 + 512 * 17408 + 512 * 5120),
                                                   _DECODE_ROWS, "54f9e436740640ef"),
    "decode_5120x17408_student_t": (23268.0 * 2.0 * 1024 + 179524.0 * 1024,) + _OLD,
    "decode_5120x17408_calibrated": (36308.0 * 2.0 * 1024 + 174080.0 * 1024,) + _OLD,
    "decode_gs_5120x17408_student_t": (33559.0 * 2.0 * 1024 + 174080.0 * 1024,) + _OLD,
    # all kernels of one encode step together (absmax, count, scans, clear, pack)
    "encode_5120x17408_student_t": ((87053 + 87092 + 1402 + 15 + 92442) * 2.0 * 1024 + (32 + 2040 + 1362 + 32694 + 63405) * 1024,) + _OLD,
}

# Wave-level instruction counts per launch of the dominant kernel (SQ_INSTS_VALU, SQ_INSTS_SALU, SQ_INSTS_LDS from one
# rocprofv3 --pmc run of this script, mean over the launches), gated by the hash of the kernel's sources like the
# traffic figures.  Reported per weight: vector and LDS instructions x 64 lanes / weights, scalar instructions / weights.
MEASURED_INSTRUCTIONS = {
    "down_proj_5120x17408_m1_student_t": ((5734195.0, 4469166.0, 1360042.0), _ROWS, "3e8407b518bc293b"),
    "gate_up_17408x5120_m1_student_t": ((6030194.0, 4450915.0, 1414314.0), _ROWS, "3e8407b518bc293b"),
    "attn_proj_5120x5120_m1_student_t": ((3570752.0, 2281697.0, 593732.0), _ROWS, "3e8407b518bc293b"),
    "down_proj_5120x17408_m1_level1_only": ((4881551.0, 4104235.0, 1254926.0), _ROWS, "3e8407b518bc293b"),
}

WORKLOADS = {
    # name: (out_f, in_f, m, weight recipe)
    "down_proj_5120x17408_m1_student_t": (5120, 17408, 1, "student_t"),
    "down_proj_5120x17408_m1_calibrated": (5120, 17408, 1, "calibrated"),
    # the reference tests' own weight recipe (tests/test_fused.py:17-22): N(0, 0.005) with 4 % N(0, 0.05) outliers
    "down_proj_5120x17408_m1_reference_recipe": (5120, 17408, 1, "outlier"),
    # no element above level 1 (but one): what the record queue and its resolution cost shows against the headline
    "down_proj_5120x17408_m1_level1_only": (5120, 17408, 1, "level1_only"),
    "down_proj_5120x17408_m1_five_level": (5120, 17408, 1, "student_t", (3, 4, 5, 6, 8)),
    # the fraction-calibrated weights in the five-level scheme: every level populated
    "down_proj_5120x17408_m1_five_level_calibrated": (5120, 17408, 1, "calibrated", (3, 4, 5, 6, 8)),
    "attn_proj_5120x5120_m1_five_level": (5120, 5120, 1, "student_t", (3, 4, 5, 6, 8)),
    "attn_proj_5120x5120_m1_calibrated": (5120, 5120, 1, "calibrated"),
    "graph64_5120x5120_m1_calibrated": (5120, 5120, 1, "calibrated"),
    # level-1 share swept between the dense mix and the almost-all-level-1 mix (the rest 8 : 1 between levels 2 and 3):
    # where the row-block kernels (--gemv-flags 8) and the level-by-level kernel (--gemv-flags 32) cross
    **{f"down_proj_5120x17408_m1_l1_share_{pct}": (5120, 17408, 1, f"l1_share_{pct}") for pct in (80, 85, 90, 95, 97, 99)},
    "attn_proj_5120x5120_m1_student_t": (5120, 5120, 1, "student_t"),
    "down_proj_5120x17408_m4_student_t": (5120, 17408, 4, "student_t"),
    "down_proj_5120x17408_m8_student_t": (5120, 17408, 8, "student_t"),
    "down_proj_5120x17408_m16_student_t": (5120, 17408, 16, "student_t"),
    "down_proj_5120x17408_m2_student_t": (5120, 17408, 2, "student_t"),
    "attn_proj_5120x5120_m2_student_t": (5120, 5120, 2, "student_t"),
    "attn_proj_5120x5120_m4_student_t": (5120, 5120, 4, "student_t"),
    "attn_proj_5120x5120_m8_student_t": (5120, 5120, 8, "student_t"),
    "attn_proj_5120x5120_m16_student_t": (5120, 5120, 16, "student_t"),
    "gate_up_17408x5120_m1_student_t": (17408, 5120, 1, "student_t"),
    "gate_up_17408x5120_m2_student_t": (17408, 5120, 2, "student_t"),
    "gate_up_17408x5120_m4_student_t": (17408, 5120, 4, "student_t"),
    "gate_up_17408x5120_m8_student_t": (17408, 5120, 8, "student_t"),
    "gate_up_17408x5120_m16_student_t": (17408, 5120, 16, "student_t"),
    "gate_up_17408x5120_m2_calibrated": (17408, 5120, 2, "calibrated"),
    "gate_up_17408x5120_m4_calibrated": (17408, 5120, 4, "calibrated"),
    "gate_up_17408x5120_m8_calibrated": (17408, 5120, 8, "calibrated"),
    "gate_up_17408x5120_m16_calibrated": (17408, 5120, 16, "calibrated"),
    "down_proj_5120x17408_m8_calibrated": (5120, 17408, 8, "calibrated"),
    # dense five-level mixes at several rows: the five-level decoder's tile mode
    "down_proj_5120x17408_m8_five_level_calibrated": (5120, 17408, 8, "calibrated", (3, 4, 5, 6, 8)),
    "gate_up_17408x5120_m8_five_level_calibrated": (17408, 5120, 8, "calibrated", (3, 4, 5, 6, 8)),
    "attn_proj_5120x5120_m8_calibrated": (5120, 5120, 8, "calibrated"),
    # 64 distinct 5120x5120 layers chained (each output feeds the next layer), one hipGraph: us per layer
    "graph64_5120x5120_m1_student_t": (5120, 5120, 1, "student_t"),
    # many activation rows: decode into LDS tiles + bf16 MFMA, five-level scheme
    "prefill_5120x5120_m512_five_level": (5120, 5120, 512, "student_t", (3, 4, 5, 6, 8)),
    "prefill_5120x5120_m512_358": (5120, 5120, 512, "student_t"),
    "prefill_5120x17408_m512_358": (5120, 17408, 512, "student_t"),
    "prefill_5120x17408_m512_five_level": (5120, 17408, 512, "student_t", (3, 4, 5, 6, 8)),
    "prefill_5120x5120_m64_five_level": (5120, 5120, 64, "student_t", (3, 4, 5, 6, 8)),
    "prefill_5120x5120_m128_five_level": (5120, 5120, 128, "student_t", (3, 4, 5, 6, 8)),
    "prefill_5120x5120_m256_five_level": (5120, 5120, 256, "student_t", (3, 4, 5, 6, 8)),
    "prefill_5120x5120_m32_five_level": (5120, 5120, 32, "student_t", (3, 4, 5, 6, 8)),
    # deploy-time encoder on the device: bf16 weight in HBM -> packed streams + rank table (m is unused)
    "encode_5120x17408_student_t": (5120, 17408, 0, "student_t"),
    "encode_5120x17408_calibrated": (5120, 17408, 0, "calibrated"),
    "encode_5120x17408_five_level": (5120, 17408, 0, "student_t", (3, 4, 5, 6, 8)),
    # full decode to bf16 in HBM (m is unused): the per-tensor format and the group-scale sibling format
    "decode_5120x17408_student_t": (5120, 17408, 0, "student_t"),
    "decode_5120x17408_calibrated": (5120, 17408, 0, "calibrated"),
    "decode_5120x17408_five_level_calibrated": (5120, 17408, 0, "calibrated", (3, 4, 5, 6, 8)),
    "decode_gs_5120x17408_student_t": (5120, 17408, 0, "student_t"),
}


def make_weight(out_f, in_f, recipe):
    from helpers import calibrated_weight, outlier_weight, student_t_weight

    if recipe == "student_t":
        return student_t_weight(out_f, in_f, seed=0)
    if recipe == "outlier":
        return outlier_weight(out_f, in_f, seed=0)
    if recipe.startswith("l1_share_"):
        l1 = int(recipe.rsplit("_", 1)[1]) / 100.0
        return calibrated_weight(out_f, in_f, seed=0, fractions=(l1, (1.0 - l1) * 8 / 9, (1.0 - l1) / 9))[0]
    if recipe == "level1_only":  # every value within the first level but the one +-127 that fixes the scale
        return calibrated_weight(out_f, in_f, seed=0, fractions=(1.0, 0.0, 0.0))[0]
    return calibrated_weight(out_f, in_f, seed=0)[0]


def cpu_baseline(weight, x, level_bits=(3, 5, 8), rows=640):
    """The reference's CPU path on the host cores: torch scatter decode of the packed
    layer to bf16 (ixrun/quantize.py:154-183 restated in ixrun_amd.quantize) followed
    by F.linear, on the first `rows` rows of the same weight so that it stays bounded;
    next to it the oracle's single-core C walk (decode + fp32 dot) over the same rows."""
    import torch.nn.functional as F

    from ixrun_amd.quantize import decode_to_weight, int8x_quantize
    from oracle import ix_oracle as oracle

    sub = int8x_quantize(weight[:rows].contiguous(), level_bits)
    n = sub["N"]
    xs = x[:1]
    xs32 = xs.float()
    t_dec, t_mm16, t_mm32 = [], [], []
    for rep in range(3 + 10):  # 3 warm-ups, 10 timed repetitions, medians
        t0 = time.perf_counter()
        w = decode_to_weight(sub, device="cpu")
        t1 = time.perf_counter()
        F.linear(xs, w)
        t2 = time.perf_counter()
        F.linear(xs32, w.float())  # the fp32 variant: the bf16 weight widened, then the product
        t3 = time.perf_counter()
        if rep >= 3:
            t_dec.append(t1 - t0), t_mm16.append(t2 - t1), t_mm32.append(t3 - t2)
    dec, mm16, mm32 = float(np.median(t_dec)), float(np.median(t_mm16)), float(np.median(t_mm32))
    pn = oracle.packed_to_numpy(sub)
    xb = xs[0].contiguous().view(torch.int16).numpy().view(np.uint16)
    reps, t0 = 0, time.perf_counter()
    while reps < 10 or time.perf_counter() - t0 < 3.0:
        oracle.fused_gemv_f32(rows, pn["in_f"], pn["level_bits"], pn["bitmaps"], pn["streams"], pn["last"],
                              pn["scale_bits"], xb)
        reps += 1
    t_c = (time.perf_counter() - t0) / reps
    return {
        "value": n / (dec + mm16) / 1e9, "unit": "G weights/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"first {rows} rows ({n} weights) of the same layer: torch CPU scatter decode {dec:.3f} s + "
                  f"F.linear in bf16 {mm16 * 1e3:.2f} ms (in fp32: {mm32 * 1e3:.2f} ms), medians of 10 after 3 warm-ups; "
                  f"host has {os.cpu_count()} logical cores, torch uses {torch.get_num_threads()} threads",
        "fp32_matmul_variant_G_weights_per_s": n / (dec + mm32) / 1e9,
        "decode_s": dec, "matmul_bf16_s": mm16, "matmul_fp32_s": mm32,
        "oracle_c_single_core_G_weights_per_s": n / t_c / 1e9,
    }


def bench_encode(args, dev):
    """Device encoder: one step = ixh_encode_scan + ixh_encode_pack over one bf16 layer that sits in HBM, into
    buffers allocated beforehand.  Distinct weight copies (> 256 MB together) are rotated so that the first pass
    reads HBM.  Algorithmic bytes: the weight once (2 B per element) and the packed streams + table once."""
    import ctypes as C

    from ixrun_amd import _lib
    from oracle import ix_oracle as oracle

    out_f, in_f, _, recipe, *rest = WORKLOADS[args.workload]
    level_bits = rest[0] if rest else (3, 5, 8)
    weight = make_weight(out_f, in_f, recipe)
    n = out_f * in_f
    copies = args.copies or 4
    w_dev = [weight.to(dev) for _ in range(copies)]
    dp, table, counts = _lib.encode_device(w_dev[0], level_bits)
    torch.cuda.synchronize()
    L = _lib.lib()
    bits = (C.c_int32 * len(level_bits))(*level_bits)
    ws_bytes = int(L.ixh_encode_workspace_bytes(out_f, in_f, len(level_bits)))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    scale = dp.tensors[-1]
    stream = _lib.current_stream(dev)

    def scan(i):
        _lib.check(L.ixh_encode_scan(w_dev[i % copies].data_ptr(), out_f, in_f, len(level_bits), bits, scale.data_ptr(),
                                     table.data_ptr(), ws.data_ptr(), ws_bytes, stream))

    def pack(i):
        _lib.check(L.ixh_encode_pack(w_dev[i % copies].data_ptr(), C.byref(dp.struct), table.data_ptr(), stream))

    for i in range(args.warmup):
        scan(i), pack(i)
    torch.cuda.synchronize()
    steps = args.steps
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    t_wall = time.perf_counter()
    for i in range(steps):
        ev[i][0].record(); scan(i); ev[i][1].record(); pack(i); ev[i][2].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t_wall) * 1e3
    t_scan = np.array([e[0].elapsed_time(e[1]) for e in ev])
    t_pack = np.array([e[1].elapsed_time(e[2]) for e in ev])
    ms = float(ev[0][0].elapsed_time(ev[-1][2]) / steps)
    packed_bytes = 2 + sum(t.numel() * t.element_size() for t in dp.tensors[:-1])
    alg_bytes = 2 * n + packed_bytes + table.numel() * 4
    # what the three passes really move: the weight three times, the streams cleared and written
    moved = 3 * 2 * n + 2 * packed_bytes + 3 * table.numel() * 4

    # CPU beside it: the oracle's C encoder (quantise + encode, one core) and the package's torch writer on a
    # bounded sample of the same weight
    rows = 640
    sub = weight[:rows].contiguous()
    wb = sub.view(torch.int16).numpy().view(np.uint16)
    t0 = time.perf_counter()
    sb, q = oracle.quantize_bf16(wb)
    oracle.encode(q, level_bits)
    t_c = time.perf_counter() - t0
    from ixrun_amd.quantize import int8x_quantize

    t0 = time.perf_counter()
    int8x_quantize(sub, level_bits)
    t_torch = time.perf_counter() - t0
    out = {
        "metric": "device INT8-X encode, G weights/s (bf16 layer in HBM -> packed streams + rank table)",
        "value": n / (ms * 1e-3) / 1e9, "unit": "G weights/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 in, fp32 divide, int8 / bit streams out", "data": "synthetic",
        "config": {"workload": args.workload, "out_f": out_f, "in_f": in_f, "level_bits": list(level_bits),
                   "weights": recipe, "level_fractions": [c / n for c in counts], "packed_bytes": packed_bytes,
                   "distinct_copies": copies},
        "us": {"scan_median": float(np.median(t_scan) * 1e3), "pack_median": float(np.median(t_pack) * 1e3)},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": alg_bytes / (ms * 1e-3) / HBM_PEAK, "traffic": measured_traffic(args.workload),
                     "note": f"algorithmic bytes = weight read once + packed output + table; the three passes move "
                             f"about {moved / 1e6:.0f} MB ({moved / (ms * 1e-3) / 1e9:.0f} GB/s)"},
        "host_wall_ms_per_step": wall_ms / steps,
        "cpu_baseline": {"value": sub.numel() / t_torch / 1e9, "unit": "G weights/s", "cores": torch.get_num_threads(),
                         "kind": "port", "sample": f"first {rows} rows of the same weight through the torch CPU writer "
                         f"({t_torch:.2f} s); the oracle's C encoder on one core: {sub.numel() / t_c / 1e9:.3f} G weights/s"},
    }
    print(json.dumps(out))


def bench_decode(args, dev):
    """Full decode: one step = one ixh_decode (or ixh_decode_gs) launch over one packed layer into a bf16 buffer.
    Distinct packed copies are rotated as in the headline workload.  Algorithmic bytes: packed streams (+ group
    scales) read, 2 bytes per weight written."""
    from ixrun_amd import _lib
    from oracle import ix_oracle as oracle

    out_f, in_f, _, recipe, *rest = WORKLOADS[args.workload]
    weight = make_weight(out_f, in_f, recipe)
    n = out_f * in_f
    grouped = args.workload.startswith("decode_gs_")
    if grouped:
        from ixrun_amd import ixgs

        packed = ixgs.int8gs_quantize(weight)
        packed_bytes = packed["total_bytes"]
        mk = lambda: (_lib.DevicePacked((3, 5, 8), out_f, in_f, [packed["b1"].to(dev), packed["b2"].to(dev)],
                                        [packed["l1"].to(dev), packed["l2"].to(dev), packed["l3"].to(dev)], None),
                      packed["group_scales"].to(dev))
    else:
        from ixrun_amd.quantize import int8x_quantize

        level_bits = tuple(rest[0]) if rest else (3, 5, 8)
        packed = int8x_quantize(weight, level_bits)
        packed_bytes = packed["total_bytes"]
        mk = lambda: (_lib.DevicePacked.from_dict(packed, dev), None)
    copies = args.copies or max(2, -(-600_000_000 // packed_bytes))
    layers = [mk() for _ in range(copies)]
    tables = [dp.prefix_build(512) for dp, _ in layers]
    out = torch.empty(n, dtype=torch.bfloat16, device=dev)

    def step(i):
        dp, scales = layers[i % copies]
        if grouped:
            dp.decode_gs(tables[i % copies], 512, scales, packed["group_size"], out)
        else:
            dp.decode(tables[i % copies], 512, out_bf16=out)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    steps = args.steps
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        step(i)
    stop.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(stop) / steps
    alg_bytes = packed_bytes + 2 * n
    # CPU beside it: the oracle's C walk (decode + dequantise) on the first rows, one core
    rows = 640
    if grouped:
        scales, q = oracle.gs_quantize(weight[:rows].contiguous().view(torch.int16).numpy().view(np.uint16), 64)
        e = oracle.gs_encode(q)
        t0 = time.perf_counter()
        oracle.gs_dequant_bf16(oracle.gs_decode_i16(q.size, e["b1"], e["b2"], e["l1"], e["l2"], e["l3"]), scales, 64)
        t_c = time.perf_counter() - t0
        level_fractions = [c / n for c in packed["counts"]]
    else:
        from ixrun_amd.quantize import int8x_quantize

        sub = int8x_quantize(weight[:rows].contiguous(), level_bits)
        t0 = time.perf_counter()
        oracle.decode_packed_bf16(sub)
        t_c = time.perf_counter() - t0
        level_fractions = [c / n for c in packed["counts"]]
    print(json.dumps({
        "metric": "full decode to bf16, G weights/s", "value": n / (ms * 1e-3) / 1e9, "unit": "G weights/s", "n_gpus": 1,
        "steps": steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8 codes x bf16/fp16 scale -> bf16", "data": "synthetic",
        "config": {"workload": args.workload, "out_f": out_f, "in_f": in_f, "weights": recipe,
                   "level_fractions": level_fractions, "packed_bytes": packed_bytes, "distinct_copies": copies},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": alg_bytes / (ms * 1e-3) / HBM_PEAK, "traffic": measured_traffic(args.workload),
                     "note": "algorithmic bytes = packed layer read + 2 bytes per weight written"},
        "cpu_baseline": {"value": rows * in_f / t_c / 1e9, "unit": "G weights/s", "cores": 1, "kind": "port",
                         "sample": f"first {rows} rows through the oracle's C decoder ({t_c:.2f} s)"},
    }))


def kernel_sources_sha16(files=None):
    """sha256 (first 16 hex digits) over kernel sources of the library (all of them, or the named ones):
    counter-derived figures are only reported for the sources they were measured on."""
    import hashlib

    h = hashlib.sha256()
    src = os.path.join(ROOT, "ixrun_amd", "csrc")
    names = sorted(files) if files is not None else sorted(n for n in os.listdir(src) if n.endswith((".hip", ".h")))
    for name in names:
        h.update(name.encode())
        h.update(open(os.path.join(src, name), "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(workload):
    """HBM bytes per launch from the committed counter runs, or None when the kernel's sources have changed since."""
    hit = MEASURED_TRAFFIC_BYTES.get(workload)
    if hit is None:
        return None
    nbytes, files, sha16 = hit
    return nbytes if files and sha16 == kernel_sources_sha16(files) else None


def measured_instructions(workload, n_weights):
    """Vector / scalar / LDS instructions per weight from the committed counter run (None when the kernel's sources
    have changed since)."""
    hit = MEASURED_INSTRUCTIONS.get(workload)
    if hit is None:
        return {"valu_per_weight": None, "salu_per_weight": None, "lds_per_weight": None}
    (valu, salu, lds), files, sha16 = hit
    if not files or sha16 != kernel_sources_sha16(files):
        return {"valu_per_weight": None, "salu_per_weight": None, "lds_per_weight": None}
    return {"valu_per_weight": round(valu * 64.0 / n_weights, 3), "salu_per_weight": round(salu / n_weights, 4),
            "lds_per_weight": round(lds * 64.0 / n_weights, 3)}


def build_layers(workload, dev, copies=0, unfused=False):
    """The packed layer of a workload (CPU generator, CPU writer: the literal recipe), `copies` device copies of it
    as StreamingLinear modules, and its activations."""
    from ixrun_amd.engine import StreamingLinear
    from ixrun_amd.quantize import int8x_quantize

    out_f, in_f, m, recipe, *rest = WORKLOADS[workload]
    level_bits = rest[0] if rest else (3, 5, 8)
    weight = make_weight(out_f, in_f, recipe)
    packed = int8x_quantize(weight, level_bits)
    chained = workload.startswith("graph64")
    copies = copies or (64 if chained else max(2, -(-600_000_000 // packed["total_bytes"])))
    layers = [StreamingLinear(packed) for _ in range(copies)]
    if unfused:
        shared = torch.empty(packed["N"], dtype=torch.bfloat16, device=dev)
        for sl in layers:
            sl._gemm_ok = False
            sl._set_shared_buf(shared)
    g = torch.Generator("cpu").manual_seed(1)
    x_host = torch.randn(m, in_f, generator=g).bfloat16()
    return weight, packed, layers, x_host, chained


def time_layers(layers, x, chained, steps_requested, warmup, min_seconds, eager=False):
    """Time steps over the layers (round-robin; chained: each output feeds the next layer).  One pass over all
    copies is captured as a hipGraph and replayed back to back; the timed region covers at least `steps_requested`
    steps and at least `min_seconds` (a region of a few hundred microseconds ends before the clocks have settled
    and reads several per cent slow).  Returns (ms per step, steps timed, graph or None, step function)."""
    copies = len(layers)
    state = {"h": x}

    def step(i):
        if not chained:
            return layers[i % copies](x)
        if i % copies == 0:
            state["h"] = x
        state["h"] = layers[i % copies](state["h"])  # the layer's output is the next layer's input
        return state["h"]

    for i in range(max(warmup, 1)):
        step(i)
    torch.cuda.synchronize()
    graph = None
    if not eager:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(copies):
                step(i)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            outs = [step(i) for i in range(copies)]  # noqa: F841  (kept alive by the graph's pool)

    def run(n_steps):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        if graph is not None:
            for _ in range(n_steps // copies):
                graph.replay()
        else:
            for i in range(n_steps):
                step(i)
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop)

    unit = copies if graph is not None else 1
    steps = max(unit, -(-steps_requested // unit) * unit)
    # warm-up the way the timed steps run (back to back, no host gaps), and a first estimate of the step time
    probe = max(unit, -(-max(warmup, 1) // unit) * unit)
    est_ms = run(probe) / probe
    est_ms = min(est_ms, run(probe) / probe)
    if est_ms * steps < min_seconds * 1e3:
        steps = -(-int(min_seconds * 1e3 / max(est_ms, 1e-6)) // unit) * unit
    ms = run(steps)
    while ms < min_seconds * 1e3 * 0.999:  # the estimate was slow (clocks still rising): lengthen and time again
        steps = -(-int(steps * 1.1 * min_seconds * 1e3 / max(ms, 1e-6)) // unit) * unit
        ms = run(steps)
    return ms / steps, steps, graph, step


def also_block(dev, args):
    """The other shapes of the hot path, each timed for a few hundred milliseconds with the headline's harness
    (distinct packed copies beyond the last-level cache, hipGraph replay): us per layer, G weights/s and the
    fraction of the roofline on algorithmic bytes (HBM; bf16 MFMA flops for the many-row workload)."""
    import gc

    from ixrun_amd import gemm_tuning
    from ixrun_amd.fused import fused_gemv

    # (workload that names the layer, [(reported name, activation rows, variant)])
    plan = [
        ("down_proj_5120x17408_m1_calibrated", [("down_proj_5120x17408_m1_calibrated", 1, "fused"),
                                                ("down_proj_5120x17408_m8_calibrated", 8, "fused")]),
        ("down_proj_5120x17408_m1_reference_recipe", [("down_proj_5120x17408_m1_reference_recipe", 1, "fused")]),
        ("down_proj_5120x17408_m1_five_level_calibrated", [("down_proj_5120x17408_m1_five_level_calibrated", 1, "fused")]),
        ("down_proj_5120x17408_m1_student_t", [("down_proj_5120x17408_m1_student_t_split_k_call", 1, "split_k"),
                                               ("down_proj_5120x17408_m1_student_t_split_k_kernel_alone", 1, "split_k_bare")]
                                              + [(f"down_proj_5120x17408_m{m}_student_t", m, "fused") for m in (4, 8, 16)]),
        ("attn_proj_5120x5120_m1_student_t", [("attn_proj_5120x5120_m1_student_t", 1, "fused")]
                                             + [(f"attn_proj_5120x5120_m{m}_student_t", m, "fused") for m in (4, 8, 16)]),
        ("gate_up_17408x5120_m2_student_t", [(f"gate_up_17408x5120_m{m}_student_t", m, "fused") for m in (1, 2, 4, 8, 16)]),
        ("graph64_5120x5120_m1_student_t", [("graph64_5120x5120_m1_student_t", 1, "fused")]),
        ("prefill_5120x17408_m512_five_level", [("prefill_5120x17408_m512_five_level", 512, "fused"),
                                                ("prefill_5120x17408_m512_five_level", 512, "unfused")]),
    ]
    out = {}
    for key, runs in plan:
        t0 = time.perf_counter()
        out_f, in_f = WORKLOADS[key][:2]
        chained = key.startswith("graph64")
        _, packed, layers, _, _ = build_layers(key, dev)
        for name, m, variant in runs:
            g = torch.Generator("cpu").manual_seed(1)
            x = torch.randn(m, in_f, generator=g).bfloat16().to(dev)
            runners = layers
            if variant == "unfused":  # decode to a bf16 buffer + library GEMM chosen by measurement: what the engine runs
                shared_w = torch.empty(packed["N"], dtype=torch.bfloat16, device=dev)
                for sl in layers:
                    sl._gemm_ok = False
                    sl._set_shared_buf(shared_w)
                gemm_tuning.enable()
            elif variant.startswith("split_k"):
                # the reference's call of this shape (ixrun/engine.py:148-159): zero the fp32 vector, fused_gemv with
                # chunk = in_f / 2 adds into it, cast to bf16 (three launches); "bare": the middle one alone
                y32 = torch.zeros(out_f, dtype=torch.float32, device=dev)
                whole = variant == "split_k"

                def make(sl):
                    def call(xin):
                        if whole:
                            y32.zero_()
                        fused_gemv(xin.reshape(-1), sl._b1, sl._b2, sl._l1, sl._l2, sl._l3, sl._q1, sl._q2, sl._scale,
                                   out_f, in_f, chunk=in_f // 2, y32=y32)
                        return y32.to(torch.bfloat16) if whole else y32
                    return call

                runners = [make(sl) for sl in layers]
            ms, steps, graph, step = time_layers(runners, x, chained, 0, 20, args.also_seconds)
            r = {"us_per_layer": round(ms * 1e3, 2), "G_weights_per_s": round(out_f * in_f / (ms * 1e-3) / 1e9, 1),
                 "steps": steps}
            if m > 16:
                flops = 2.0 * m * out_f * in_f
                r["TFLOP_per_s"] = round(flops / (ms * 1e-3) / 1e12, 1)
                r["frac_mfma"] = round(flops / (ms * 1e-3) / MFMA_BF16_PEAK, 4)
                # the same step against the HBM roofline: packed layer + activations in + outputs out
                alg_bytes = packed["total_bytes"] + m * in_f * 2 + m * out_f * 2
                r["frac_hbm"] = round(alg_bytes / (ms * 1e-3) / HBM_PEAK, 4)
                r["traffic"] = measured_traffic(name if variant == "fused" else name + "_unfused")
                out.setdefault(name, {})["ixh_gemm" if variant == "fused" else "decode_plus_tuned_library_gemm"] = r
            else:
                alg_bytes = packed["total_bytes"] + m * in_f * 2 + m * out_f * 2
                r["frac_hbm"] = round(alg_bytes / (ms * 1e-3) / HBM_PEAK, 4)
                r["level_fractions"] = [round(c / packed["N"], 5) for c in packed["counts"]]
                r["bits_per_weight"] = round(packed["bits_per_weight"], 3)
                out[name] = r
            del graph, step, runners
            torch.cuda.synchronize()
        out[runs[-1][0]]["wall_s"] = round(time.perf_counter() - t0, 1)
        del layers
        gc.collect()
        torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the timed region is never shorter than --min-seconds, whatever --steps says: a run of a few hundred steps
    # (10 ms) ends before the clocks have settled and reads about 8 % slower on the headline layer
    ap.add_argument("--steps", type=int, default=9800)
    ap.add_argument("--warmup", type=int, default=980)
    ap.add_argument("--min-seconds", type=float, default=0.2, help="shortest timed region (0 = exactly --steps)")
    ap.add_argument("--workload", default="down_proj_5120x17408_m1_student_t", choices=list(WORKLOADS))
    ap.add_argument("--copies", type=int, default=0, help="distinct packed copies to rotate over (0 = enough for 600 MB)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-also", action="store_true", help="skip the block of other workloads timed beside the headline")
    ap.add_argument("--also-seconds", type=float, default=0.15, help="timed region of each workload of that block")
    ap.add_argument("--eager", action="store_true", help="time eager launches instead of hipGraph replays")
    ap.add_argument("--unfused", action="store_true",
                    help="many-row workloads: decode the bf16 weight to HBM and call the library GEMM instead")
    ap.add_argument("--tune-gemm", action="store_true",
                    help="with --unfused: let the library GEMM of the many-row path be chosen by measurement")
    ap.add_argument("--set-option", action="append", default=[], metavar="NAME=VALUE",
                    help="library switch for comparisons (ixh_set_option), e.g. gemv_tiles=-1 or decode_kernel=staged")
    ap.add_argument("--gemv-flags", type=int, default=0,
                    help="extra IXH_GEMV_* flags of every fused call, for comparisons (16 = the staged any-scheme kernel)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three 256 MiB device copies (known traffic) so that counter runs can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (one MI355X holds the whole layer); "
                 "run with --gpus 1")
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    dev = torch.device("cuda:0")
    for item in args.set_option:
        from ixrun_amd import _lib

        name, _, value = item.partition("=")
        _lib.set_option(name, value if name == "decode_kernel" and not value.lstrip("-").isdigit() else int(value))

    if args.workload.startswith("encode_"):
        return bench_encode(args, dev)
    if args.workload.startswith("decode_"):
        return bench_decode(args, dev)

    out_f, in_f, m, recipe, *rest = WORKLOADS[args.workload]
    level_bits = rest[0] if rest else (3, 5, 8)
    headline = args.workload == "down_proj_5120x17408_m1_student_t"
    t0 = time.perf_counter()
    weight, packed, layers, x_host, chained = build_layers(args.workload, dev, args.copies, args.unfused)
    copies = len(layers)
    prep_s = time.perf_counter() - t0
    if args.tune_gemm:
        from ixrun_amd import gemm_tuning
        gemm_tuning.enable()
    for sl in layers:
        sl._gemv_flags = args.gemv_flags
        sl._plans = {}
    x = x_host.to(dev)
    table_bytes = layers[0]._table.numel() * 4
    # algorithmic bytes of one step: the packed layer, the activations in, the outputs out
    alg_bytes = packed["total_bytes"] + m * in_f * 2 + m * out_f * 2

    if args.calibrate_copy:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    t_wall = time.perf_counter()
    ms_per_step, steps, graph, step = time_layers(layers, x, chained, args.steps, args.warmup, args.min_seconds,
                                                   eager=args.eager)
    wall_ms = (time.perf_counter() - t_wall) * 1e3

    # eager launches with an event pair around every call, for the spread and the host cost
    n_ev = min(steps, 240)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_ev)]
    for i, (a, b) in enumerate(evs):
        a.record()
        step(i)
        b.record()
    torch.cuda.synchronize()
    per_call = np.array([a.elapsed_time(b) for a, b in evs]) * 1e3  # us

    us = ms_per_step * 1e3
    weights_per_s = out_f * in_f / (ms_per_step * 1e-3)
    achieved = alg_bytes / (ms_per_step * 1e-3)
    out = {
        "metric": "fused decode+GEMV G weights/s & % HBM peak (5120x17408, batch 1); us/layer",
        "value": weights_per_s / 1e9, "unit": "G weights/s", "n_gpus": 1, "steps": steps,
        "steps_requested": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "us_per_layer": us, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16 activations x int8 codes, fp32 accumulate", "data": "synthetic",
        "config": {
            "workload": args.workload, "out_f": out_f, "in_f": in_f, "batch": m, "level_bits": list(level_bits),
            "weights": recipe, "level_fractions": [c / packed["N"] for c in packed["counts"]],
            "bits_per_weight": packed["bits_per_weight"], "packed_bytes": packed["total_bytes"],
            "rank_table_bytes": table_bytes, "distinct_copies": copies,
        },
        "roofline": {
            "bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": achieved / HBM_PEAK, "traffic": measured_traffic(args.workload),
            **measured_instructions(args.workload, out_f * in_f),
            "note": "algorithmic bytes = packed layer + x + y per launch; time = HIP-event time of the timed region / "
                    "steps; traffic = HBM bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this script; "
                    "valu / lds_per_weight = wave instructions x 64 lanes / weights, salu_per_weight = scalar "
                    "instructions / weights, from an SQ_INSTS_* run (all null when the kernel sources have changed "
                    "since those runs)",
        },
        "launch": "eager" if graph is None else f"hipGraph of {copies} layer launches, replayed {steps // copies}x",
        "timed_region": f"{steps} steps = {ms_per_step * steps:.1f} ms: at least --steps ({args.steps}) and at least "
                        f"--min-seconds ({args.min_seconds} s) of back-to-back replays",
        "eager_per_call_us": {"median": float(np.median(per_call)), "min": float(per_call.min()),
                        "p90": float(np.percentile(per_call, 90))},
        "host_wall_ms_per_step": wall_ms / steps,
        "prep_s": prep_s,
    }
    if m > 16:
        flops = 2.0 * m * out_f * in_f
        out["roofline"] = {
            "bound": "mfma", "achieved": flops / (ms_per_step * 1e-3) / 1e12, "peak": MFMA_BF16_PEAK / 1e12,
            "unit": "TFLOP/s", "frac": flops / (ms_per_step * 1e-3) / MFMA_BF16_PEAK,
            "traffic": None if args.unfused else measured_traffic(args.workload),
            "note": "2*M*N*K flops per launch pair (GEMM + slice reduce); the kernel is bound by the VALU decode "
                    "that feeds the matrix cores, not by MFMA issue",
        }
        out["path"] = "decode to HBM + library GEMM" if args.unfused else "fused decode + MFMA (ixh_gemm)"
        if args.unfused and args.tune_gemm:
            out["path"] += ", GEMM kernel chosen by measurement (torch.cuda.tunable)"
    del graph, step, layers
    import gc

    gc.collect()
    torch.cuda.empty_cache()
    if headline and not args.no_also and not args.eager:
        out["also"] = also_block(dev, args)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(weight, x_host, level_bits)
        out["cpu_baseline"]["speedup_vs_cpu"] = out["value"] / out["cpu_baseline"]["value"]
    print(json.dumps(out))


if __name__ == "__main__":
    main()
