#!/usr/bin/env python3
"""Benchmark of the int4 decode linears on one MI355X.

A "step" is one pass over the Janus-Pro-1B decoder linear set at M=1: per layer
q/k/v/o 2048->2048, gate and up 2048->5632, down 5632->2048, times 24 layers
with distinct seeded weights (168 GEMVs, 642,539,520 algorithmic bytes), all
int4 with group size 128.  Operands are resident in HBM before the timed region.

Prints one JSON line.  ``value`` is the aggregate algorithmic GB/s of the step;
``roofline`` prices the dominant kernel against the 8 TB/s HBM peak; ``cpu_baseline``
times the PyTorch dequant + matmul path on the host cores over a bounded sample;
``detail`` carries the other launch strategies, per-call latencies and the M=32
rollout-batch figure.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

HBM_PEAK_GBS = 8000.0
HIDDEN, INTER, LAYERS, GROUP, HEAD = 2048, 5632, 24, 128, 16384
ROOT = os.path.dirname(os.path.abspath(__file__))

# (name, K, N) in the order the decoder layer applies them
LAYER_LINEARS = [("q", HIDDEN, HIDDEN), ("k", HIDDEN, HIDDEN), ("v", HIDDEN, HIDDEN),
                 ("o", HIDDEN, HIDDEN), ("gate", HIDDEN, INTER), ("up", HIDDEN, INTER),
                 ("down", INTER, HIDDEN)]


def make_weights(seed: int, K: int, N: int, G: int, device):
    """Seeded synthetic packed weights, generated on the device.

    Uniform 32-bit words are eight independent uniform nibbles; scales are
    |N(0, 0.02)| as bf16 (zeros replaced), zero-point words uniform with the
    unused high nibbles of the last word cleared.
    """
    gen = torch.Generator(device=device).manual_seed(seed)
    groups = K // G
    zwords = (groups + 7) // 8
    qweight = torch.randint(-2 ** 31, 2 ** 31, (N, K // 8), generator=gen, device=device,
                            dtype=torch.int64).to(torch.int32)
    scales = (torch.randn((N, groups), generator=gen, device=device) * 0.02).abs()
    scales = torch.where(scales < 1e-6, torch.full_like(scales, 1e-3), scales).to(torch.bfloat16)
    qzeros = torch.randint(-2 ** 31, 2 ** 31, (N, zwords), generator=gen, device=device,
                           dtype=torch.int64).to(torch.int32)
    used = groups - 8 * (zwords - 1)
    if used < 8:
        keep = (1 << (4 * used)) - 1
        qzeros[:, -1] &= keep
    return qweight.contiguous(), scales.contiguous(), qzeros.contiguous()


def make_x(seed: int, M: int, K: int, device):
    gen = torch.Generator(device=device).manual_seed(seed)
    return torch.randn((M, K), generator=gen, device=device).to(torch.bfloat16).contiguous()


def time_region(fn, steps: int, warmup: int):
    """ms per call of ``fn`` over ``steps`` calls, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def time_blocks(fn, steps: int, warmup: int, blocks: int = 7, min_warm_ms: float = 200.0):
    """ms per call of ``fn``: ``blocks`` HIP-event regions of ``steps`` back-to-back calls each.

    The device is first warmed by ``warmup`` calls and then by time (at least ``min_warm_ms`` of
    calls): the clocks of an idle device take tens of milliseconds of load to settle, so a short
    fixed warm-up count measures the ramp.  Returns ``(median, sorted list of the block figures)``.
    """
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < min_warm_ms:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
    per_block = []
    for _ in range(blocks):
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(steps):
            fn()
        end.record()
        torch.cuda.synchronize()
        per_block.append(start.elapsed_time(end) / steps)
    per_block.sort()
    return per_block[len(per_block) // 2], per_block


def build_set(cfg: int, M: int, device, with_head: bool, hidden: int = HIDDEN, inter: int = INTER,
              layers: int = LAYERS, head: int = HEAD, canonical: bool = True):
    """All linears of one decode step: list of dicts with operands and byte counts.

    Activations follow the decoder layer (policy.py:673-678): q, k and v of a layer read one tensor,
    gate and up another, o_proj, down_proj and the head one each; no two layers share an input.
    """
    from visionrl_amd import ops
    from visionrl_amd.int4_format import algorithmic_bytes

    items = []
    linears = [("q", hidden, hidden), ("k", hidden, hidden), ("v", hidden, hidden), ("o", hidden, hidden),
               ("gate", hidden, inter), ("up", hidden, inter), ("down", inter, hidden)]
    shared = {"q": 0, "k": 0, "v": 0, "o": 1, "gate": 2, "up": 2, "down": 3}
    for layer in range(layers):
        xs = {}
        for proj, (name, K, N) in enumerate(linears):
            slot = shared[name]
            if slot not in xs:
                xs[slot] = make_x(1000 * cfg + 100000 + 10 * layer + slot, M, K, device)
            qw, sc, qz = make_weights(1000 * cfg + 10 * layer + proj, K, N, GROUP, device)
            it = {"name": f"l{layer}.{name}", "layer": layer, "proj": name, "K": K, "N": N, "x": xs[slot],
                  "prepacked": ops.int4_prepack(qw, sc, qz, GROUP),
                  "bytes": algorithmic_bytes(M, K, N, GROUP)}
            if canonical:
                it.update({"qweight": qw, "scales": sc, "qzeros": qz})
            items.append(it)
    if with_head:
        qw, sc, qz = make_weights(1000 * cfg + 999, hidden, head, GROUP, device)
        it = {"name": "gen_head", "layer": layers, "proj": "head", "K": hidden, "N": head,
              "x": make_x(1000 * cfg + 100999, M, hidden, device), "prepacked": ops.int4_prepack(qw, sc, qz, GROUP),
              "bytes": algorithmic_bytes(M, hidden, head, GROUP)}
        if canonical:
            it.update({"qweight": qw, "scales": sc, "qzeros": qz})
        items.append(it)
    return items


def check_outputs(items, outputs, what: str, tolerance_counts: dict | None = None):
    """Every output of a timed launch against a float64 product over the bit-exact dequantised weights,
    computed on the device by the library's dequant kernel and a torch matmul.  Raises on a miss: a
    throughput figure of a launch with wrong results is worth nothing.

    Bound per element: max(1 bf16 ulp, 1e-2 |y_ref|) where |y_ref| >= 2^-6 sum|x w|, with 2^-18 sum|x w|
    of fp32 reassociation noise allowed on top below that.
    """
    from visionrl_amd import ops

    worst = 0.0
    counts = {"outputs": 0, "cancelled_below_2^-6_sum_abs": 0, "beyond_strict_bound": 0}
    for it, y in zip(items, outputs):
        if "qweight" in it:
            w = ops.int4_dequant(it["qweight"], it["scales"], it["qzeros"], GROUP).double()
        else:
            continue
        x = it["x"].double()
        ref = x @ w.t()
        aref = x.abs() @ w.abs().t()
        got = y.double()
        # one bf16 step at |ref|: 2^(floor(log2|ref|) - 7), never below the smallest normal's
        ulp = torch.exp2(torch.floor(torch.log2(ref.abs().clamp_min(2.0 ** -126))) - 7)
        tol = torch.maximum(ulp, 1e-2 * ref.abs())
        tol = torch.where(ref.abs() >= 2.0 ** -6 * aref, tol, tol + 2.0 ** -18 * aref)
        err = (got - ref).abs()
        if not bool((err <= tol).all()):
            bad = int((err > tol).sum())
            raise RuntimeError(f"{what}: {it['name']} has {bad} of {err.numel()} outputs out of tolerance "
                               f"(worst error {float((err - tol).max()):.3e} beyond the bound)")
        worst = max(worst, float((err / aref.clamp_min(1e-300)).max()))
        counts["outputs"] += err.numel()
        counts["cancelled_below_2^-6_sum_abs"] += int((ref.abs() < 2.0 ** -6 * aref).sum())
        counts["beyond_strict_bound"] += int((err > torch.maximum(ulp, 1e-2 * ref.abs())).sum())
    if tolerance_counts is not None:
        # how many outputs passed only on the extra term (all of them cancelled ones: the rest were held to the
        # strict bound above)
        tolerance_counts.update(counts)
    return worst


def measure_set(items, steps: int, warmup: int):
    """Time one decode step's linear set under each launch strategy."""
    from visionrl_amd import ops

    total_bytes = sum(it["bytes"] for it in items)
    out = {"launches_per_step": {}, "ms_per_step": {}, "GBps": {}}

    def record(name, ms, launches):
        out["ms_per_step"][name] = ms
        out["GBps"][name] = total_bytes / (ms * 1e-3) / 1e9
        out["launches_per_step"][name] = launches

    # one launch for the whole set, weights in the prepacked (MFMA-shaped) layout
    grouped = ops.GroupedGemv([(it["x"], it["prepacked"], False) for it in items])
    ms, per_block = time_blocks(grouped.launch, steps, warmup)
    record("grouped_1_launch", ms, 1)
    out["grouped_1_launch_blocks_ms"] = per_block
    # the launch that was just timed, every output of every record
    out["grouped_1_launch_tolerance_counts"] = {}
    out["grouped_1_launch_worst_backward_error"] = check_outputs(items, grouped.outputs, "grouped launch",
                                                                 out["grouped_1_launch_tolerance_counts"])

    # the comparison build whose dot product runs on the vector unit (v_dot2_f32_bf16) instead of the matrix
    # cores: same blob, same dequantisation, same stream (one activation row only)
    if all(it["x"].shape[0] == 1 for it in items):
        vdot = ValuDotLaunch([(it["x"], it["prepacked"], False) for it in items])
        ms_v, blocks_v = time_blocks(vdot.launch, steps, warmup, blocks=5, min_warm_ms=100.0)
        record("grouped_1_launch_valu_dot", ms_v, 1)
        out["grouped_1_launch_valu_dot_blocks_ms"] = blocks_v
        check_outputs(items, vdot.outputs, "grouped launch, vector-unit dot product")
        del vdot

    # the same launch over the canonical layout (no load-time repack)
    canon = ops.GroupedGemv([(it["x"], it["qweight"], it["scales"], it["qzeros"], GROUP, False)
                             for it in items])
    record("grouped_1_launch_canonical_layout", time_region(canon.launch, steps, warmup), 1)
    del canon

    # one launch per linear, stream ordered
    def eager():
        for it in items:
            ops.int4_gemv(it["x"], it["qweight"], it["scales"], it["qzeros"], GROUP)

    record("per_linear_eager", time_region(eager, max(3, steps // 20), max(1, warmup // 20)), len(items))

    # the same launches replayed from a HIP graph
    try:
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            eager()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            eager()
        record("per_linear_hip_graph", time_region(graph.replay, max(5, steps // 5), max(2, warmup // 5)), len(items))
    except Exception as exc:  # graph capture is an extra, never the headline
        out["hip_graph_error"] = repr(exc)[:200]

    # launches a real decoder layer could issue: q|k|v together, o, gate|up together, down
    by_layer = {}
    for it in items:
        by_layer.setdefault(it["layer"], []).append(it)
    plans = []
    for layer in sorted(by_layer):
        its = {it["proj"]: it for it in by_layer[layer]}
        for names in (("q", "k", "v"), ("o",), ("gate", "up"), ("down",), ("head",)):
            sel = [its[n] for n in names if n in its]
            if sel:
                probs = [(it["x"], it["prepacked"], False) for it in sel]
                direct = all(it["x"].shape[0] <= ops.DirectGemv.MAX_ROWS for it in sel)
                plans.append(ops.DirectGemv(probs) if direct else ops.GroupedGemv(probs))

    def layered():
        for plan in plans:
            plan.launch()

    record("per_layer_4_launches", time_region(layered, max(5, steps // 5), max(2, warmup // 5)), len(plans))
    try:
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            layered()
        record("per_layer_4_launches_hip_graph",
               time_region(graph.replay, max(5, steps // 5), max(2, warmup // 5)), len(plans))
    except Exception as exc:
        out["layered_hip_graph_error"] = repr(exc)[:200]
    return out, total_bytes, grouped


def fused_gate_up_launch(device, steps: int, warmup: int):
    """Configuration 5a: fused gate||up with the SiLU epilogue, K=4096, N=2x11008, M=8, one grouped launch over 24
    distinct weight sets (1.1 GB: beyond the memory-side cache); the outputs are compared with the unfused
    float64 product afterwards."""
    from visionrl_amd import ops
    from visionrl_amd.int4_format import algorithmic_bytes

    K, I, M = 4096, 11008, 8
    sets, canon = [], []
    for i in range(24):
        qw, sc, qz = make_weights(5000 + i, K, 2 * I, GROUP, device)
        sets.append(ops.int4_prepack(qw, sc, qz, GROUP))
        if i < 2:
            canon.append((qw, sc, qz))
        del qw, sc, qz
    x = make_x(5007, M, K, device)
    nbytes = 24 * algorithmic_bytes(M, K, 2 * I, GROUP, fused_gate_up=True)
    grouped = ops.GroupedGemv([(x, pw, True) for pw in sets])
    ms, blocks = time_blocks(grouped.launch, steps, warmup, blocks=5, min_warm_ms=50.0)
    worst = 0.0
    for (qw, sc, qz), y in zip(canon, grouped.outputs):   # silu(gate) * up in float64 over the bit-exact weights
        w = ops.int4_dequant(qw, sc, qz, GROUP).double()
        acc, mag = x.double() @ w.t(), x.double().abs() @ w.abs().t()
        gate, up = acc[:, :I], acc[:, I:]
        ref = torch.nn.functional.silu(gate) * up
        err = (y.double() - ref).abs()
        # one bf16 rounding of the product, and the fp32 accumulation noise of either factor carried through
        # (the slope of SiLU stays below 1.1)
        tol = 2.0 ** -7 * ref.abs() + 2.0 ** -17 * (1.1 * mag[:, :I] * up.abs() +
                                                     torch.nn.functional.silu(gate).abs() * mag[:, I:])
        if not bool((err <= tol + 1e-30).all()):
            raise RuntimeError("fused gate||up launch: outputs out of tolerance")
        worst = max(worst, float((err / ref.abs().clamp_min(1e-6)).median()))
    return {"ms_per_24_weight_sets": ms, "us_per_weight_set": ms * 1e3 / 24, "GBps": nbytes / (ms * 1e-3) / 1e9,
            "pct_hbm_peak": 100.0 * nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "blocks_ms": blocks,
            "algorithmic_bytes_per_launch": nbytes, "median_relative_error_of_checked_outputs": worst}


def other_configs(device, steps: int, warmup: int):
    """The remaining benchmark configurations, one grouped launch each (prepacked layout)."""
    from visionrl_amd import ops
    from visionrl_amd.int4_format import algorithmic_bytes

    res = {}
    # 7B-class shapes: hidden 4096, intermediate 11008, 30 layers, head 4096 -> 16384
    for M in (1, 8, 16):
        items = build_set(4, M, device, with_head=True, hidden=4096, inter=11008, layers=30, head=16384)
        nbytes = sum(it["bytes"] for it in items)
        grouped = ops.GroupedGemv([(it["x"], it["prepacked"], False) for it in items])
        ms, per_block = time_blocks(grouped.launch, max(10, steps // 10), max(2, warmup // 10), blocks=5,
                                    min_warm_ms=100.0)
        counts = {}
        res[f"7b_class_m{M}"] = {"ms_per_step": ms, "GBps": nbytes / (ms * 1e-3) / 1e9,
                                 "pct_hbm_peak": 100.0 * nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                 "blocks_ms": per_block, "algorithmic_bytes_per_step": nbytes, "gemvs": len(items),
                                 "worst_backward_error": check_outputs(items, grouped.outputs, f"7B-class set, M={M}",
                                                                       counts),
                                 "tolerance_counts": counts,
                                 # HBM bytes per launch by rocprofv3 FETCH_SIZE + WRITE_SIZE runs of this launch
                                 # (profiles/gemv_stream_kernel_7b_class_m1_m8_m16.txt), not measured in this run
                                 "traffic": load_traffic(f"gemv_stream_kernel_7b_m{M}")}
        del items, grouped
        torch.cuda.empty_cache()
    res["fused_gate_up_silu_k4096_i11008_m8"] = fused_gate_up_launch(device, max(10, steps // 10), max(2, warmup // 10))
    # profiles/gemv_stream_kernel_fused_gate_up_k4096_i11008_m8.txt
    res["fused_gate_up_silu_k4096_i11008_m8"]["traffic"] = load_traffic("gemv_stream_kernel_5a")
    torch.cuda.empty_cache()
    # group-size sweep, K=5632, N=2048, M=1: single launches over 48 distinct weight sets in a HIP graph
    sweep = {}
    for G in (32, 64, 128):
        K, N = 5632, 2048
        ws = [make_weights(5100 + i, K, N, G, device) for i in range(48)]
        x = make_x(5107, 1, K, device)
        ys = [torch.empty((1, N), dtype=torch.bfloat16, device=device) for _ in ws]
        direct = [ops.DirectGemv([(x, ops.int4_prepack(qw, sc, qz, G), False)]) for qw, sc, qz in ws]

        def rotate():
            for (qw, sc, qz), y in zip(ws, ys):
                ops.int4_gemv_into(y, x, qw, sc, qz, G)

        def rotate_direct():
            for launch in direct:
                launch.launch()

        entry = {"distinct_weights": len(ws),
                 "pool_bytes_canonical": sum(t.numel() * t.element_size() for w in ws for t in w)}
        for name, fn in (("canonical", rotate), ("prepacked", rotate_direct)):
            fn()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                fn()
            ms = time_region(graph.replay, max(5, steps // 20), 2) / len(ws)
            entry[f"us_per_call_{name}_hip_graph"] = ms * 1e3
            entry[f"GBps_{name}"] = algorithmic_bytes(1, K, N, G) / (ms * 1e-3) / 1e9
            del graph
        sweep[f"G{G}"] = entry
        del ws, ys, direct
        torch.cuda.empty_cache()
    res["group_size_sweep_k5632_n2048_m1"] = sweep
    return res


POOL_MIN_BYTES = 280 * 1024 * 1024   # a rotating pool of weights must exceed the 256 MB memory-side cache


def per_call_latency(items, steps: int):
    """us per single-GEMV launch for each distinct shape, rotating over the distinct weights."""
    from visionrl_amd import ops

    res = {}
    shapes = {}
    for it in items:
        shapes.setdefault((it["K"], it["N"]), []).append(it)
    for (K, N), group in shapes.items():
        # the pool a call rotates over is larger than the 256 MB memory-side cache in either layout, so that
        # every call streams its weights from HBM: further distinct weight sets are made up to that size
        group = list(group)
        canon_bytes = lambda it: sum(it[k].numel() * it[k].element_size() for k in ("qweight", "scales", "qzeros"))
        extra = 0
        while min(sum(canon_bytes(it) for it in group), sum(it["prepacked"].blob.numel() for it in group)) \
                <= POOL_MIN_BYTES:
            qw, sc, qz = make_weights(777000 + 1000 * extra + K % 997, K, N, GROUP, group[0]["x"].device)
            group.append({"K": K, "N": N, "x": group[extra % len(group)]["x"], "qweight": qw, "scales": sc, "qzeros": qz,
                          "prepacked": ops.int4_prepack(qw, sc, qz, GROUP), "bytes": group[0]["bytes"]})
            extra += 1
        outs = [torch.empty((it["x"].shape[0], N), dtype=torch.bfloat16, device=it["x"].device)
                for it in group]

        def rotate_op():
            for it in group:
                ops.int4_gemv(it["x"], it["qweight"], it["scales"], it["qzeros"], GROUP)

        def rotate_direct():
            for it, y in zip(group, outs):
                ops.int4_gemv_into(y, it["x"], it["qweight"], it["scales"], it["qzeros"], GROUP)

        graph = torch.cuda.CUDAGraph()
        rotate_direct()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            rotate_direct()
        # the same matrices through the plan-free launch over the prepacked layout (records as
        # kernel arguments, waves of a workgroup split K), replayed from a HIP graph
        plans = [ops.DirectGemv([(it["x"], it["prepacked"], False)]) for it in group]

        def rotate_plans():
            for plan in plans:
                plan.launch()

        graph_p = torch.cuda.CUDAGraph()
        rotate_plans()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph_p):
            rotate_plans()
        ms_plan = time_region(graph_p.replay, max(5, steps // 10), 2) / len(group)
        reps = max(2, steps // 50)
        ms_op = time_region(rotate_op, reps, 1) / len(group)
        ms_direct = time_region(rotate_direct, reps, 1) / len(group)
        ms_graph = time_region(graph.replay, max(5, steps // 10), 2) / len(group)
        res[f"{K}x{N}"] = {"us_per_call_torch_op": ms_op * 1e3,
                           "us_per_call_direct": ms_direct * 1e3,
                           "us_per_call_hip_graph": ms_graph * 1e3,
                           "us_per_call_prepacked_hip_graph": ms_plan * 1e3,
                           "GBps_hip_graph": group[0]["bytes"] / (min(ms_graph, ms_plan) * 1e-3) / 1e9,
                           "distinct_weights": len(group),
                           "pool_bytes_canonical": sum(canon_bytes(it) for it in group),
                           "pool_bytes_prepacked": sum(it["prepacked"].blob.numel() for it in group)}
        del group, outs, plans, graph, graph_p
        torch.cuda.empty_cache()
    return res


def module_path(items, steps: int):
    """The drop-in modules as a decode step calls them: q, k, v, o, gate||up, down per layer, M=1."""
    from visionrl_amd.linear import Int4GateUpSiLU, Int4Linear

    layers = {}
    for it in items:
        if it["proj"] != "head":
            layers.setdefault(it["layer"], {})[it["proj"]] = Int4Linear.from_packed(
                it["qweight"], it["scales"], it["qzeros"], GROUP)
    x_h = items[0]["x"].reshape(1, 1, HIDDEN)
    out = {}
    for mode in ("canonical", "prepacked", "prepacked_qkv_grouped"):
        stack = []
        for mods in layers.values():
            q, k, v, o = mods["q"], mods["k"], mods["v"], mods["o"]
            gate_up, down = Int4GateUpSiLU(mods["gate"], mods["up"]), mods["down"]
            for m in (q, k, v, o, gate_up, down):
                m._packed = None
                m._group = None
                if mode != "canonical":
                    m.prepack_()
            if mode == "prepacked_qkv_grouped":
                q.group_with(k, v)
            stack.append((q, k, v, o, gate_up, down))

        def step():
            for q, k, v, o, gate_up, down in stack:
                q(x_h), k(x_h), v(x_h)
                o(x_h)
                down(gate_up(x_h))

        with torch.no_grad():
            eager_ms = time_region(step, max(3, steps // 50), 1)
            graph = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph):
                step()
            graph_ms = time_region(graph.replay, max(5, steps // 10), 2)
        out[mode] = {"eager_ms_per_step": eager_ms, "hip_graph_ms_per_step": graph_ms,
                     "launches_per_step": len(stack) * (4 if mode == "prepacked_qkv_grouped" else 6)}
        del graph, stack
        torch.cuda.empty_cache()
    return out


def prompt_pass_linears(device, steps: int):
    """The linears of the prompt pass (vrl/models/families/janus_pro/policy.py:523, iteration 0: 2B x 256 rows)
    through the int4 modules: every module dequantises its weight (bit-exact tile) and calls the library GEMM;
    with ``keep_dense_()`` the bf16 tile is kept between calls.  Four layers' modules, milliseconds per
    24-layer pass (the measured four scaled by six), at 2 x 256 and 32 x 256 rows."""
    from visionrl_amd.linear import Int4GateUpSiLU, Int4Linear

    layers = []
    for layer in range(4):
        mods = {}
        for proj, (K, N) in (("q", (HIDDEN, HIDDEN)), ("k", (HIDDEN, HIDDEN)), ("v", (HIDDEN, HIDDEN)),
                             ("o", (HIDDEN, HIDDEN)), ("gate", (HIDDEN, INTER)), ("up", (HIDDEN, INTER)),
                             ("down", (INTER, HIDDEN))):
            qw, sc, qz = make_weights(8000 + 10 * layer + len(mods), K, N, GROUP, device)
            mods[proj] = Int4Linear.from_packed(qw, sc, qz, GROUP)
        layers.append((mods["q"], mods["k"], mods["v"], mods["o"], Int4GateUpSiLU(mods["gate"], mods["up"]), mods["down"]))
    out = {}
    for rows in (512, 8192):
        x = make_x(8100, rows, HIDDEN, device)
        entry = {}
        for keep in (False, True):
            for mods in layers:
                for m in mods:
                    m.keep_dense_(keep)

            def run():
                for q, k, v, o, gate_up, down in layers:
                    q(x), k(x), v(x)
                    o(x)
                    down(gate_up(x))

            with torch.no_grad():
                ms = time_region(run, max(5, steps // 40), 2)
            entry["kept_dense_ms" if keep else "dequant_per_call_ms"] = ms * LAYERS / len(layers)
        out[f"rows{rows}"] = entry
    return out


def decode_tail(device, steps: int):
    """CFG + softmax + draw + log-probability over [2B, 16384] logits: fused launch vs the tensor ops."""
    import torch.nn.functional as F
    from visionrl_amd import ops

    out = {}
    for B in (1, 16):
        gen = torch.Generator(device=device).manual_seed(6000 + B)
        logits = (torch.randn((2 * B, HEAD), generator=gen, device=device) * 3).to(torch.bfloat16)
        w, T = 5.0, 1.0

        def torch_ops():
            cond, uncond = logits.chunk(2, dim=0)
            guided = uncond + w * (cond - uncond)
            probs = F.softmax(guided / T, dim=-1)
            sampled = torch.multinomial(probs, num_samples=1).squeeze(-1)
            lp = F.log_softmax(cond / T, dim=-1).gather(-1, sampled.unsqueeze(-1)).squeeze(-1)
            return sampled, lp

        def fused():
            return ops.cfg_sample(logits, w, T)

        # per call from a graph of 16 calls: a graph of one call is dominated by what launching a graph
        # costs (about 10 us), which a decode step pays once for all of its launches
        calls = 16
        entry = {"calls_per_graph": calls}
        for name, fn in (("torch_ops", torch_ops), ("fused", fused)):
            entry[f"{name}_eager_us"] = time_region(fn, max(20, steps // 5), 5) * 1e3
            graph = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph):
                for _ in range(calls):
                    fn()
            entry[f"{name}_hip_graph_us"] = time_region(graph.replay, max(20, steps // 5), 5) / calls * 1e3
            del graph
        out[f"B{B}"] = entry
    return out


def decode_head_and_tail(device, steps: int, heads: int = 16):
    """The image-token head (2048 -> 16384, int4) and the sampling tail per decode step: the plan-free head launch
    followed by the tail launch, against the one call that does both (vrl_int4_head_sample_bf16).  One HIP graph
    per form holds ``heads`` calls, each over a head of its own (16 x 18.6 MB: the weights do not stay in the
    L2 caches between calls); microseconds per call."""
    from visionrl_amd import ops

    packed = []
    for i in range(heads):
        qw, sc, qz = make_weights(7000 + i, HIDDEN, HEAD, 128, device)
        packed.append(ops.int4_prepack(qw, sc, qz, 128))
        del qw, sc, qz
    out = {"heads": heads, "shape": f"{HIDDEN}->{HEAD}, G=128"}
    for B in (1, 4, 16):
        x = (make_x(7100 + B, 2 * B, HIDDEN, device).float() * 0.5).to(torch.bfloat16)
        noise = torch.empty((B, HEAD), dtype=torch.bfloat16, device=device).exponential_(1.0)
        ws = ops.head_sample_workspace(B, HEAD, device)
        res = (torch.empty(B, dtype=torch.int64, device=device), torch.empty(B, dtype=torch.float32, device=device))
        launches = [ops.DirectGemv([(x, pw, False)]) for pw in packed]

        def one_call():
            for pw in packed:
                ops.head_sample(x, pw, 5.0, 1.0, noise=noise, workspace=ws, out=res)

        def head_then_tail():
            for launch in launches:
                (logits,) = launch.launch()
                ops.cfg_sample(logits, 5.0, 1.0, noise=noise)

        def head_only():
            for launch in launches:
                launch.launch()

        entry = {}
        for name, fn in (("one_call", one_call), ("head_then_tail", head_then_tail), ("head_only", head_only)):
            fn()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                fn()
            entry[f"{name}_us"] = time_region(graph.replay, max(20, steps // 5), 5) / heads * 1e3
            del graph
        out[f"B{B}"] = entry
    return out


def ar_decode_loop(device, tokens: int = 48, only: str | None = None, batches=(1, 16), prompt: int = 304,
                   shape=(HIDDEN, INTER, LAYERS, 16)):
    """ms per decode step of the image-token loop on a Janus-Pro-1B shaped policy (random weights) after a
    context of ``prompt`` tokens (304 by default, then 48 generated tokens: where a generation over a
    256-slot prompt starts; its middle is at 544 slots, its end at 832).

    ``reference_style`` is the loop of vrl/models/families/janus_pro/policy.py:624-731 with the trunk's
    dynamic cache and the torch formulas for the tail, without its per-row cache copies and host
    read-backs (so a lower bound for the reference); ``static_*`` is visionrl_amd.ar_decode over the
    trunk module, ``native_*`` the same with the trunk as visionrl_amd.decode_step (5 launches per layer, 6 with adapters).
    """
    import types

    hidden, inter, layers, heads = shape   # Janus-Pro-1B by default; (4096, 11008, 30, 32) is the 7B-class trunk

    import torch.nn.functional as F
    from torch import nn
    from transformers import LlamaConfig, LlamaModel

    from visionrl_amd.ar_decode import StaticARSampler
    from visionrl_amd.policy_glue import apply_int4_to_policy

    cfg = LlamaConfig(hidden_size=hidden, intermediate_size=inter, num_hidden_layers=layers,
                      num_attention_heads=heads, num_key_value_heads=heads, vocab_size=128,
                      max_position_embeddings=1024)

    class MMGPT(nn.Module):
        def __init__(self):
            super().__init__()
            self.language_model = types.SimpleNamespace(model=LlamaModel(cfg).to(torch.bfloat16).eval())
            self.gen_head = nn.Linear(hidden, HEAD, bias=False).to(torch.bfloat16)
            self.gen_embed = nn.Embedding(HEAD, hidden).to(torch.bfloat16)

        def prepare_gen_img_embeds(self, ids):
            return self.gen_embed(ids)

    class Policy:
        def __init__(self):
            self.mmgpt = MMGPT()
            self.config = types.SimpleNamespace(cfg_weight=5.0, temperature=1.0, image_token_num=tokens)

        def _base(self):
            return self.mmgpt

        def _lm_trunk(self):
            return self.mmgpt.language_model.model

    @torch.no_grad()
    def reference_style(policy, cond, uncond, cmask, umask, n_img):
        trunk, base = policy._lm_trunk(), policy._base()
        B = cond.shape[0]
        toks = torch.empty(B, n_img, dtype=torch.long, device=device)
        lps = torch.empty(B, n_img, dtype=torch.float32, device=device)
        embeds, attn, past = torch.cat([cond, uncond]), torch.cat([cmask, umask]), None
        for pos in range(n_img):
            out = trunk(inputs_embeds=embeds, attention_mask=attn, use_cache=True, past_key_values=past)
            past = out.past_key_values
            logits = base.gen_head(out.last_hidden_state[:, -1:, :]).squeeze(1)
            c, u = logits.chunk(2, dim=0)
            probs = F.softmax((u + 5.0 * (c - u)) / 1.0, dim=-1)
            sampled = torch.multinomial(probs, num_samples=1).squeeze(-1)
            lp = F.log_softmax(c / 1.0, dim=-1).gather(-1, sampled.unsqueeze(-1)).squeeze(-1)
            toks[:, pos], lps[:, pos] = sampled, lp
            embeds = base.prepare_gen_img_embeds(torch.cat([sampled, sampled]).unsqueeze(-1))
            attn = torch.cat([attn, torch.ones(2 * B, 1, dtype=attn.dtype, device=device)], dim=1)
        return toks, lps

    def per_token_ms(fn):
        """fn(n) samples n image tokens; the prompt pass and the first token are timed apart (n = 1)
        and subtracted, so the figure is the cost of one decode step at cache lengths
        prompt .. prompt + tokens."""
        def timed(n):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn(n)
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3
        fn(tokens)   # warm-up (and graph capture where there is one)
        return (timed(tokens) - min(timed(1), timed(1))) / (tokens - 1)

    out = {"tokens_per_call": tokens, "prompt_tokens": prompt,
           "model": f"LlamaModel {layers} x ({hidden}, {inter}), {heads} heads, head {hidden}->{HEAD}, random weights"}
    with torch.device(device):
        torch.manual_seed(0)
        policy = Policy()
    policy.mmgpt.to(device)
    policy._lm_trunk().to(device)
    inputs = {}
    for B in batches:
        g = torch.Generator(device=device).manual_seed(7000 + B)
        inputs[B] = (torch.randn((B, prompt, hidden), generator=g, device=device).to(torch.bfloat16),
                     torch.randn((B, prompt, hidden), generator=g, device=device).to(torch.bfloat16),
                     torch.ones((B, prompt), dtype=torch.long, device=device),
                     torch.ones((B, prompt), dtype=torch.long, device=device))
    for B in batches if only is None else ():
        entry = out.setdefault(f"B{B}", {})
        entry["bf16_reference_style_ms_per_token"] = per_token_ms(
            lambda n: reference_style(policy, *inputs[B], n))
        sampler = StaticARSampler(policy, graph=True, fused_tail=False, native=False)
        entry["bf16_static_hip_graph_ms_per_token"] = per_token_ms(
            lambda n: sampler.sample_image_tokens(*inputs[B], image_token_num=n))
        del sampler
        torch.cuda.empty_cache()
    class LoraWrapper(nn.Module):
        """The forward of a PEFT LoRA wrapper (not installed here) with the reference's defaults:
        rank 32, alpha 64, float32 adapter weights on q/k/v/o_proj (policy.py:81-88, :298-324)."""

        def __init__(self, base, r=32, alpha=64):
            super().__init__()
            self.base_layer = base
            self.lora_A = nn.ModuleDict({"default": nn.Linear(base.in_features, r, bias=False)})
            self.lora_B = nn.ModuleDict({"default": nn.Linear(r, base.out_features, bias=False)})
            self.scaling, self.active_adapters = {"default": alpha / r}, ["default"]
            self.merged = self.disable_adapters = False
            nn.init.normal_(self.lora_B["default"].weight, std=0.01)

        def forward(self, x):
            a, b = self.lora_A["default"], self.lora_B["default"]
            return (self.base_layer(x) + b(a(x.to(a.weight.dtype))) * self.scaling["default"]).to(x.dtype)

    def with_adapters(on: bool):
        for layer in policy._lm_trunk().layers:
            for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
                mod = getattr(layer.self_attn, name)
                if on and not isinstance(mod, LoraWrapper):
                    setattr(layer.self_attn, name, LoraWrapper(mod).to(device))
                elif not on and isinstance(mod, LoraWrapper):
                    setattr(layer.self_attn, name, mod.base_layer)

    apply_int4_to_policy(policy, group_size=GROUP)
    torch.cuda.empty_cache()
    if only in (None, "int4_lora_native_hip_graph"):
        with_adapters(True)
        for B in batches:
            entry = out.setdefault(f"B{B}", {})
            for name, native in (("int4_lora_static_hip_graph", False), ("int4_lora_native_hip_graph", True)):
                if only is not None and name != only:
                    continue
                sampler = StaticARSampler(policy, graph=True, native=native)
                entry[f"{name}_ms_per_token"] = per_token_ms(
                    lambda n: sampler.sample_image_tokens(*inputs[B], image_token_num=n))
                del sampler
                torch.cuda.empty_cache()
        with_adapters(False)
    for B in batches:
        entry = out.setdefault(f"B{B}", {})
        if only is None:
            entry["int4_reference_style_ms_per_token"] = per_token_ms(
                lambda n: reference_style(policy, *inputs[B], n))
        for name, graph, native in (("int4_static_eager", False, False), ("int4_static_hip_graph", True, False),
                                    ("int4_native_eager", False, True), ("int4_native_hip_graph", True, True)):
            if only is not None and name != only:
                continue
            sampler = StaticARSampler(policy, graph=graph, native=native)
            entry[f"{name}_ms_per_token"] = per_token_ms(
                lambda n: sampler.sample_image_tokens(*inputs[B], image_token_num=n))
            del sampler
            torch.cuda.empty_cache()
        if only is None:   # a whole image: 40-token prompt, 576 image tokens, prompt pass included
            short = tuple(t[:, :40].contiguous() for t in inputs[B])
            sampler = StaticARSampler(policy)
            sampler.sample_image_tokens(*short, image_token_num=576)   # records the step for this shape
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            sampler.sample_image_tokens(*short, image_token_num=576)
            torch.cuda.synchronize()
            entry["int4_native_hip_graph_s_per_576_token_image_batch"] = time.perf_counter() - t0
            del sampler
            torch.cuda.empty_cache()
    return out


def launch_floor_us(device, nodes: int = 96, reps: int = 50):
    """us per node of a HIP graph of tiny dependent kernels: what a launch costs with no work in it."""
    t = torch.zeros(64, device=device)
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        for _ in range(nodes):
            t.add_(1.0)
    return time_region(graph.replay, reps, 3) / nodes * 1e3


def bench_library():
    """``libvrl_bench.so``: the measurement kernels (nothing in the product path loads it)."""
    import ctypes

    from visionrl_amd.build import BENCH_LIB_PATH

    if not os.path.exists(BENCH_LIB_PATH):
        raise RuntimeError(f"{BENCH_LIB_PATH} is missing: build it with `python -m visionrl_amd.build`")
    return ctypes.CDLL(BENCH_LIB_PATH)


class ValuDotLaunch:
    """The grouped launch of ``ops.GroupedGemv`` run by the comparison build of its kernel whose dot product is
    on the vector unit (``v_dot2_f32_bf16``) instead of the matrix cores: plain prepacked problems of one
    activation row and group size 128, in a plan large enough for the throughput form.  The build lives in
    ``libvrl_bench.so``; the plan and the outputs are the product library's."""

    def __init__(self, problems):
        import ctypes

        from visionrl_amd import _lib, ops

        for x, pw, fused in problems:
            if x.shape[0] != 1 or fused or pw.group_size != 128:
                raise ValueError("the vector-unit build takes plain prepacked problems of one row, group size 128")
        self.grouped = ops.GroupedGemv(problems)
        if self.grouped.info.variant != 2 or self.grouped.info.block_threads != 256:
            raise ValueError("the vector-unit build takes plans of the four-wave throughput form")
        self.outputs = self.grouped.outputs
        self._lib = bench_library()
        self._lib.vrl_bench_gemv_grouped_valu_dot_bf16.restype = ctypes.c_int
        self._lib.vrl_bench_gemv_grouped_valu_dot_bf16.argtypes = [ctypes.c_void_p, ctypes.POINTER(_lib.PlanInfo),
                                                                   ctypes.c_void_p]
        self._byref = ctypes.byref(self.grouped.info)

    def launch(self):
        g = self.grouped
        with torch.cuda.device(g.device):
            rc = self._lib.vrl_bench_gemv_grouped_valu_dot_bf16(g.plan.data_ptr(), self._byref,
                                                                torch.cuda.current_stream(g.device).cuda_stream)
        if rc:
            raise RuntimeError(f"vrl_bench_gemv_grouped_valu_dot_bf16 failed: {rc}")
        return self.outputs


def stream_read(device, nbytes: int, steps: int, warmup: int):
    """GB/s of a plain non-temporal streaming read of ``nbytes`` (the size of the headline launch's
    algorithmic bytes) by ``stream_read_kernel`` of csrc/bench_kernels.hip: what the memory system
    gives a kernel that does nothing with the data, as the reference point for the GEMV figures."""
    import ctypes

    lib = bench_library()
    lib.vrl_bench_stream_read.restype = ctypes.c_int
    lib.vrl_bench_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int,
                                          ctypes.c_void_p]
    nbytes = nbytes // 4096 * 4096
    buf = torch.randint(-2 ** 31, 2 ** 31, (nbytes // 8,), device=device, dtype=torch.int64)
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    out = {"bytes": nbytes}
    best = None
    for waves_per_cu in (16, 28, 32):
        def launch():
            rc = lib.vrl_bench_stream_read(buf.data_ptr(), nbytes, sink.data_ptr(), waves_per_cu,
                                           torch.cuda.current_stream(device).cuda_stream)
            if rc:
                raise RuntimeError(f"vrl_bench_stream_read failed: {rc}")
        ms, per_block = time_blocks(launch, steps, warmup, blocks=5, min_warm_ms=100.0)
        out[f"waves_per_cu_{waves_per_cu}"] = {"ms": ms, "GBps": nbytes / (ms * 1e-3) / 1e9, "blocks_ms": per_block}
        if best is None or ms < best:
            best = ms
    out["ms"] = best
    out["GBps"] = nbytes / (best * 1e-3) / 1e9
    return out


def cpu_single_gemv(seconds: float = 4.0):
    """The single 2048 x 2048 GEMV at M = 1 on the host cores: PyTorch dequant + matmul per call, and the
    matmul alone over a weight dequantised beforehand (us per call, median)."""
    from oracle import int4_oracle as oracle  # the checker, used here as the reported CPU baseline

    cpu = torch.device("cpu")
    K = N = HIDDEN
    qw, sc, qz = make_weights(1001, K, N, GROUP, cpu)
    x = make_x(1007, 1, K, cpu)
    w = oracle.torch_dequant(qw, sc, qz, GROUP)

    def median_us(fn, budget):
        fn()
        times = []
        t_end = time.perf_counter() + budget
        while len(times) < 10 or (time.perf_counter() < t_end and len(times) < 2000):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        times.sort()
        return times[len(times) // 2] * 1e6, len(times)

    full_us, n_full = median_us(lambda: oracle.torch_cpu_linear(x, qw, sc, qz, GROUP), seconds * 0.75)
    mm_us, n_mm = median_us(lambda: torch.nn.functional.linear(x, w), seconds * 0.25)
    nbytes = oracle.algorithmic_bytes(1, K, N, GROUP)
    return {"shape": f"M=1, K={K}, N={N}, G={GROUP}", "dequant_plus_matmul_us_per_call": full_us,
            "dequant_plus_matmul_GBps": nbytes / (full_us * 1e-6) / 1e9, "calls": n_full,
            "matmul_only_us_per_call": mm_us, "matmul_only_calls": n_mm,
            "matmul_only_GBps_of_bf16_weight": (2 * K * N) / (mm_us * 1e-6) / 1e9}


def cpu_baseline(seconds: float = 12.0):
    """PyTorch dequant + matmul on the host cores over one decoder layer's seven linears."""
    from oracle import int4_oracle as oracle  # the checker, used here as the reported CPU baseline

    cpu = torch.device("cpu")
    ops_cpu = []
    nbytes = 0
    for proj, (name, K, N) in enumerate(LAYER_LINEARS):
        qw, sc, qz = make_weights(2000 + proj, K, N, GROUP, cpu)
        ops_cpu.append((make_x(2007, 1, K, cpu), qw, sc, qz))
        nbytes += oracle.algorithmic_bytes(1, K, N, GROUP)

    def layer():
        for x, qw, sc, qz in ops_cpu:
            oracle.torch_cpu_linear(x, qw, sc, qz, GROUP)

    layer()
    t0 = time.perf_counter()
    reps = 0
    while True:
        layer()
        reps += 1
        el = time.perf_counter() - t0
        if el >= seconds or reps >= 200:
            break
    return {"value": nbytes * reps / el / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{reps} passes over one decoder layer's 7 linears (M=1, {nbytes} B each pass), "
                      f"torch CPU dequant + F.linear, {el:.1f} s",
            "us_per_layer_pass": el / reps * 1e6,
            "host_cpu_count": os.cpu_count(),
            "single_gemv": cpu_single_gemv()}


def load_traffic(kernel: str):
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    try:
        with open(path) as fh:
            return json.load(fh).get(kernel)
    except (OSError, ValueError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-headline", action="store_true",
                    help="run just the grouped decode-step launches (for profilers)")
    ap.add_argument("--rows", type=int, default=1, choices=(1, 8, 16, 32),
                    help="with --only-headline: 1 = the M=1 set (default), 32 = the rollout-batch set plus the "
                         "image-token head; with --shapes 7b: 1, 8 or 16 rows")
    ap.add_argument("--shapes", default="1b", choices=("1b", "7b", "5a"),
                    help="with --only-headline: 1b = the Janus-Pro-1B set (default); 7b = the 7B-class set plus its "
                         "head (configuration 4); 5a = the fused gate||up launch over 24 weight sets, K=4096, "
                         "N=2x11008, M=8 (configuration 5a)")
    ap.add_argument("--valu-dot", action="store_true",
                    help="with --only-headline (M=1): the comparison build whose dot product runs on the vector unit")
    ap.add_argument("--single-calls", action="store_true",
                    help="loop single-GEMV launches over distinct weights per shape and exit (for profilers)")
    ap.add_argument("--lora", action="store_true", help="with --ar-decode: LoRA adapters on q/k/v/o_proj")
    ap.add_argument("--ar-decode", type=int, default=0, metavar="B",
                    help="run only the recorded decode loop at batch B on the int4 policy and exit (for profilers)")
    ap.add_argument("--context", type=int, default=304, metavar="SLOTS",
                    help="with --ar-decode: tokens in the cache before the timed steps (304: the start of a "
                         "generation, 520: its middle, 784: its end)")
    ap.add_argument("--trunk-7b", action="store_true",
                    help="with --ar-decode: the 7B-class trunk (30 x (4096, 11008), 32 heads) instead of the 1B one")
    ap.add_argument("--attn-decode", type=int, default=0, metavar="ROWS",
                    help="run 8 attention decode launches (16 heads x 128, slot 330 of 384) over distinct caches "
                         "at ROWS rows and exit (for counter runs)")
    ap.add_argument("--head-sample", action="store_true",
                    help="only the head + sampling tail of a decode step: two launches against the one call")
    ap.add_argument("--stream-read", action="store_true",
                    help="time the plain streaming read of 642.5 MB and exit (for profilers)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run plain 1 GiB device copies and exit (reference point for HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus 1 only)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X: no ROCm device is visible")

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=device).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": 1 << 30, "copy_bytes_written": 1 << 30, "copies": args.steps}))
        return
    from visionrl_amd import ops

    if args.attn_decode:
        rows, heads, dim, slots, at = args.attn_decode, 16, 128, 384, 330
        new = lambda *shape: torch.randn(shape, device=device).to(torch.bfloat16)
        q, k, v = new(rows, heads * dim), new(rows, heads * dim), new(rows, heads * dim)
        caches = [(new(rows, heads, slots, dim), new(rows, heads, slots, dim)) for _ in range(8)]
        cos, sin = new(slots, dim), new(slots, dim)
        mask = torch.ones((rows, slots), dtype=torch.uint8, device=device)
        pos = torch.tensor([at], dtype=torch.int64, device=device)
        out = torch.empty((rows, heads * dim), dtype=torch.bfloat16, device=device)
        for kc, vc in caches:
            ops.rope_attn_decode(q, k, v, kc, vc, cos, sin, mask, pos, dim ** -0.5, out=out)
        torch.cuda.synchronize()
        print(json.dumps({"attn_decode_launches": len(caches), "rows": rows,
                          "cache_bytes_read_per_launch": rows * heads * at * dim * 2 * 2}))
        return
    if args.ar_decode:
        which = "int4_lora_native_hip_graph" if args.lora else "int4_native_hip_graph"
        shape = (4096, 11008, 30, 32) if args.trunk_7b else (HIDDEN, INTER, LAYERS, 16)
        print(json.dumps(ar_decode_loop(device, only=which, batches=(args.ar_decode,), shape=shape,
                                        prompt=args.context)))
        return
    if args.single_calls:
        for M in (1, 32):
            for K, N in ((HIDDEN, HIDDEN), (HIDDEN, INTER), (INTER, HIDDEN), (HIDDEN, HEAD)):
                ws = [make_weights(100 + i, K, N, GROUP, device) for i in range(40)]
                x = make_x(1, M, K, device)
                y = torch.empty((M, N), dtype=torch.bfloat16, device=device)
                direct = []
                if M <= ops.DirectGemv.MAX_ROWS:   # the plan-free launch over the prepacked layout
                    direct = [ops.DirectGemv([(x, ops.int4_prepack(qw, sc, qz, GROUP), False)]) for qw, sc, qz in ws]
                for _ in range(3):
                    for qw, sc, qz in ws:
                        ops.int4_gemv_into(y, x, qw, sc, qz, GROUP)
                    for launch in direct:
                        launch.launch()
                torch.cuda.synchronize()
        print(json.dumps({"single_calls": "done"}))
        return

    if args.head_sample:
        print(json.dumps({"decode_head_and_tail": decode_head_and_tail(device, args.steps),
                          "decode_tail_cfg_sample": decode_tail(device, args.steps),
                          "prompt_pass_linears": prompt_pass_linears(device, args.steps)}))
        return

    if args.stream_read:
        print(json.dumps({"stream_read": stream_read(device, 642_539_520, args.steps, args.warmup)}))
        return

    if args.only_headline and args.shapes == "5a":
        print(json.dumps(fused_gate_up_launch(device, args.steps, args.warmup)))
        return
    if args.only_headline and args.shapes == "7b":
        if args.rows == 32:
            raise SystemExit("the 7B-class configuration is quoted at 1, 8 and 16 rows")
        items = build_set(4, args.rows, device, with_head=True, hidden=4096, inter=11008, layers=30, head=16384)
    elif args.only_headline and args.rows == 32:
        items = build_set(3, 32, device, with_head=True)
    elif args.only_headline and args.rows != 1:
        raise SystemExit("the 1B set is quoted at 1 and 32 rows")
    else:
        items = build_set(2, 1, device, with_head=False)
    torch.cuda.synchronize()

    if args.only_headline:
        launcher = ValuDotLaunch if args.valu_dot else ops.GroupedGemv
        grouped = launcher([(it["x"], it["prepacked"], False) for it in items])
        ms, per_block = time_blocks(grouped.launch, args.steps, args.warmup)
        nbytes = sum(it["bytes"] for it in items)
        counts = {}
        worst = check_outputs(items, grouped.outputs, "grouped launch", counts)
        print(json.dumps({"shapes": args.shapes, "rows": args.rows, "valu_dot": bool(args.valu_dot), "ms_per_step": ms,
                          "blocks_ms": per_block,
                          "algorithmic_bytes_per_step": nbytes, "GBps": nbytes / (ms * 1e-3) / 1e9,
                          "outputs_checked": len(items), "worst_backward_error": worst, "tolerance_counts": counts}))
        return

    strat, total_bytes, grouped = measure_set(items, args.steps, args.warmup)
    headline = "grouped_1_launch"
    ms = strat["ms_per_step"][headline]
    blocks = strat["grouped_1_launch_blocks_ms"]
    value = strat["GBps"][headline]
    # the dominant kernel's own duration: the grouped kernel is the whole step, one launch each, so the
    # HIP-event regions that time the step (on the stream the launches go to) are the kernel's average
    # launch duration too; the median of the blocks is reported, the spread beside it
    kernel_ms = ms
    achieved = total_bytes / (kernel_ms * 1e-3) / 1e9
    try:
        read = stream_read(device, total_bytes, max(20, args.steps), args.warmup)
    except Exception as exc:  # the reference point is an extra, never the headline
        read = {"error": repr(exc)[:300]}

    latency = per_call_latency(items, args.steps)
    try:
        latency["empty_kernel_hip_graph_node_us"] = launch_floor_us(device)
    except Exception as exc:
        latency["empty_kernel_error"] = repr(exc)[:200]
    try:
        modules = module_path(items, args.steps)
    except Exception as exc:
        modules = {"error": repr(exc)[:300]}
    try:
        tail = decode_tail(device, args.steps)
    except Exception as exc:
        tail = {"error": repr(exc)[:300]}
    try:
        prompt = prompt_pass_linears(device, args.steps)
    except Exception as exc:
        prompt = {"error": repr(exc)[:300]}
    try:
        head_tail = decode_head_and_tail(device, args.steps)
    except Exception as exc:
        head_tail = {"error": repr(exc)[:300]}
    best = max(strat["GBps"], key=lambda k: strat["GBps"][k])

    del items, grouped
    torch.cuda.empty_cache()

    # rollout batch M=32 plus the image-token head
    items32 = build_set(3, 32, device, with_head=True)
    strat32, bytes32, grouped32 = measure_set(items32, max(10, args.steps), max(2, args.warmup))
    kernel32_ms = strat32["ms_per_step"]["grouped_1_launch"]   # one launch per step: the same regions
    del items32, grouped32
    torch.cuda.empty_cache()

    try:
        ar_loop = ar_decode_loop(device)
    except Exception as exc:
        ar_loop = {"error": repr(exc)[:300]}
    torch.cuda.empty_cache()
    # the same step where a generation over a prompt padded to 256 slots spends its time: around slot
    # 256 + 288 (its middle) and around slot 800 (its end)
    for name, ctx in (("B1_at_544_slots", 520), ("B1_at_808_slots", 784)):
        try:
            long_run = ar_decode_loop(device, only="int4_native_hip_graph", batches=(1,), prompt=ctx)
            if isinstance(ar_loop, dict):
                ar_loop[name] = long_run["B1"]
        except Exception as exc:
            if isinstance(ar_loop, dict):
                ar_loop[name] = {"error": repr(exc)[:300]}
        torch.cuda.empty_cache()

    try:
        others = other_configs(device, args.steps, args.warmup)
    except Exception as exc:  # the other configurations are detail, never the headline
        others = {"error": repr(exc)[:300]}

    single = latency.get(f"{HIDDEN}x{HIDDEN}", {})
    chain = {}
    if isinstance(ar_loop, dict) and "B1" in ar_loop:
        step_ms = ar_loop["B1"].get("int4_native_hip_graph_ms_per_token")
        if step_ms:
            # the int4 weights one decode step of the 1B policy streams: the 168 trunk linears and the head
            from visionrl_amd.int4_format import algorithmic_bytes
            step_bytes = LAYERS * sum(algorithmic_bytes(2, K, N, GROUP) for _, K, N in LAYER_LINEARS) + \
                algorithmic_bytes(2, HIDDEN, HEAD, GROUP)
            chain = {"what": "one decode step of a Janus-Pro-1B shaped policy at B=1 (2 rows): 24 dependent layers "
                             "(five launches each), head and sampling tail, replayed from one HIP graph",
                     "ms_per_step": step_ms, "GBps_of_int4_weights": step_bytes / (step_ms * 1e-3) / 1e9,
                     "cache_slots": "304 + 48 (the start of a generation); ms_per_step_at_544_slots: its middle",
                     "ms_per_step_at_544_slots": (ar_loop.get("B1_at_544_slots") or {}).get(
                         "int4_native_hip_graph_ms_per_token"),
                     "ms_per_step_at_808_slots": (ar_loop.get("B1_at_808_slots") or {}).get(
                         "int4_native_hip_graph_ms_per_token"),
                     "linears_only_4_launches_per_layer_hip_graph_ms": strat["ms_per_step"].get(
                         "per_layer_4_launches_hip_graph")}

    result = {
        "metric": "int4 GEMV GB/s (% of HBM peak) + us/call, Janus-1B shapes at M=1 and M=32",
        "value": value,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "ms_per_step_blocks": blocks,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "Janus-Pro-1B decoder linear set, M=1: 24 layers x (4x 2048->2048, "
                               "2x 2048->5632, 1x 5632->2048), int4 group 128, 168 GEMVs, distinct weights, "
                               "one activation tensor per distinct input (q|k|v and gate|up share theirs)",
                   "algorithmic_bytes_per_step": total_bytes,
                   "launch": "one grouped launch per step (all 168 GEMVs in one kernel), weights "
                             "repacked once at load into the MFMA-shaped layout",
                   "timing": f"median of {len(blocks)} HIP-event blocks of --steps launches after --warmup launches "
                             "and at least 200 ms of launches; every output of the timed launch checked afterwards"},
        "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBS,
        "us_per_call": {"config": "single 2048x2048 GEMV, M=1 (BASELINE configuration 1), rotating over distinct "
                                  "weight sets that together exceed the 256 MB memory-side cache in either layout",
                        "distinct_weights": single.get("distinct_weights"),
                        "pool_bytes_canonical": single.get("pool_bytes_canonical"),
                        "pool_bytes_prepacked": single.get("pool_bytes_prepacked"),
                        "hip_graph_node": single.get("us_per_call_prepacked_hip_graph"),
                        "eager_c_abi": single.get("us_per_call_direct"),
                        "eager_torch_op": single.get("us_per_call_torch_op")},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": load_traffic("gemv_stream_kernel"),
                     "traffic_source": "profiles/traffic.json: rocprofv3 FETCH_SIZE + WRITE_SIZE runs of this launch "
                                       "(profiles/gemv_stream_kernel_janus1b_m1.txt), not measured in this run",
                     "kernel": "gemv_stream_kernel", "bytes_per_launch": total_bytes,
                     "avg_launch_ms": kernel_ms, "launch_ms_min_max": [blocks[0], blocks[-1]],
                     "stream_read_GBps": read.get("GBps"),
                     "frac_of_stream_read": (achieved / read["GBps"]) if read.get("GBps") else None},
        # the same kernel in its 32-row build (16-wave workgroups), the M=32 half of the metric
        "roofline_m32": {"bound": "hbm", "achieved": bytes32 / (kernel32_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                         "unit": "GB/s", "frac": bytes32 / (kernel32_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                         "traffic": load_traffic("gemv_stream_kernel_m32"), "kernel": "gemv_stream_kernel",
                         "bytes_per_launch": bytes32, "avg_launch_ms": kernel32_ms,
                         "launch_ms_blocks": strat32["grouped_1_launch_blocks_ms"]},
        # the shipped decode path is a chain of dependent launches: its figure, beside the independent set's
        "dependent_chain": chain,
        "cpu_baseline": None if args.no_cpu else cpu_baseline(),
        "detail": {"m1": strat, "m1_best_strategy": best, "m1_us_per_call": latency, "stream_read": read,
                   "m32_plus_head": strat32, "m32_algorithmic_bytes_per_step": bytes32,
                   "m1_through_modules": modules, "decode_tail_cfg_sample": tail, "decode_head_and_tail": head_tail,
                   "prompt_pass_linears": prompt,
                   "ar_decode_loop_1b": ar_loop,
                   "other_configs": others},
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
