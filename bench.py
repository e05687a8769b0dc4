"""Benchmark of the grouped packed-GGUF matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload pair|decode|multi|gathered|layer|dense|down]

Default workload ("pair"): the 256-expert MoE gate+up pair, Q5_K weights [512, 2048] per
expert and projection, T = 8192 tokens x top-8 with Zipf-skewed routing (65 536 expert-sorted
rows), one step = grouped_mmq_pair forward + its grad-input (both cotangents ~ N(0,1)).
Inputs are synthetic and resident in HBM before the timed region.  Prints ONE JSON line.

`roofline` describes the kernel that takes most of the step, timed with HIP events recorded
by the library around each of its launches inside the timed region.  `cpu_baseline` times
the oracle's dequantize-to-fp32 plus torch.matmul on the host cores over a bounded sample
of the same workload (a baseline only).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for entry in (ROOT, ROOT / "torch-ggml-ops_amd", ROOT / "tests"):   # (tests/: the synthetic blocks and routing)
    if str(entry) not in sys.path:
        sys.path.insert(0, str(entry))

import torch  # noqa: E402

PEAK = {"hbm": 8000.0, "int8": 5000.0, "bf16": 2500.0, "fp32_vector": 157.3}  # GB/s, TOP/s, TFLOP/s (dense, published)
# What the forward algorithm allows: every int8 matrix-core result of a 32-value block needs two fp32 vector
# operations (x weight-block scale, x activation-block scale + accumulate), and packed fp32 forms are not used,
# so the vector pipe delivers fp32_vector / 4 lane-operations per second (the published figure counts a fused
# multiply-add as two and the packed form as two more) and every two of them complete 32 multiply-adds = 64 ops.
VALU_BOUND_INT8 = PEAK["fp32_vector"] / 4 / 2 * 64  # TOP/s: 1258.4, i.e. 25.2 % of the int8 matrix-core peak
# Arithmetic type of the forward dot products by the library's operand kind (forward_operand_for).
OPERAND_DTYPE = {"int8": "int8", "half": "fp16 holding exact integers", "scaled": "fp16 carrying the scales"}


def build_pair_workload(device, tokens=8192, experts=256, top_k=8, n=512, k=2048, qtype=13, seed=2024):
    import synth

    token_of_row, indices, offsets, _ = synth.zipf_routing(tokens, experts, top_k, seed, device=device)
    generator = torch.Generator(device=device).manual_seed(seed + 1)
    hidden = torch.randn(tokens, k, device=device, generator=generator).to(torch.bfloat16)
    rows = token_of_row.numel()
    return {
        "x": hidden.index_select(0, token_of_row).contiguous(),
        "first": synth.random_packed_weight(qtype, (experts, n), k, seed + 2, device=device),
        "second": synth.random_packed_weight(qtype, (experts, n), k, seed + 3, device=device),
        "grad_first": torch.randn(rows, n, device=device, generator=generator).to(torch.bfloat16),
        "grad_second": torch.randn(rows, n, device=device, generator=generator).to(torch.bfloat16),
        "indices": indices,
        "offsets": offsets,
        "rows": rows, "n": n, "k": k, "qtype": qtype, "experts": experts, "tokens": tokens, "top_k": top_k,
    }


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` on the default workload, from the committed counter summary
    (rocprofv3 FETCH_SIZE and WRITE_SIZE passes scaled by a copy kernel of known size); None if absent."""
    path = ROOT / "profiles" / "grouped_pair_q5k_hbm_traffic.json"
    try:
        entry = json.loads(path.read_text())["kernels"][kernel]
        return float(entry["fetch_bytes"]) + float(entry["write_bytes"])
    except (OSError, KeyError, ValueError):
        return None


def measured_pipe_busy(kernel):
    """Fraction of the kernel's time its matrix and vector pipes were busy on the default workload, from the committed
    counter summary (rocprofv3 SQ_VALU_MFMA_BUSY_CYCLES, SQ_ACTIVE_INST_VALU and SQ_BUSY_CYCLES); None if absent."""
    path = ROOT / "profiles" / "grouped_pair_q5k_pipe_utilisation.json"
    try:
        return json.loads(path.read_text())["kernels"][kernel]
    except (OSError, KeyError, ValueError):
        return None


def decode_traffic():
    """HBM bytes per launch of the single-row kernel on the 132 MB dense matrix (the decode workload's best case):
    FETCH_SIZE from the committed counter summary plus the bf16 output row; None if absent."""
    path = ROOT / "profiles" / "decode_gemv_hbm_traffic.json"
    try:
        entry = json.loads(path.read_text())["kernels"]["mmq_gemv_kernel<12, 1, 1, false>"]
        return float(entry["fetch_bytes"]) + 28672 * 2
    except (OSError, KeyError, ValueError):
        return None


def pair_step(w):
    ops = torch.ops.torch_ggml_ops
    out_first, out_second = ops.grouped_mmq_pair.default(
        w["x"], w["first"], w["second"], w["indices"], w["offsets"], w["qtype"], w["n"]
    )
    grad_input = ops.grouped_mmq_pair_grad_input.default(
        w["grad_first"], w["grad_second"], w["first"], w["second"], w["indices"], w["offsets"], w["qtype"], w["k"]
    )
    return out_first, out_second, grad_input


def measure_pair_format(device, name, qtype, steps=10, warmup=3):
    """The default workload with another weight format (the reference's model packs its gate and up projections as
    IQ2_S): step time by the wall clock, kernel times from the event brackets."""
    from torch_ggml_ops import _native

    w = build_pair_workload(device, qtype=qtype)
    for _ in range(warmup):
        pair_step(w)
    torch.cuda.synchronize()
    _native.lib.tgo_profile_enable(1)
    start = time.perf_counter()
    for _ in range(steps):
        pair_step(w)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    kernels = {name_: _native.profile_read(name_) for name_ in ("quantize", "forward", "pack_cotangent", "grad_input")}
    _native.lib.tgo_profile_enable(0)
    flops = 4 * 2.0 * w["rows"] * w["n"] * w["k"]
    record = {
        "workload": f"grouped_mmq_pair fwd+bwd, gate+up {name} [512,2048], same routing as the headline workload",
        "value": flops / (elapsed / steps) / 1e12, "unit": "TFLOP/s", "ms_per_step": elapsed / steps * 1e3, "steps": steps,
        "forward_operands": _native.forward_operand_for(qtype, w["rows"], w["n"], 2),
        "kernels_us": {k: total / launches * 1e3 for k, (total, launches) in kernels.items() if launches},
    }
    del w
    torch.cuda.empty_cache()
    return record


def cpu_baseline_pair(w, budget_seconds=15.0):
    """Dequantize to fp32 with the oracle + torch.matmul, forward and grad-input, group by group."""
    from oracle import gguf_oracle as oracle

    threads = torch.get_num_threads()
    n, k, qtype = w["n"], w["k"], w["qtype"]
    offsets = w["offsets"].cpu().tolist()
    indices = w["indices"].cpu().tolist()
    x = w["x"].cpu().float()
    grads = (w["grad_first"].cpu().float(), w["grad_second"].cpu().float())
    weights = (w["first"].cpu().numpy(), w["second"].cpu().numpy())
    flops, groups, passes = 0.0, 0, 0
    start = time.perf_counter()
    while time.perf_counter() - start < budget_seconds:
        begin = 0
        for expert, end in zip(indices, offsets):
            for packed, grad in zip(weights, grads):
                dense = torch.from_numpy(oracle.dequant_f32(qtype, packed[expert], k))
                _ = x[begin:end] @ dense.T
                _ = grad[begin:end] @ dense
                flops += 2 * 2.0 * (end - begin) * n * k
            begin = end
            groups += 1
            if time.perf_counter() - start > 2 * budget_seconds:
                break
        passes += 1
    elapsed = time.perf_counter() - start
    return {
        "value": flops / elapsed / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{groups} expert groups in {passes} pass(es) over the workload's {len(indices)} groups ({w['rows']} rows), "
        f"oracle dequant to fp32 + torch.matmul forward and grad-input, {elapsed:.1f} s",
    }


def measure_decode(args, device) -> dict:
    """Decode regime (HBM-bound): T in {1,4,8} tokens x top-8 over 256 experts through the gate+up pair
    (IQ2_S [512,2048]) and the down projection (Q6_K [2048,512]), plus a dense Q3_K [4096,2048] row.
    Every call uses a different seeded routing out of eight, so successive calls touch different experts
    and the weights (392 MB in total) do not stay in the 256 MB last-level cache."""
    import torch_ggml_ops as tgo
    import synth
    from torch_ggml_ops import _native

    experts, top_k = 256, 8
    gate = synth.random_packed_weight(synth.IQ2_S, (experts, 512), 2048, 11, device=device)
    up = synth.random_packed_weight(synth.IQ2_S, (experts, 512), 2048, 12, device=device)
    down = synth.random_packed_weight(synth.Q6_K, (experts, 2048), 512, 13, device=device)
    dense = [synth.random_packed_weight(synth.Q3_K, (4096,), 2048, 20 + i, device=device) for i in range(96)]
    generator = torch.Generator(device=device).manual_seed(5)
    report = {}
    cases = set(args.decode_cases.split(","))
    for tokens in (1, 4, 8):
        if f"T{tokens}" not in cases:
            continue
        routings = []
        for variant in range(8):
            token_of_row, indices, offsets, _ = synth.zipf_routing(tokens, experts, top_k, 100 * tokens + variant, device=device)
            hidden = torch.randn(tokens, 2048, device=device, generator=generator).to(torch.bfloat16)
            routings.append((hidden.index_select(0, token_of_row).contiguous(), indices, offsets))
        mid = [torch.randn(r[0].shape[0], 512, device=device, generator=generator).to(torch.bfloat16) for r in routings]

        def step(i):
            x, indices, offsets = routings[i % 8]
            tgo.grouped_mmq_pair(x, gate, up, indices, offsets, synth.IQ2_S, 512)
            tgo.grouped_mmq(mid[i % 8], down, indices, offsets, synth.Q6_K, 2048)

        # (a layer call is tens of microseconds: timed over enough calls that the first ones, which still grow
        # torch's allocator pools, and the closing synchronisation do not set the figures)
        steps, warmup = max(args.steps, 100), max(args.warmup, 20)
        for i in range(warmup):
            step(i)
        torch.cuda.synchronize()
        _native.lib.tgo_profile_enable(1)
        start = time.perf_counter()
        for i in range(steps):
            step(i)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        kernel_ms, launches = _native.profile_read("forward_gemv")
        quantize_ms, _ = _native.profile_read("quantize")   # (zero where the GEMV kernels quantize their own rows)
        _native.lib.tgo_profile_enable(0)
        if launches == 0:
            continue  # too many rows per expert for the GEMV family: that shape belongs to the MFMA benchmark
        graph_fields = {}
        if not args.no_graph_replays:
            # the same layer call replayed from a HIP graph (one routing): what a serving loop would do about launch cost
            capture_stream = torch.cuda.Stream()
            capture_stream.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(capture_stream):
                step(0)
            torch.cuda.current_stream().wait_stream(capture_stream)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=capture_stream):
                step(0)
            # (a replay is tens of microseconds: enough of them that the closing synchronisation does not set the figure)
            replays = max(args.steps, 200)
            for _ in range(max(args.warmup, 50)):
                graph.replay()
            torch.cuda.synchronize()
            graph_start = time.perf_counter()
            for _ in range(replays):
                graph.replay()
            torch.cuda.synchronize()
            graph_elapsed = time.perf_counter() - graph_start
            # the whole layer from token activations and the router's choices (tgo.moe_layer: routing, gate+up with the
            # activation, down projection, weighted return to the tokens), replayed from a graph
            hidden = torch.randn(tokens, 2048, device=device, generator=generator).to(torch.bfloat16)
            slot_experts = torch.stack([torch.randperm(experts, device=device, generator=generator)[:top_k] for _ in range(tokens)])
            slot_weights = torch.softmax(torch.randn(tokens, top_k, device=device, generator=generator), dim=1)

            def layer():
                return tgo.moe_layer(hidden, slot_experts, slot_weights, gate, up, down, synth.IQ2_S, synth.Q6_K, 512)

            with torch.no_grad():
                capture_stream.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(capture_stream):
                    layer()
                torch.cuda.current_stream().wait_stream(capture_stream)
                torch.cuda.synchronize()
                layer_graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(layer_graph, stream=capture_stream):
                    layer()
                for _ in range(max(args.warmup, 50)):
                    layer_graph.replay()
                torch.cuda.synchronize()
                layer_start = time.perf_counter()
                for _ in range(replays):
                    layer_graph.replay()
                torch.cuda.synchronize()
                layer_elapsed = time.perf_counter() - layer_start
        active = sum(r[1].numel() for r in routings) / 8
        expert_bytes = 2 * 512 * 8 * 82 + 2048 * 2 * 210
        weight_bytes = active * expert_bytes
        if not args.no_graph_replays:
            # (the whole-layer replay routes every token to top_k different experts drawn uniformly: more experts, and
            # so more weight bytes, than the skewed routings of the layer calls above)
            layer_active = int(slot_experts.unique().numel())
            graph_fields = {
                "us_per_layer_call_graph_replay": graph_elapsed / replays * 1e6,
                "us_per_moe_layer_graph_replay": layer_elapsed / replays * 1e6,
                "graph_replays_timed": replays,
                "moe_layer_active_experts": layer_active,
                "moe_layer_weight_MB": layer_active * expert_bytes / 1e6,
                "moe_layer_GBps_graph_replay": layer_active * expert_bytes / (layer_elapsed / replays) / 1e9,
            }
        report[f"T{tokens}"] = {
            "active_experts": active,
            "weight_MB": weight_bytes / 1e6,
            "layer_calls_timed": steps,
            "us_per_layer_call": elapsed / steps * 1e6,
            **graph_fields,
            "GBps_end_to_end": weight_bytes / (elapsed / steps) / 1e9,
            "gemv_kernel_us_per_step": kernel_ms / steps * 1e3,
            "quantize_kernel_us_per_step": quantize_ms / steps * 1e3,
            "launches_per_layer_call": launches / steps + (2 if quantize_ms > 0 else 0),
            "GBps_gemv_kernels": weight_bytes / (kernel_ms / steps * 1e-3) / 1e9,
        }
    x = torch.randn(1, 2048, device=device, generator=generator).to(torch.bfloat16)
    if "dense" not in cases:
        dense = []
    for i in range(args.warmup if dense else 0):
        tgo.mmq(x, dense[i % 96], synth.Q3_K, 4096)
    torch.cuda.synchronize()
    _native.lib.tgo_profile_enable(1)
    start = time.perf_counter()
    for i in range(args.steps * 4 if dense else 0):
        tgo.mmq(x, dense[i % 96], synth.Q3_K, 4096)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    kernel_ms, launches = _native.profile_read("forward_gemv")
    _native.lib.tgo_profile_enable(0)
    dense_bytes = 4096 * 8 * 110
    if launches:
        report["dense_Q3_K_M1"] = {
            "weight_MB": dense_bytes / 1e6,
            "us_per_call": elapsed / (args.steps * 4) * 1e6,
            "gemv_kernel_us": kernel_ms / launches * 1e3,
            "GBps_gemv_kernel": dense_bytes / (kernel_ms / launches * 1e-3) / 1e9,
        }
    # a matrix large enough for bandwidth to matter: one FFN projection of a 70B-class dense model, M = 1, 2, 8, 16
    big_n, big_k = 28672, 8192
    big = [synth.random_packed_weight(synth.Q4_K, (big_n,), big_k, 40 + i, device=device) for i in range(3)] if "big" in cases else []
    big_bytes = big_n * (big_k // 256) * 144
    for m in (1, 2, 8, 16) if big else ():
        xb = torch.randn(m, big_k, device=device, generator=generator).to(torch.bfloat16)
        for i in range(args.warmup):
            tgo.mmq(xb, big[i % 3], synth.Q4_K, big_n)
        torch.cuda.synchronize()
        _native.lib.tgo_profile_enable(1)
        start = time.perf_counter()
        for i in range(args.steps):
            tgo.mmq(xb, big[i % 3], synth.Q4_K, big_n)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        kernel_ms, launches = _native.profile_read("forward_gemv")
        _native.lib.tgo_profile_enable(0)
        report[f"dense_Q4_K_{big_n}x{big_k}_M{m}"] = {
            "name": f"{big_n}x{big_k}_M{m}",
            "weight_MB": big_bytes / 1e6,
            "us_per_call": elapsed / args.steps * 1e6,
            "gemv_kernel_us": kernel_ms / launches * 1e3,
            "GBps_gemv_kernel": big_bytes / (kernel_ms / launches * 1e-3) / 1e9,
        }
    if "skewed" in cases:
        # a small batch that the host cannot tell from an even one: every expert listed, one group of 200 rows and 56
        # single rows (the kernel family is chosen from rows and listed groups; the large group's eight-row tasks share
        # the expert's weights through the L2)
        sizes = [0] * experts
        sizes[7] = 200
        for i in range(56):
            sizes[20 + 3 * i] = 1
        offsets = torch.tensor(sizes, dtype=torch.int64).cumsum(0).to(torch.int32).to(device)
        indices = torch.arange(experts, dtype=torch.int64, device=device)
        x = torch.randn(sum(sizes), 2048, device=device, generator=generator).to(torch.bfloat16)
        for _ in range(args.warmup):
            tgo.grouped_mmq_pair(x, gate, up, indices, offsets, synth.IQ2_S, 512)
        torch.cuda.synchronize()
        _native.lib.tgo_profile_enable(1)
        for _ in range(args.steps):
            tgo.grouped_mmq_pair(x, gate, up, indices, offsets, synth.IQ2_S, 512)
        torch.cuda.synchronize()
        kernel_ms, launches = _native.profile_read("forward_gemv")
        _native.lib.tgo_profile_enable(0)
        skew_bytes = 57 * 2 * 512 * 8 * 82
        if launches:
            report["skewed_256_rows_57_experts"] = {
                "weight_MB": skew_bytes / 1e6,
                "kernel_family": _native.lib.tgo_forward_kernel_family(sum(sizes), experts).decode(),
                "gemv_kernel_us": kernel_ms / launches * 1e3,
                "GBps_gemv_kernel": skew_bytes / (kernel_ms / launches * 1e-3) / 1e9,
            }
    for record in report.values():
        rate = record.get("GBps_gemv_kernels", record.get("GBps_gemv_kernel"))
        if rate is not None:
            record["frac_of_hbm_peak"] = rate / PEAK["hbm"]
            # the north-star target of the decode regime next to what was measured: 0.70 of the HBM peak
            record["roofline"] = {"bound": "hbm", "achieved": rate, "peak": PEAK["hbm"], "unit": "GB/s",
                                  "frac": rate / PEAK["hbm"], "target_frac": 0.70,
                                  "traffic": decode_traffic() if "28672x8192_M1" in str(record.get("name", "")) else None}
    return report


def run_decode(args, device) -> None:
    report = measure_decode(args, device)
    best = max(v.get("GBps_gemv_kernels", v.get("GBps_gemv_kernel", 0.0)) for v in report.values())
    print(json.dumps({
        "metric": "decode-regime weight bandwidth (GEMV kernels), 256-expert MoE shape",
        "value": best, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": True, "dtype": "int8 dot products, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "decode: T in {1,4,8} x top-8, pair IQ2_S [512,2048] + down Q6_K [2048,512]; dense Q3_K [4096,2048] M=1; "
                   "dense Q4_K [28672,8192] M=1, 2, 8, 16 (value = best case)"},
        "roofline": {"bound": "hbm", "achieved": best, "peak": PEAK["hbm"], "unit": "GB/s", "frac": best / PEAK["hbm"],
                     "traffic": decode_traffic()},
        "cases": report,
    }))


def _native_kind(qtype: int, rows: int, out_features: int, projections: int) -> str:
    from torch_ggml_ops import _native

    return _native.forward_operand_for(qtype, rows, out_features, projections)


def run_multi(args, device) -> None:
    """Several dense projections of one input (attention q/k/v of a GQA layer: 4096 -> 4096, 1024, 1024, Q4_K,
    4096 token rows): three `mmq` calls against one `mmq_multi`, which quantizes the activations once."""
    import torch_ggml_ops as tgo
    import synth
    from torch_ggml_ops import prepared

    rows, k, widths = 4096, 4096, (4096, 1024, 1024)
    generator = torch.Generator(device=device).manual_seed(9)
    x = torch.randn(rows, k, device=device, generator=generator).to(torch.bfloat16)
    weights = [synth.random_packed_weight(synth.Q4_K, (n,), k, 60 + i, device=device) for i, n in enumerate(widths)]
    qtypes = [synth.Q4_K] * len(widths)

    def separate():
        return [tgo.mmq(x, w, q, n) for w, q, n in zip(weights, qtypes, widths)]

    def fused():
        return tgo.mmq_multi(x, weights, qtypes, widths)

    timings = {}
    for name, fn in (("separate", separate), ("multi", fused)):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        start = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        timings[name] = (time.perf_counter() - start) / args.steps
    flops = 2.0 * rows * k * sum(widths)
    print(json.dumps({
        "metric": "dense multi-projection forward throughput (q/k/v of one input, activations quantized once)",
        "value": flops / timings["multi"] / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": timings["multi"] * 1e3, "higher_is_better": True,
        "dtype": OPERAND_DTYPE[prepared.multi_operand(qtypes, rows, widths)] + " dot products, fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": "dense q/k/v: x [4096, 4096] bf16 x Q4_K [4096 | 1024 | 1024, 4096]"},
        "separate_mmq_ms": timings["separate"] * 1e3,
        "speedup_over_separate_calls": timings["separate"] / timings["multi"],
    }))


def _kernel_us(_native, names):
    """Average kernel time per launch (us) from the library's event brackets, for each kernel id in `names`."""
    out = {}
    for name in names:
        total_ms, count = _native.profile_read(name)
        if count:
            out[name] = total_ms / count * 1e3
    return out


def measure_dense_cell(args, device, qtype, n, m, k=2048, weight=None) -> dict:
    """Forward and grad-input kernel time of one dense cell (kernel time from the HIP-event brackets)."""
    import torch_ggml_ops as tgo
    import synth
    from torch_ggml_ops import _native

    if weight is None:
        weight = synth.random_packed_weight(qtype, (n,), k, 7 + qtype, device=device)
    generator = torch.Generator(device=device).manual_seed(m)
    x = torch.randn(m, k, device=device, generator=generator).to(torch.bfloat16)
    dy = torch.randn(m, n, device=device, generator=generator).to(torch.bfloat16)
    record = {}
    for label, fn, kernels in (
        ("fwd", lambda: tgo.mmq(x, weight, qtype, n), ("quantize", "forward", "forward_gemv")),
        ("dx", lambda: torch.ops.torch_ggml_ops.mmq_grad_input.default(dy, weight, qtype, k), ("pack_cotangent", "grad_input")),
    ):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        _native.lib.tgo_profile_enable(1)
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        times = _kernel_us(_native, kernels)
        _native.lib.tgo_profile_enable(0)
        total = sum(times.values())
        record[label + "_us"] = round(total, 1)
        record[label + "_TFLOPs"] = round(2.0 * m * n * k / total / 1e6, 1)
        if m <= 16:
            record[label + "_weight_GBps"] = round(weight.numel() / total / 1e3, 1)
    record["forward_operands"] = _native.forward_operand_for(qtype, m, n, 1) if m > 32 else "int8 (GEMV family)"
    return record


def run_dense(args, device) -> None:
    """The dense parity configuration as a sweep: five formats x M in {1, 16, 512, 4096} x N in {2048, 4096},
    K = 2048, forward and grad-input; kernel time per call (quantize + multiply, pack + multiply) and TFLOP/s or,
    for the bandwidth-bound small-M rows, weight GB/s."""
    import torch_ggml_ops as tgo
    import synth
    from torch_ggml_ops import _native

    k = 2048
    names = {11: "Q3_K", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 22: "IQ2_S"}
    rows_out = {}
    best = 0.0
    for qtype, qname in names.items():
        for n in (2048, 4096):
            weight = synth.random_packed_weight(qtype, (n,), k, 7 + qtype, device=device)
            for m in (1, 16, 512, 4096):
                record = measure_dense_cell(args, device, qtype, n, m, k, weight)
                best = max(best, record["fwd_TFLOPs"], record["dx_TFLOPs"])
                rows_out[f"{qname}_N{n}_M{m}"] = record
    print(json.dumps({
        "metric": "dense mmq forward / grad-input kernel time over the dense parity shapes (value = best TFLOP/s of the sweep)",
        "value": best, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": True, "dtype": "int8 or fp16 dot products (forward, per cell), bf16 (grad-input), fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": "dense mmq: Q3_K/Q4_K/Q5_K/Q6_K/IQ2_S x M in {1,16,512,4096} x N in {2048,4096}, K=2048; "
                               "kernel time from HIP-event brackets (launch gaps included)"},
        "cases": rows_out,
    }))


def measure_down(args, device) -> dict:
    """The down projection of the default workload's model: grouped_mmq, 256 experts, Q4_K [2048, 512],
    4096 tokens x top-8 with the same skewed routing (32 768 rows); forward and grad-input kernel times."""
    import torch_ggml_ops as tgo
    import synth
    from torch_ggml_ops import _native

    experts, n, k, qtype = 256, 2048, 512, 12
    token_of_row, indices, offsets, _ = synth.zipf_routing(4096, experts, 8, 11, device=device)
    rows = token_of_row.numel()
    generator = torch.Generator(device=device).manual_seed(3)
    x = torch.randn(rows, k, device=device, generator=generator).to(torch.bfloat16)
    dy = torch.randn(rows, n, device=device, generator=generator).to(torch.bfloat16)
    copies = [synth.random_packed_weight(qtype, (experts, n), k, 73 + i, device=device) for i in range(3)]
    counter = [0]

    def forward():
        counter[0] += 1
        return tgo.grouped_mmq(x, copies[counter[0] % 3], indices, offsets, qtype, n)

    def grad_input():
        counter[0] += 1
        return torch.ops.torch_ggml_ops.grouped_mmq_grad_input.default(dy, copies[counter[0] % 3], indices, offsets, qtype, k)

    flops = 2.0 * rows * n * k
    algorithmic = copies[0].numel() + rows * k * 2 + rows * n * 2
    result = {}
    for label, fn, kernels in (("forward", forward, ("quantize", "forward")),
                               ("grad_input", grad_input, ("pack_cotangent", "grad_input"))):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        _native.lib.tgo_profile_enable(1)
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        times = _kernel_us(_native, kernels)
        _native.lib.tgo_profile_enable(0)
        total = sum(times.values())
        result[label] = {"kernels_us": {key: round(value, 1) for key, value in times.items()}, "total_us": round(total, 1),
                         "TFLOPs": round(flops / total / 1e6, 1), "algorithmic_GBps": round(algorithmic / total / 1e3, 1)}
    result["rows"] = rows
    result["flops_per_direction"] = flops
    result["algorithmic_bytes"] = algorithmic
    # the forward of this shape is HBM-bound on this part (arithmetic intensity 216 FLOP/B, below the ridge)
    result["forward"]["frac_of_hbm_peak"] = result["forward"]["algorithmic_GBps"] / PEAK["hbm"]
    result["grad_input"]["frac_of_hbm_peak"] = result["grad_input"]["algorithmic_GBps"] / PEAK["hbm"]
    return result


def run_down(args, device) -> None:
    result = measure_down(args, device)
    rows, flops, algorithmic = result.pop("rows"), result.pop("flops_per_direction"), result.pop("algorithmic_bytes")
    both = result["forward"]["total_us"] + result["grad_input"]["total_us"]
    print(json.dumps({
        "metric": "grouped MMQ down projection fwd+bwd throughput (kernel time)", "value": 2 * flops / both / 1e6,
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": both / 1e3,
        "higher_is_better": True,
        "dtype": OPERAND_DTYPE[_native_kind(12, rows, 2048, 1)] + " (forward dot products), bf16 (grad-input), fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": f"grouped_mmq fwd+bwd: 256 experts, down Q4_K [2048,512], T=4096 x top-8 ({rows} rows), "
                               "Zipf-skewed routing; three weight copies in turn"},
        "roofline": {"bound": "hbm", "achieved": algorithmic / result["forward"]["total_us"] / 1e3, "peak": 8000.0,
                     "unit": "GB/s", "frac": algorithmic / result["forward"]["total_us"] / 1e3 / 8000.0, "traffic": None},
        "cases": result,
    }))


def run_gathered(args, device) -> None:
    """The default workload's forward from unsorted token activations: `index_select` to expert-sorted rows
    followed by `grouped_mmq_pair`, against `grouped_mmq_pair_gathered`, whose quantizer reads the token rows."""
    import torch_ggml_ops as tgo
    import synth

    tokens, experts, top_k, n, k, qtype, seed = 8192, 256, 8, 512, 2048, 13, 2024
    token_of_row, indices, offsets, _ = synth.zipf_routing(tokens, experts, top_k, seed, device=device)
    generator = torch.Generator(device=device).manual_seed(seed + 1)
    hidden = torch.randn(tokens, k, device=device, generator=generator).to(torch.bfloat16)
    first = synth.random_packed_weight(qtype, (experts, n), k, seed + 2, device=device)
    second = synth.random_packed_weight(qtype, (experts, n), k, seed + 3, device=device)
    rows = token_of_row.numel()

    def separate():
        return tgo.grouped_mmq_pair(hidden.index_select(0, token_of_row), first, second, indices, offsets, qtype, n)

    def fused():
        return tgo.grouped_mmq_pair_gathered(hidden, token_of_row, first, second, indices, offsets, qtype, n)

    timings = {}
    for name, fn in (("index_select", separate), ("gathered", fused)):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        start = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        timings[name] = (time.perf_counter() - start) / args.steps
    flops = 2 * 2.0 * rows * n * k
    print(json.dumps({
        "metric": "grouped gate+up forward throughput from unsorted token activations (gather folded into the quantizer)",
        "value": flops / timings["gathered"] / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": timings["gathered"] * 1e3, "higher_is_better": True,
        "dtype": OPERAND_DTYPE[_native_kind(13, rows, n, 2)] + " dot products, fp32 accumulate", "data": "synthetic",
        "config": {"workload": f"grouped_mmq_pair forward: 256 experts, gate+up Q5_K [512,2048], T=8192 x top-8 ({rows} rows), "
                               "token activations [8192, 2048] + int64 row index"},
        "index_select_then_pair_ms": timings["index_select"] * 1e3,
        "speedup_over_index_select": timings["index_select"] / timings["gathered"],
    }))


def run_layer(args, device) -> None:
    """Forward of one SwiGLU mixture-of-experts layer from token activations to token outputs (`moe_layer`):
    routing sort, gathered gate+up pair, activation, down projection, routing-weighted combine."""
    import torch_ggml_ops as tgo
    import synth
    from torch_ggml_ops import _native

    tokens, experts, top_k, intermediate, features, qtype, seed = 8192, 256, 8, 512, 2048, 13, 2024
    token_of_row, indices, offsets, _ = synth.zipf_routing(tokens, experts, top_k, seed, device=device)
    # recover per-token choices from the benchmark's routing: the expert of every sorted row, regrouped by token
    expert_of_row = torch.repeat_interleave(indices, torch.diff(offsets.long(), prepend=offsets.new_zeros(1).long()))
    by_token = torch.argsort(token_of_row, stable=True)
    slot_experts = expert_of_row[by_token].reshape(tokens, top_k).contiguous()
    generator = torch.Generator(device=device).manual_seed(seed + 1)
    hidden = torch.randn(tokens, features, device=device, generator=generator).to(torch.bfloat16)
    slot_weights = torch.softmax(torch.randn(tokens, top_k, device=device, generator=generator), dim=-1)
    gate = synth.random_packed_weight(qtype, (experts, intermediate), features, seed + 2, device=device)
    up = synth.random_packed_weight(qtype, (experts, intermediate), features, seed + 3, device=device)
    down = synth.random_packed_weight(qtype, (experts, features), intermediate, seed + 4, device=device)

    def step():
        return tgo.moe_layer(hidden, slot_experts, slot_weights, gate, up, down, qtype, qtype, intermediate)

    def unfused_step():
        # the same layer with the activation on the caller's side of the pair operator
        row_index, slot_rows, expert_indices, expert_offsets = tgo.route(slot_experts, experts)
        gate_rows, up_rows = tgo.grouped_mmq_pair_gathered(
            hidden, row_index, gate, up, expert_indices, expert_offsets, qtype, intermediate
        )
        activated = torch.nn.functional.silu(gate_rows) * up_rows
        rows_out = tgo.grouped_mmq(activated, down, expert_indices, expert_offsets, qtype, features)
        return tgo.moe_combine(rows_out, slot_rows, slot_weights)

    for _ in range(args.warmup):
        unfused_step()
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(args.steps):
        unfused_step()
    torch.cuda.synchronize()
    unfused = (time.perf_counter() - start) / args.steps

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    _native.lib.tgo_profile_enable(1)
    start = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = (time.perf_counter() - start) / args.steps
    kernels = {}
    for name in ("quantize", "forward", "combine"):
        total_ms, launches = _native.profile_read(name)
        if launches:
            kernels[name] = {"avg_ms": total_ms / launches, "launches_per_step": launches / args.steps}
    _native.lib.tgo_profile_enable(0)
    # forward + backward of the layer (gradient of the token activations), with the down projection and the
    # combine as one step (its backward gathers and scales the per-token gradient while packing the cotangent)
    # against the two separate operators (whose backward builds the expert-sorted gradient with torch operators)
    grad_out = torch.randn(tokens, features, device=device, generator=generator).to(torch.bfloat16)

    def two_step_layer(x):
        row_index, slot_rows, expert_indices, expert_offsets = tgo.route(slot_experts, experts)
        activated = tgo.grouped_mmq_swiglu(x, gate, up, expert_indices, expert_offsets, qtype, intermediate, row_index)
        rows_out = tgo.grouped_mmq(activated, down, expert_indices, expert_offsets, qtype, features)
        return tgo.moe_combine(rows_out, slot_rows, slot_weights)

    training = {}
    for name, fn in (("fused_down_combine", lambda x: tgo.moe_layer(x, slot_experts, slot_weights, gate, up, down, qtype, qtype, intermediate)),
                     ("two_step_combine", two_step_layer)):
        x = hidden.clone().requires_grad_(True)
        for _ in range(args.warmup):
            fn(x).backward(grad_out)
        torch.cuda.synchronize()
        start = time.perf_counter()
        for _ in range(args.steps):
            fn(x).backward(grad_out)
        torch.cuda.synchronize()
        training[name + "_fwd_bwd_ms"] = (time.perf_counter() - start) / args.steps * 1e3
    rows = tokens * top_k
    combine_bytes = 2.0 * features * (rows + tokens) + 12.0 * rows
    combine_rate = combine_bytes / (kernels["combine"]["avg_ms"] * 1e-3) / 1e9
    kernels["combine"].update({"achieved": combine_rate, "unit": "GB/s", "frac_of_peak": combine_rate / PEAK["hbm"]})
    flops = 3 * 2.0 * rows * intermediate * features
    print(json.dumps({
        "metric": "SwiGLU MoE layer forward throughput, token activations in, token outputs out",
        "value": flops / elapsed / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": elapsed * 1e3, "higher_is_better": True,
        "dtype": OPERAND_DTYPE[_native_kind(qtype, rows, intermediate, 2)] + " dot products, fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": f"moe_layer forward: 256 experts, gate/up/down Q5_K, features 2048, intermediate 512, "
                               f"T=8192 x top-8 ({rows} sorted rows)"},
        "kernels": kernels,
        "caller_side_activation_ms": unfused * 1e3,
        "training": training,
    }))


def main() -> None:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=5)
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--decode-cases", default="T1,T4,T8,dense,big,skewed",
                        help="decode workload: which cases to run (T1, T4, T8: MoE layer calls; dense: Q3_K [4096,2048] "
                        "single row; big: Q4_K [28672,8192] with 1..16 rows; skewed: 256 rows, 200 of them in one of 57 "
                        "groups, all 256 experts listed)")
    parser.add_argument("--no-graph-replays", action="store_true",
                        help="decode workload: leave out the graph replays (profiler runs: per-dispatch averages then "
                             "cover the eager layer calls only)")
    parser.add_argument("--no-sub-records", action="store_true",
                        help="pair workload only: skip the down-projection and decode sub-records")
    parser.add_argument("--workload", choices=("pair", "decode", "multi", "gathered", "layer", "dense", "down"), default="pair")
    parser.add_argument(
        "--quant", choices=("Q3_K", "Q4_K", "Q5_K", "Q6_K", "IQ2_S"), default="Q5_K",
        help="weight format of the pair workload (the metric is quoted on Q5_K; the others are for comparison)",
    )
    parser.add_argument(
        "--calibration-copy", action="store_true",
        help="after the timed region, run one 256 MiB device-to-device copy (a kernel of known traffic for "
        "scaling rocprofv3's FETCH_SIZE / WRITE_SIZE counters; not timed, not part of the result)",
    )
    parser.add_argument("--operand", choices=("auto", "half", "int8", "scaled"), default="auto",
                        help="matrix operands of the MFMA forward kernels: fp16 numbers holding the exact integers, int8, "
                        "or the library's default (fp16 for IQ2_S, int8 for the other formats)")
    args = parser.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")

    import torch_ggml_ops  # noqa: F401
    from torch_ggml_ops import _native

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    _native.set_forward_operand(args.operand)
    if args.workload == "decode":
        run_decode(args, device)
        return
    if args.workload == "multi":
        run_multi(args, device)
        return
    if args.workload == "dense":
        run_dense(args, device)
        return
    if args.workload == "down":
        run_down(args, device)
        return
    if args.workload == "gathered":
        run_gathered(args, device)
        return
    if args.workload == "layer":
        run_layer(args, device)
        return
    quant_ids = {"Q3_K": 11, "Q4_K": 12, "Q5_K": 13, "Q6_K": 14, "IQ2_S": 22}
    w = build_pair_workload(device, qtype=quant_ids[args.quant])
    rows, n, k = w["rows"], w["n"], w["k"]

    for _ in range(args.warmup):
        pair_step(w)
    torch.cuda.synchronize()
    _native.lib.tgo_profile_enable(1)
    start = time.perf_counter()
    for _ in range(args.steps):
        pair_step(w)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    kernels = {name: _native.profile_read(name) for name in ("quantize", "forward", "pack_cotangent", "grad_input")}
    _native.lib.tgo_profile_enable(0)
    if args.calibration_copy:
        source = torch.empty(256 << 20, dtype=torch.uint8, device=device).random_(0, 255)
        target = torch.empty_like(source)
        target.copy_(source)
        torch.cuda.synchronize()

    ms_per_step = elapsed / args.steps * 1e3
    flops_projection = 2.0 * rows * n * k
    step_flops = 4 * flops_projection  # two projections forward + two Jacobian products backward
    active = w["indices"].numel()
    weight_bytes = 2 * active * n * (k // 256) * _native.lib.tgo_block_bytes(w["qtype"])

    # the forward multiplies int8 operands, fp16 numbers holding the same integers, or fp16 numbers that carry the
    # scales as well: the library's choice for this call unless --operand forces one
    operand_kind = _native.forward_operand_for(w["qtype"], rows, n, 2)
    half_operands = operand_kind in ("half", "scaled")
    forward_peak = PEAK["bf16"] if half_operands else PEAK["int8"]   # fp16 and bf16 share the dense matrix peak
    forward_dtype = OPERAND_DTYPE[operand_kind]
    # bytes the quantizer moves: bf16 in; int8 or fp16 values, an fp32 scale and sum per 32 values, and for the scaled
    # operands a power of two and eight fp16 block sums per 256 values and a power of two per row out
    quantize_bytes = rows * k * 2 + rows * k * (2 if half_operands else 1) + 2 * rows * (k // 32) * 4
    if operand_kind == "scaled":
        quantize_bytes += rows * (k // 256) * 20 + rows * 4
    # per-launch algorithmic work of each profiled kernel
    per_launch = {
        "forward": ("mfma", 2 * flops_projection / 1e12, forward_peak, "TFLOP/s"),  # both projections per launch
        "grad_input": ("mfma", 2 * flops_projection / 1e12, PEAK["bf16"], "TFLOP/s"),  # both products per launch
        "quantize": ("hbm", quantize_bytes / 1e9, PEAK["hbm"], "GB/s"),
        "pack_cotangent": ("hbm", 2 * 2 * rows * n * 2 / 1e9, PEAK["hbm"], "GB/s"),  # both cotangents read + written
    }
    breakdown = {}
    for name, (total_ms, launches) in kernels.items():
        if launches:
            breakdown[name] = {"avg_ms": total_ms / launches, "launches_per_step": launches / args.steps}
    dominant = max(
        (name for name in breakdown if name in per_launch),
        key=lambda name: breakdown[name]["avg_ms"] * breakdown[name]["launches_per_step"],
    )
    bound, work, peak, unit = per_launch[dominant]
    achieved = work / (breakdown[dominant]["avg_ms"] * 1e-3)
    roofline = {
        "kernel": dominant,
        "bound": bound,
        "achieved": achieved,
        "peak": peak,
        "unit": unit,
        "frac": achieved / peak,
        "traffic": measured_traffic(dominant) if args.quant == "Q5_K" else None,
        "avg_launch_ms": breakdown[dominant]["avg_ms"],
        # achieved / what two fp32 vector operations per matrix-core result allow (forward kernel only)
        "valu_bound": VALU_BOUND_INT8 if dominant == "forward" and not half_operands else None,
        "valu_bound_frac": achieved / VALU_BOUND_INT8 if dominant == "forward" and not half_operands else None,
    }
    for name in breakdown:
        if name in per_launch:
            b, wk, pk, un = per_launch[name]
            breakdown[name].update({"achieved": wk / (breakdown[name]["avg_ms"] * 1e-3), "unit": un, "frac_of_peak": wk / (breakdown[name]["avg_ms"] * 1e-3) / pk})
    if "forward" in breakdown and not half_operands:
        breakdown["forward"]["valu_bound_frac"] = breakdown["forward"]["achieved"] / VALU_BOUND_INT8
    if args.quant == "Q5_K":
        # what keeps the two matrix-core kernels from their peak: pipe occupancy from the committed counter runs
        for name in ("forward", "grad_input"):
            if name in breakdown:
                breakdown[name]["pipes"] = measured_pipe_busy(name)

    result = {
        "metric": "grouped MMQ pair forward+backward throughput, 256-expert MoE shape",
        "value": step_flops / (elapsed / args.steps) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": forward_dtype + " (forward dot products) / bf16 (grad-input), fp32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": f"grouped_mmq_pair fwd+bwd: 256 experts, gate+up {args.quant} [512,2048], T=8192 x top-8 "
            "Zipf(1.1)-skewed routing",
            "rows": rows,
            "active_experts": active,
            "quant_type": args.quant,
            "forward_operands": operand_kind,
        },
        "weight_GBps": weight_bytes * 2 / (elapsed / args.steps) / 1e9,  # read once forward, once backward
        "roofline": roofline,
        "kernels": breakdown,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_pair(w)
    if not args.no_sub_records and args.quant == "Q5_K":
        # the other configurations of the same model, timed in the same run (kernel time from the event brackets)
        del w
        torch.cuda.empty_cache()
        down = measure_down(args, device)
        result["down"] = {
            "workload": f"grouped_mmq down projection: 256 experts, Q4_K [2048,512], T=4096 x top-8 ({down['rows']} rows)",
            "forward": down["forward"], "grad_input": down["grad_input"],
        }
        result["pair_iq2s"] = measure_pair_format(device, "IQ2_S", 22)
        decode = measure_decode(args, device)
        result["decode"] = {
            "workload": "T in {1,4,8} x top-8 over 256 experts: gate+up IQ2_S [512,2048] + down Q6_K [2048,512]; "
                        "dense Q3_K [4096,2048] M=1; dense Q4_K [28672,8192] M=1..16; 256 rows skewed onto one of 57 "
                        "experts; weight GB/s of the kernels, each with its roofline block (target 0.70 of HBM)",
            "cases": decode,
        }
        # the matrix-core-bound cell of the dense configuration: M = 4096 rows against [4096, 2048], every format
        result["dense_M4096"] = {
            "workload": "dense mmq forward / grad-input, x [4096, 2048] x W [4096, 2048]: kernel time and TFLOP/s "
                        "(peak 2500 for fp16/bf16 operands, 5000 for int8)",
            "cases": {name: measure_dense_cell(args, device, qtype, 4096, 4096)
                      for qtype, name in ((11, "Q3_K"), (12, "Q4_K"), (13, "Q5_K"), (14, "Q6_K"), (22, "IQ2_S"))},
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
