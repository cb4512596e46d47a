#!/usr/bin/env python3
"""Headline benchmark: dense INT8 attention at N=32K, Hq16/Hkv4/D128, BF16, one MI355X.

A step is one ``int8_attention(q, k, v)`` call on inputs resident in HBM: Q/K/V
preparation plus the fused attention kernel, as the reference's latency figures
include quantisation (reference README.md:102-106).  The JSON line reports
dense-equivalent TOPS (4*B*Hq*Lq*Lk*D operations per call, reference
benchmarks/plot_scaling.py:66-75), the roofline fraction of the attention
kernel against the dense INT8 MFMA peak, and the numpy oracle timed on the host
cores on the reference's CPU-sized configuration (N=1024) as the CPU baseline.  The same
line carries two short side measurements, timed by whoever runs this file: sparse reuse
against dense at about half coverage (``config.sparse_reuse``) and the masked
configuration (``config.masked``).

The other workloads (``--workload``) follow the reference's measurement protocol
(benchmarks/common.py:184-220): every method is warmed up, then timed in samples of
several calls between two events, with the methods' positions rotated through every slot
and each complete rotation reversed; seeds 0/1/2; medians of the per-seed medians.
``--output FILE`` writes the records as JSON (schema of benchmarks/common.py:321-360),
``--report FILE`` prints such a file as Markdown tables and ``--plot PNG`` draws its dense-
equivalent throughput and SQNR over the sequence length (the role of reference
benchmarks/plot_scaling.py).  ``--workload mask_tiles`` is the broadcast-mask comparison of
reference benchmarks/masks.py (interleaved empty key tiles, optionally against a second build of
the library given with ``--baseline-library``); ``--workload profile_ranges`` wraps warmed calls in
named profiler ranges for ``rocprofv3 --marker-trace`` (the role of reference
benchmarks/profile_operators.py); ``--workload clock`` launches the dense kernel on random and on
all-zero operands (same cycle count, different sustained clock: for a ``--pmc GRBM_GUI_ACTIVE`` run).
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

INT8_MFMA_PEAK_TOPS = 5000.0  # MI355X dense INT8, published
# HBM/Infinity-Cache bytes of one launch of the dense attention kernel at the headline
# shape, from rocprofv3 FETCH_SIZE (299610 KiB raw x 2.0 calibration) + WRITE_SIZE
# (131070 KiB x 1.0); the commands and the copy calibration are in
# profiles/attention_dense_32k_counters.md.
ATTENTION_KERNEL_TRAFFIC_BYTES_32K = int((299610.0 * 2.0 + 131070.0) * 1024)
SHAPE = dict(batch=1, q_heads=16, kv_heads=4, head_dim=128)
SEEDS = (0, 1, 2)


def dense_equivalent_ops(batch, q_heads, q_len, k_len, head_dim):
    return 4.0 * batch * q_heads * q_len * k_len * head_dim


def make_inputs(torch, length, seed, device):
    generator = torch.Generator(device=device).manual_seed(seed)
    shape_q = (SHAPE["batch"], SHAPE["q_heads"], length, SHAPE["head_dim"])
    shape_k = (SHAPE["batch"], SHAPE["kv_heads"], length, SHAPE["head_dim"])
    q = torch.randn(shape_q, generator=generator, device=device, dtype=torch.bfloat16)
    k = torch.randn(shape_k, generator=generator, device=device, dtype=torch.bfloat16)
    v = torch.randn(shape_k, generator=generator, device=device, dtype=torch.bfloat16)
    return q, k, v


def fp32_reference(torch, q, k, v, chunk=2048, mask=None):
    """FP32 SDPA in query chunks (reference benchmarks/common.py:134-145); ``mask`` is a
    broadcastable boolean (True = visible) or additive mask."""
    group = q.shape[1] // k.shape[1]
    kf = k.float().repeat_interleave(group, 1).transpose(-1, -2)
    vf = v.float().repeat_interleave(group, 1)
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    for start in range(0, q.shape[2], chunk):
        scores = q[:, :, start : start + chunk].float() @ kf * q.shape[-1] ** -0.5
        if mask is not None:
            rows = mask if mask.shape[-2] == 1 else mask[..., start : start + chunk, :]
            scores = scores.masked_fill(~rows, float("-inf")) if rows.dtype == torch.bool else scores + rows
        out[:, :, start : start + chunk] = torch.softmax(scores, dim=-1).nan_to_num(nan=0.0) @ vf
    return out


def accuracy(torch, actual, reference):
    """The accuracy record of reference benchmarks/common.py:148-164."""
    import math

    error = actual.float() - reference
    rmse = error.pow(2).mean().sqrt().item()
    rms = reference.pow(2).mean().sqrt().item()
    nrmse = rmse / max(rms, 1e-12)
    return {"rmse": rmse, "nrmse": nrmse, "sqnr_db": -20.0 * math.log10(max(nrmse, 1e-30)),
            "mae": error.abs().mean().item(), "max_abs": error.abs().max().item(),
            "max_channel_bias": error.mean(dim=2).abs().max().item(), "reference_rms": rms}


def percentile(values, fraction):
    ordered = sorted(values)
    position = (len(ordered) - 1) * fraction
    low = int(position)
    high = min(low + 1, len(ordered) - 1)
    return ordered[low] + (ordered[high] - ordered[low]) * (position - low)


def measure_methods(torch, methods, samples=10, calls_per_sample=20, warmup=20):
    """Paired timing of several callables on identical inputs (the protocol of reference
    benchmarks/common.py:184-220): all are warmed up first; sample i then runs every method
    once, ``calls_per_sample`` calls between two events on the current stream, in an order
    that is the name list rotated by i and reversed on every other complete rotation, so
    that each method takes every position (including first after the idle gap) equally often."""
    names = list(methods)
    stream = torch.cuda.current_stream()
    for function in methods.values():
        for _ in range(warmup):
            function()
    torch.cuda.synchronize()
    recorded = {name: [] for name in names}
    for sample in range(samples):
        cycle, shift = divmod(sample, len(names))
        base = names if cycle % 2 == 0 else names[::-1]
        for name in base[shift:] + base[:shift]:
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record(stream)
            for _ in range(calls_per_sample):
                methods[name]()
            end.record(stream)
            end.synchronize()
            recorded[name].append(begin.elapsed_time(end) / calls_per_sample)
    return {name: {"median_ms": statistics.median(values), "p10_ms": percentile(values, 0.1),
                   "p90_ms": percentile(values, 0.9), "samples_ms": [round(v, 5) for v in values],
                   "calls_per_sample": calls_per_sample, "warmup": warmup}
            for name, values in recorded.items()}


def calls_for(ops):
    """Calls per sample: twenty for short problems, fewer as the call gets long."""
    return max(2, min(20, int(4e13 / max(ops, 1.0))))


RECORDS = []  # per-seed records of a --workload run, in the reference's result schema


def case_label(batch, q_heads, kv_heads, q_len, k_len, dim):
    return f"B{batch}_Hq{q_heads}_Hkv{kv_heads}_Lq{q_len}_Lk{k_len}_D{dim}"


def add_record(case, shape, seed, qk_distribution, value_distribution, mode, stage, timing, error=None,
               memory=None, sparse=None):
    """One measurement of one method on one seed, with the field names of reference
    benchmarks/common.py:250-268 (so that its report tool reads the files written here)."""
    RECORDS.append({"case": case, "shape": shape, "seed": seed, "layout": "hnd",
                    "qk_distribution": qk_distribution, "value_distribution": value_distribution,
                    "implementation": "risaattention_amd", "v_quantization": mode, "stage": stage,
                    "timing": timing, "accuracy": error, "memory": memory, "sparse": sparse})


def peak_memory(torch, function):
    """Device memory a call allocates beyond what is resident (reference benchmarks/common.py:222-233)."""
    torch.cuda.synchronize()
    resident = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    output = function()
    torch.cuda.synchronize()
    peak = max(0, torch.cuda.max_memory_allocated() - resident) / 1024**2
    del output
    return {"peak_incremental_mib": peak}


GROUP_FIELDS = ("case", "layout", "qk_distribution", "value_distribution", "implementation", "v_quantization", "stage")


def summarize_records(records):
    """Per (case, method): median over the seeds of the per-seed medians, mean accuracy, mean
    sparse figures (the aggregation of reference benchmarks/report.py:23-63)."""
    groups = {}
    for record in records:
        groups.setdefault(tuple(record[field] for field in GROUP_FIELDS), []).append(record)
    rows = []
    for key, members in groups.items():
        row = dict(zip(GROUP_FIELDS, key))
        row["seed_count"] = len(members)
        for metric in ("median_ms", "p10_ms", "p90_ms"):
            row[metric] = statistics.median(member["timing"][metric] for member in members)
        errors = [member["accuracy"] for member in members if member["accuracy"] is not None]
        for metric in ("nrmse", "rmse", "sqnr_db", "mae", "max_abs", "max_channel_bias"):
            row[metric] = statistics.mean(error[metric] for error in errors) if errors else None
        row["nrmse_std"] = statistics.stdev(error["nrmse"] for error in errors) if len(errors) > 1 else (0 if errors else None)
        memory = [member["memory"]["peak_incremental_mib"] for member in members if member["memory"]]
        row["peak_incremental_mib"] = statistics.median(memory) if memory else None
        sparse = [member["sparse"] for member in members if member["sparse"]]
        for metric in ("coverage", "pattern_index_mib", "exact_construction_recall", "current_recall"):
            row[metric] = statistics.mean(entry[metric] for entry in sparse) if sparse else None
        rows.append(row)
    return rows


def time_calls(torch, fn, calls, warmup=2):
    """Mean of ``calls`` back-to-back calls, HIP events on the current stream."""
    stream = torch.cuda.current_stream()
    for _ in range(warmup):
        fn()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record(stream)
    for _ in range(calls):
        fn()
    end.record(stream)
    end.synchronize()
    return begin.elapsed_time(end) / calls


def sqnr_db(torch, actual, reference):
    noise = (actual.float() - reference.float()).pow(2).mean().item()
    signal = reference.float().pow(2).mean().item()
    return 10.0 * __import__("math").log10(max(signal, 1e-30) / max(noise, 1e-30))


def workload_sweep(torch, risa, args, device):
    """Dense sweep over N, seeds 0/1/2, both V modes timed as a pair on the same inputs;
    latency includes Q/K/V preparation; median of the per-seed medians, mean NRMSE."""
    rows = []
    batch, q_heads, kv_heads, dim = SHAPE["batch"], SHAPE["q_heads"], SHAPE["kv_heads"], SHAPE["head_dim"]
    for length in ([args.length] if args.length else (512, 1024, 2048, 4096, 8192, 16384, 32768)):
        ops = dense_equivalent_ops(batch, q_heads, length, length, dim)
        case = case_label(batch, q_heads, kv_heads, length, length, dim)
        shape = dict(batch=batch, q_heads=q_heads, kv_heads=kv_heads, q_len=length, k_len=length, head_dim=dim)
        first = len(RECORDS)
        for seed in SEEDS:
            q, k, v = make_inputs(torch, length, seed, device)
            methods = {mode: (lambda mode=mode: risa.int8_attention(q, k, v, v_quantization=mode))
                       for mode in ("absmax", "midpoint_affine")}
            timing = measure_methods(torch, methods, samples=args.samples, calls_per_sample=calls_for(ops),
                                     warmup=args.method_warmup)
            reference = fp32_reference(torch, q, k, v)
            for mode, method in methods.items():
                add_record(case, shape, seed, "normal", "normal", mode, "dense", timing[mode],
                           accuracy(torch, method(), reference), peak_memory(torch, method))
            del reference
        for summary in summarize_records(RECORDS[first:]):
            ms = summary["median_ms"]
            rows.append({"N": length, "v_quantization": summary["v_quantization"], "ms": round(ms, 4),
                         "p10_ms": round(summary["p10_ms"], 4), "p90_ms": round(summary["p90_ms"], 4),
                         "tops": round(ops / (ms * 1e-3) / 1e12, 1), "nrmse": round(summary["nrmse"], 5),
                         "nrmse_std": round(summary["nrmse_std"], 6), "sqnr_db": round(summary["sqnr_db"], 2),
                         "peak_incremental_mib": round(summary["peak_incremental_mib"], 1)})
    return rows


def sweep_cells(torch, risa, device, skip=((32768, "absmax"),), seed=0):
    """The other cells of the reference's dense table (README.md:115-123) on one seed, for the
    default line: whole-call latency (mean of a few back-to-back calls) and NRMSE against FP32
    SDPA per sequence length and V mode.  ``--workload sweep`` is the full protocol."""
    batch, q_heads, kv_heads, dim = SHAPE["batch"], SHAPE["q_heads"], SHAPE["kv_heads"], SHAPE["head_dim"]
    cells = []
    for length in (512, 1024, 2048, 4096, 8192, 16384, 32768):
        ops = dense_equivalent_ops(batch, q_heads, length, length, dim)
        q, k, v = make_inputs(torch, length, seed, device)
        reference = fp32_reference(torch, q, k, v)
        for mode in ("absmax", "midpoint_affine"):
            if (length, mode) in skip:
                continue
            call = lambda: risa.int8_attention(q, k, v, v_quantization=mode)
            ms = time_calls(torch, call, calls_for(ops) * 2, warmup=3)
            cells.append({"N": length, "v_quantization": mode, "ms": round(ms, 4),
                          "tops": round(ops / (ms * 1e-3) / 1e12, 1),
                          "nrmse": round(accuracy(torch, call(), reference)["nrmse"], 5)})
        del reference
    return cells


def outlier_inputs(torch, shape_q, shape_k, seed, device):
    generator = torch.Generator(device=device).manual_seed(seed)
    q = torch.randn(shape_q, generator=generator, device=device)
    k = torch.randn(shape_k, generator=generator, device=device)
    v = torch.randn(shape_k, generator=generator, device=device)
    channels = shape_q[-1]
    hot = torch.randperm(channels, generator=generator, device=device)[: max(1, channels // 100)]
    for tensor in (q, k, v):
        tensor[..., hot] *= 20.0
    return q.bfloat16(), k.bfloat16(), v.bfloat16()


def masked_variants(torch, batch, q_len, k_len, device):
    key_padding = torch.ones(batch, 1, 1, k_len, dtype=torch.bool, device=device)
    key_padding[1, ..., int(k_len * 0.9):] = False
    generator = torch.Generator(device=device).manual_seed(1)
    bias = torch.randn(batch, 1, q_len, k_len, generator=generator, device=device)  # float32
    rowmask = torch.ones(batch, 1, q_len, k_len, dtype=torch.bool, device=device)
    rowmask[0, :, :7] = False  # fully masked rows
    # two block-structured boolean masks beside the reference's five variants: eight packed
    # documents (block diagonal) and a causal window of 1024 keys
    rows = torch.arange(q_len, device=device)[:, None]
    keys = torch.arange(k_len, device=device)[None, :]
    documents = ((rows * 8 // q_len) == (keys * 8 // k_len))[None, None].expand(batch, 1, q_len, k_len).contiguous()
    window = ((keys <= rows) & (keys > rows - 1024))[None, None].expand(batch, 1, q_len, k_len).contiguous()
    return {"plain": dict(), "causal": dict(is_causal=True), "key_padding": dict(attn_mask=key_padding),
            "additive_bias": dict(attn_mask=bias), "bool_mask_lse": dict(attn_mask=rowmask, return_lse=True),
            "document_mask": dict(attn_mask=documents), "window_mask": dict(attn_mask=window)}


def workload_masked(torch, risa, args, device, dims=(64, 128), seeds=None, samples=None):
    """Unequal lengths, outlier channels; plain, causal, key-padding mask, additive bias, boolean
    mask + LSE, timed as one rotating group per seed and head dim."""
    rows = []
    batch, heads, q_len, k_len = 2, 24, 4096, 4608
    variants = masked_variants(torch, batch, q_len, k_len, device)
    for dim in dims:
        ops = dense_equivalent_ops(batch, heads, q_len, k_len, dim)
        case = case_label(batch, heads, heads, q_len, k_len, dim)
        shape = dict(batch=batch, q_heads=heads, kv_heads=heads, q_len=q_len, k_len=k_len, head_dim=dim)
        first = len(RECORDS)
        for seed in (seeds or SEEDS):
            q, k, v = outlier_inputs(torch, (batch, heads, q_len, dim), (batch, heads, k_len, dim), seed, device)
            methods = {name: (lambda kwargs=kwargs: risa.int8_attention(q, k, v, **kwargs)) for name, kwargs in variants.items()}
            timing = measure_methods(torch, methods, samples=samples or args.samples, calls_per_sample=10,
                                     warmup=args.method_warmup)
            for name in variants:
                add_record(case, shape, seed, "outlier_channels", "outlier_channels", "absmax", name, timing[name])
        summaries = {summary["stage"]: summary for summary in summarize_records(RECORDS[first:])}
        for name in variants:
            ms = summaries[name]["median_ms"]
            rows.append({"D": dim, "variant": name, "ms": round(ms, 4),
                         "vs_plain": round(ms / summaries["plain"]["median_ms"], 3),
                         "tops": round(ops / (ms * 1e-3) / 1e12 * (0.5 if name == "causal" else 1.0), 1)})
    return rows


def clustered_inputs(torch, length, groups, seed, device):
    generator = torch.Generator(device=device).manual_seed(seed)
    dim = SHAPE["head_dim"]
    per_group = length // groups

    # one centroid per (KV head, token group), shared by K and by the query heads of
    # that KV head's group, plus unit noise (reference benchmarks/sparse.py:30-60)
    kv_heads, q_heads = SHAPE["kv_heads"], SHAPE["q_heads"]
    centroids = torch.randn(1, kv_heads, groups, dim, generator=generator, device=device) * 3.0
    tokens = centroids.repeat_interleave(per_group, 2)
    q = tokens.repeat_interleave(q_heads // kv_heads, 1)
    q = q + torch.randn(q.shape, generator=generator, device=device)
    k = tokens + torch.randn(tokens.shape, generator=generator, device=device)
    v = torch.randn(1, SHAPE["kv_heads"], length, dim, generator=generator, device=device)
    return q, k, v, generator


def workload_sparse(torch, risa, args, device):
    """Construct at theta=0.99 on block-structured Q/K, then five drifting reuse calls."""
    rows = []
    for length in ([args.length] if args.length else (4096, 8192, 16384, 32768)):
        q32, k32, v32, generator = clustered_inputs(torch, length, 64, 0, device)
        q, k, v = q32.bfloat16(), k32.bfloat16(), v32.bfloat16()
        construct_ms = time_calls(torch, lambda: risa.construct_sparse_int8_attention(q, k, v, theta=0.99), 3, 1)
        _, pattern = risa.construct_sparse_int8_attention(q, k, v, theta=0.99)
        dense_samples, sparse_samples, quality = [], [], []
        for _ in range(5):
            q32 = q32 + 0.05 * torch.randn(q32.shape, generator=generator, device=device)
            k32 = k32 + 0.05 * torch.randn(k32.shape, generator=generator, device=device)
            v32 = v32 + 0.05 * torch.randn(v32.shape, generator=generator, device=device)
            q, k, v = q32.bfloat16(), k32.bfloat16(), v32.bfloat16()
            dense_samples.append(time_calls(torch, lambda: risa.int8_attention(q, k, v), 5, 1))
            sparse_samples.append(time_calls(torch, lambda: risa.sparse_int8_attention(q, k, v, pattern), 5, 1))
            sparse_out = risa.sparse_int8_attention(q, k, v, pattern)
            quality.append(sqnr_db(torch, sparse_out, fp32_reference(torch, q, k, v)))
        dense_ms, sparse_ms = statistics.median(dense_samples), statistics.median(sparse_samples)
        rows.append({"N": length, "construct_ms": round(construct_ms, 4), "dense_ms": round(dense_ms, 4),
                     "sparse_ms": round(sparse_ms, 4), "speedup": round(dense_ms / sparse_ms, 3),
                     "coverage": round(pattern.coverage, 4), "measured_mass": round(pattern.measured_retained_mass, 5),
                     "sqnr_db_vs_fp32": round(min(quality), 2)})
    # Half coverage: on unstructured N(0,1) inputs every tile carries about the same
    # mass, so theta = 0.5 keeps about half of the tiles of every query block.
    length = args.length or 32768
    q, k, v = make_inputs(torch, length, 0, device)
    _, pattern = risa.construct_sparse_int8_attention(q, k, v, theta=0.5)
    dense_ms = time_calls(torch, lambda: risa.int8_attention(q, k, v), 10, 2)
    sparse_ms = time_calls(torch, lambda: risa.sparse_int8_attention(q, k, v, pattern), 10, 2)
    rows.append({"N": length, "inputs": "unstructured N(0,1), theta=0.5", "dense_ms": round(dense_ms, 4),
                 "sparse_ms": round(sparse_ms, 4), "speedup": round(dense_ms / sparse_ms, 3),
                 "coverage": round(pattern.coverage, 4)})
    return rows


def block_prototype_inputs(torch, length, seed, device):
    """Q/K = N(0,1) + one of two prototypes of norm 8 per 128-token block (alternating), V ~
    N(0,1); clean tensors for the construction, tensors drifted by 0.05 for the reuse
    (reference benchmarks/sparse.py:30-60)."""
    dim, kv_heads, q_heads = SHAPE["head_dim"], SHAPE["kv_heads"], SHAPE["q_heads"]
    generator = torch.Generator(device=device).manual_seed(seed)
    draw = lambda *shape: torch.randn(shape, generator=generator, device=device)
    clean_q, clean_k, v32 = draw(1, q_heads, length, dim), draw(1, kv_heads, length, dim), draw(1, kv_heads, length, dim)
    prototypes = draw(1, kv_heads, 2, dim)
    prototypes = prototypes * (8.0 / prototypes.norm(dim=-1, keepdim=True))
    block = (torch.arange(length, device=device) // 128) % 2
    clean_k = clean_k + prototypes[:, :, block]
    clean_q = clean_q + prototypes.repeat_interleave(q_heads // kv_heads, 1)[:, :, block]
    drifted_q = (clean_q + 0.05 * draw(*clean_q.shape)).bfloat16()
    drifted_k = (clean_k + 0.05 * draw(*clean_k.shape)).bfloat16()
    return clean_q.bfloat16(), clean_k.bfloat16(), v32.bfloat16(), drifted_q, drifted_k


def sparse_blocks_case(torch, risa, length, mode, seeds, samples, method_warmup, device, with_quality=True):
    """One row of the reference's sparse table: construction / dense / reuse timed as a
    rotating group on every seed; medians of the per-seed medians."""
    from risaattention_amd.fp32_patterns import measure_pattern_recall

    batch, q_heads, kv_heads, dim = SHAPE["batch"], SHAPE["q_heads"], SHAPE["kv_heads"], SHAPE["head_dim"]
    ops = dense_equivalent_ops(batch, q_heads, length, length, dim)
    case = case_label(batch, q_heads, kv_heads, length, length, dim)
    shape = dict(batch=batch, q_heads=q_heads, kv_heads=kv_heads, q_len=length, k_len=length, head_dim=dim)
    first = len(RECORDS)
    for seed in seeds:
        q0, k0, v, drifted_q, drifted_k = block_prototype_inputs(torch, length, seed, device)
        build = lambda: risa.construct_sparse_int8_attention(q0, k0, v, theta=0.99, v_quantization=mode)
        _, pattern = build()
        dense = lambda: risa.int8_attention(drifted_q, drifted_k, v, v_quantization=mode)
        reuse = lambda: risa.sparse_int8_attention(drifted_q, drifted_k, v, pattern, v_quantization=mode)
        methods = {"construct": build, "dense": dense, "reuse": reuse}
        timing = measure_methods(torch, methods, samples=samples, calls_per_sample=calls_for(ops), warmup=method_warmup)
        errors = {name: None for name in methods}
        sparse = None
        if with_quality:
            reference = fp32_reference(torch, drifted_q, drifted_k, v)
            errors["dense"] = accuracy(torch, dense(), reference)
            errors["reuse"] = accuracy(torch, reuse(), reference)
            del reference
            sparse = {"coverage": pattern.coverage, "pattern_index_mib": pattern.index_bytes / 1024**2,
                      "retained_mass_target": 0.99, "measured_retained_mass": pattern.measured_retained_mass,
                      "exact_construction_recall": measure_pattern_recall(q0, k0, pattern),
                      "current_recall": measure_pattern_recall(drifted_q, drifted_k, pattern)}
        else:
            sparse = {"coverage": pattern.coverage, "pattern_index_mib": pattern.index_bytes / 1024**2,
                      "retained_mass_target": 0.99, "measured_retained_mass": pattern.measured_retained_mass,
                      "exact_construction_recall": float("nan"), "current_recall": float("nan")}
        for name, method in methods.items():
            add_record(case, shape, seed, "video_blocks", "normal", mode, name, timing[name], errors[name],
                       peak_memory(torch, method) if with_quality else None, None if name == "dense" else sparse)
    summaries = {summary["stage"]: summary for summary in summarize_records(RECORDS[first:])}
    row = {"N": length, "v_quantization": mode, "inputs": "two prototypes of norm 8 alternating per 128-token block, "
           "theta 0.99, drift 0.05 (the reference README's sparse table)", "seeds": list(seeds),
           "construct_ms": round(summaries["construct"]["median_ms"], 4),
           "dense_ms": round(summaries["dense"]["median_ms"], 4),
           "reuse_ms": round(summaries["reuse"]["median_ms"], 4),
           "coverage": round(summaries["reuse"]["coverage"], 4)}
    row["speedup"] = round(row["dense_ms"] / row["reuse_ms"], 3)
    if with_quality:
        row["sparse_sqnr_db"] = round(summaries["reuse"]["sqnr_db"], 2)
        row["dense_sqnr_db"] = round(summaries["dense"]["sqnr_db"], 2)
        row["exact_construction_recall"] = round(summaries["reuse"]["exact_construction_recall"], 5)
        row["current_recall"] = round(summaries["reuse"]["current_recall"], 5)
        row["construct_peak_mib"] = round(summaries["construct"]["peak_incremental_mib"], 1)
    return row


def workload_sparse_blocks(torch, risa, args, device):
    """The sparse table of the reference's README (README.md:127-142): about half of the key
    tiles carry the mass of every query block."""
    rows = []
    for length in ([args.length] if args.length else (1024, 2048, 4096, 8192, 16384, 32768)):
        for mode in ("absmax", "midpoint_affine"):
            rows.append(sparse_blocks_case(torch, risa, length, mode, SEEDS, args.samples, args.method_warmup, device))
    return rows


def workload_prepare(torch, risa, args, device):
    """Q/K/V preparation alone at the headline head counts: the one-call entry point
    (merged launches) against risa_quantize_qk + risa_quantize_v (one launch per kernel)."""
    from risaattention_amd import native
    from risaattention_amd.policy import DTYPE_CODES

    lib = native.library()
    rows = []
    batch, q_heads, kv_heads, dim = SHAPE["batch"], SHAPE["q_heads"], SHAPE["kv_heads"], SHAPE["head_dim"]
    for length in ([args.length] if args.length else (1024, 4096, 32768)):
        q, k, v = make_inputs(torch, length, 0, device)
        for mode in ("absmax", "midpoint_affine"):
            affine = int(mode == "midpoint_affine")
            packed = risa.prequantize_int8_attention(q, k, v, v_quantization=mode)
            anchors = torch.empty(batch, kv_heads, dtype=torch.int32, device=device)
            workspace = torch.empty(max(1, lib.risa_quantize_v_workspace_bytes(batch, kv_heads, length, dim, affine)),
                                    dtype=torch.uint8, device=device)
            stream = native.current_stream(device)
            code = DTYPE_CODES[q.dtype]
            qk_args = (q.data_ptr(), packed.q.data_ptr(), packed.q_scale.data_ptr(), k.data_ptr(),
                       packed.k.data_ptr(), packed.k_scale.data_ptr())
            v_args = (v.data_ptr(), packed.v.data_ptr(), packed.v_scale.data_ptr(), packed.v_center.data_ptr(),
                      packed.v_tile_sum.data_ptr(), workspace.data_ptr(), workspace.numel())

            def separate():
                native.check(lib.risa_quantize_qk(*qk_args, batch, q_heads, length, kv_heads, length, dim,
                                                  packed.cta_k, *q.stride()[:3], *k.stride()[:3], code,
                                                  anchors.data_ptr(), None, stream))
                native.check(lib.risa_quantize_v(*v_args, batch, kv_heads, length, dim, packed.v.shape[-1],
                                                 packed.cta_k, *v.stride()[:3], code, affine, None, stream))

            def merged():
                native.check(lib.risa_sdpa_quantize(*qk_args, *v_args, batch, q_heads, length, kv_heads, length,
                                                    dim, packed.cta_k, *q.stride()[:3], *k.stride()[:3],
                                                    *v.stride()[:3], code, affine, anchors.data_ptr(), None, stream))

            in_bytes = (q.numel() + k.numel() + v.numel()) * q.element_size()
            out_bytes = q.numel() + k.numel() + v.numel()
            merged_ms = time_calls(torch, merged, 20)
            rows.append({"N": length, "v_quantization": mode,
                         "separate_ms": round(time_calls(torch, separate, 20), 4),
                         "merged_ms": round(merged_ms, 4),
                         "merged_gb_per_s": round((in_bytes + out_bytes) / (merged_ms * 1e-3) / 1e9, 1)})
    return rows


def workload_video(torch, risa, args, device):
    """Video-DiT-scale sampling loop: one construction, nine drifting reuses, packed-operand replay."""
    frames, per_frame, heads, dim = 21, 1560, 40, 128
    length = frames * per_frame
    generator = torch.Generator(device=device).manual_seed(0)
    position = torch.arange(length, device=device, dtype=torch.float32)
    frame, patch = (position // per_frame) / frames, (position % per_frame) / per_frame
    frequency = torch.arange(1, dim // 4 + 1, device=device, dtype=torch.float32)
    phase = torch.rand(heads, 1, dim // 4, generator=generator, device=device) * 6.2831853
    parts = []
    for coordinate in (frame, patch):
        angle = coordinate[None, :, None] * frequency[None, None, :] * 6.2831853 + phase
        parts += [torch.sin(angle), torch.cos(angle)]
    smooth = torch.cat(parts, dim=-1)[None] * 2.0  # [1, H, N, D]
    q32 = smooth + 0.5 * torch.randn(smooth.shape, generator=generator, device=device)
    k32 = smooth + 0.5 * torch.randn(smooth.shape, generator=generator, device=device)
    v32 = torch.randn(smooth.shape, generator=generator, device=device)
    del smooth
    q, k, v = q32.bfloat16(), k32.bfloat16(), v32.bfloat16()
    dense_ms = time_calls(torch, lambda: risa.int8_attention(q, k, v), 3, 1)
    construct_ms = time_calls(torch, lambda: risa.construct_sparse_int8_attention(q, k, v, theta=0.99), 2, 1)
    _, pattern = risa.construct_sparse_int8_attention(q, k, v, theta=0.99)
    reuse = []
    for _ in range(9):
        q32 += 0.03 * torch.randn(q32.shape, generator=generator, device=device)
        k32 += 0.03 * torch.randn(k32.shape, generator=generator, device=device)
        q, k = q32.bfloat16(), k32.bfloat16()
        reuse.append(time_calls(torch, lambda: risa.sparse_int8_attention(q, k, v, pattern), 2, 1))
    packed = risa.prequantize_int8_attention(q, k, v)
    prequantize_ms = time_calls(torch, lambda: risa.prequantize_int8_attention(q, k, v), 5, 1)
    replay_ms = time_calls(torch, lambda: risa.int8_attention_from_prequantized(packed), 3, 1)
    ops = dense_equivalent_ops(1, heads, length, length, dim)
    return {"N": length, "heads": heads, "dense_ms": round(dense_ms, 3), "dense_tops": round(ops / dense_ms / 1e9, 1),
            "construct_ms": round(construct_ms, 3), "reuse_ms_median": round(statistics.median(reuse), 3),
            "coverage": round(pattern.coverage, 4), "prequantize_ms": round(prequantize_ms, 3),
            "from_prequantized_ms": round(replay_ms, 3),
            "loop_speedup_vs_dense": round(10 * dense_ms / (construct_ms + sum(reuse)), 3)}


def empty_key_tiles(tiles, fraction):
    """Which key tiles a broadcast mask hides for a given empty fraction: the first
    ``int(tiles * fraction)`` of the order even tiles, then odd tiles, so that hidden and
    visible tiles interleave instead of forming a prefix (reference benchmarks/masks.py:60-66)."""
    order = list(range(0, tiles, 2)) + list(range(1, tiles, 2))
    return sorted(order[: int(tiles * fraction)])


def interleaved_key_mask(torch, k_len, head_dim, fraction, mask_dtype, device):
    """[1,1,1,Lk] key mask with whole key tiles hidden; boolean, or FP32 with -inf for hidden keys."""
    tile = 64 if head_dim <= 64 or k_len <= 1024 else 128
    visible = torch.ones(1, 1, 1, k_len, dtype=torch.bool, device=device)
    for index in empty_key_tiles(-(-k_len // tile), fraction):
        visible[..., index * tile : (index + 1) * tile] = False
    if mask_dtype == "fp32":
        return torch.zeros(visible.shape, dtype=torch.float32, device=device).masked_fill(~visible, float("-inf"))
    return visible


def workload_mask_tiles(torch, risa, args, device):
    """Broadcast key masks that hide 0 / 25 / 50 / 75 % of the key tiles, boolean and FP32: what
    skipping whole tiles saves.  With ``--baseline-library`` every call is also made through that
    second build in the same process: outputs compared first, then both timed in one rotating group
    (the protocol of reference benchmarks/masks.py:40-110 over compare_native.py:40-53)."""
    from risaattention_amd import native

    batch, q_heads, kv_heads, dim = SHAPE["batch"], SHAPE["q_heads"], SHAPE["kv_heads"], SHAPE["head_dim"]
    length = args.length or 4096
    fractions = args.empty_fraction or [0.0, 0.25, 0.5, 0.75]
    if any(not 0.0 <= fraction <= 1.0 for fraction in fractions):
        raise SystemExit("--empty-fraction must lie in [0, 1]")
    mask_dtypes = ("bool", "fp32") if args.mask_dtype == "both" else (args.mask_dtype,)
    modes = ("absmax", "midpoint_affine") if args.v_modes == "both" else (args.v_modes,)
    baseline = native.load_library(args.baseline_library) if args.baseline_library else None
    ops = dense_equivalent_ops(batch, q_heads, length, length, dim)
    case = case_label(batch, q_heads, kv_heads, length, length, dim)
    shape = dict(batch=batch, q_heads=q_heads, kv_heads=kv_heads, q_len=length, k_len=length, head_dim=dim)
    first = len(RECORDS)
    for seed in SEEDS:
        q, k, v = make_inputs(torch, length, seed, device)
        for mask_dtype in mask_dtypes:
            for fraction in fractions:
                mask = interleaved_key_mask(torch, length, dim, fraction, mask_dtype, device)
                reference = fp32_reference(torch, q, k, v, mask=mask)
                methods, errors, comparisons = {}, {}, {}
                for mode in modes:
                    call = lambda mode=mode: risa.int8_attention(q, k, v, attn_mask=mask, v_quantization=mode)
                    after = call()
                    errors[f"after/{mode}"] = accuracy(torch, after, reference)
                    methods[f"after/{mode}"] = call
                    if baseline is not None:
                        def through_baseline(call=call):
                            with native.using_library(baseline):
                                return call()

                        before = through_baseline()
                        torch.testing.assert_close(before, after, atol=0.002, rtol=0.01)
                        comparisons[mode] = {"bitwise_equal": torch.equal(before, after),
                                             "max_abs_difference": (before.float() - after.float()).abs().max().item()}
                        errors[f"before/{mode}"] = accuracy(torch, before, reference)
                        methods[f"before/{mode}"] = through_baseline
                timing = measure_methods(torch, methods, samples=args.samples, calls_per_sample=calls_for(ops),
                                         warmup=args.method_warmup)
                for name in methods:
                    label, mode = name.split("/")
                    add_record(case, shape, seed, "normal", "normal", mode, f"{label}/mask_{mask_dtype}_empty_{fraction}",
                               timing[name], errors[name])
                    RECORDS[-1].update(mask_empty_fraction=fraction, mask_dtype=mask_dtype, build=label,
                                       native_comparison=comparisons.get(mode))
                del reference
    return mask_tile_rows(RECORDS[first:], ops)


def mask_tile_rows(records, ops):
    """Summary rows of the mask-tile records: per (build, mask dtype, V mode, empty fraction) the
    median over the seeds of the per-seed medians, its ratio to the same method with nothing
    hidden, and the mean NRMSE."""
    rows = []
    for summary in summarize_records(records):
        members = [record for record in records if record["stage"] == summary["stage"]
                   and record["v_quantization"] == summary["v_quantization"]]
        rows.append({"build": members[0]["build"], "mask_dtype": members[0]["mask_dtype"],
                     "v_quantization": summary["v_quantization"], "empty_fraction": members[0]["mask_empty_fraction"],
                     "ms": round(summary["median_ms"], 4), "tops": round(ops / (summary["median_ms"] * 1e-3) / 1e12, 1),
                     "nrmse": None if summary["nrmse"] is None else round(summary["nrmse"], 5),
                     "bitwise_equal_to_baseline": (None if members[0]["native_comparison"] is None else
                                                   all(member["native_comparison"]["bitwise_equal"] for member in members))})
    for row in rows:
        full = [other["ms"] for other in rows if other["empty_fraction"] == 0.0 and
                all(other[key] == row[key] for key in ("build", "mask_dtype", "v_quantization"))]
        row["vs_nothing_hidden"] = round(row["ms"] / full[0], 3) if full else None
    return rows


def profile_range_names(stage, modes):
    """Names of the profiler ranges one pass of ``--workload profile_ranges`` opens, in order."""
    return [f"risa/{stage}/{mode}" for mode in modes]


def workload_profile_ranges(torch, risa, args, device):
    """Warmed calls inside named profiler ranges (torch.cuda.nvtx is rocTX on PyTorch-ROCm), for
    ``rocprofv3 --marker-trace --kernel-trace -- python3 bench.py --workload profile_ranges``.
    No latency is reported: durations under a profiler are not benchmark figures (reference
    benchmarks/profile_operators.py:1-66)."""
    length = args.length or 512
    modes = ("absmax", "midpoint_affine") if args.v_modes == "both" else (args.v_modes,)
    q, k, v = make_inputs(torch, length, 0, device)
    methods = {}
    for mode in modes:
        if args.stage == "attend":
            packed = risa.prequantize_int8_attention(q, k, v, v_quantization=mode)
            methods[mode] = lambda packed=packed: risa.int8_attention_from_prequantized(packed)
        elif args.stage == "quantize":
            methods[mode] = lambda mode=mode: risa.prequantize_int8_attention(q, k, v, v_quantization=mode)
        else:
            methods[mode] = lambda mode=mode: risa.int8_attention(q, k, v, v_quantization=mode)
    for method in methods.values():
        for _ in range(args.method_warmup):
            method()
    torch.cuda.synchronize()
    names = profile_range_names(args.stage, modes)
    for _ in range(args.calls):
        for name, method in zip(names, methods.values()):
            with torch.cuda.nvtx.range(name):
                method()
    torch.cuda.synchronize()
    return [{"N": length, "stage": args.stage, "range": name, "calls": args.calls, "warmup": args.method_warmup}
            for name in names]


def scaling_series(records):
    """What the scaling plot shows, from per-seed records: for every method (stage and V mode)
    and sequence length, the dense-equivalent TOPS of the median over the seeds of the per-seed
    median latencies and the mean SQNR (reference benchmarks/plot_scaling.py:66-75, 118-133:
    4*B*Hq*Lq*Lk*D operations whatever the method skips).  Only equal Q/K lengths are plotted."""
    series = {}
    for row in summarize_records([r for r in records if r["shape"]["q_len"] == r["shape"]["k_len"]]):
        shape = next(r["shape"] for r in records if r["case"] == row["case"])
        ops = dense_equivalent_ops(shape["batch"], shape["q_heads"], shape["q_len"], shape["k_len"], shape["head_dim"])
        label = f"{row['stage']}/{row['v_quantization']}"
        series.setdefault(label, []).append({"length": shape["q_len"], "tops": ops / (row["median_ms"] * 1e-3) / 1e12,
                                             "sqnr_db": row["sqnr_db"], "sqnr_db_std": None})
    for label, points in series.items():
        points.sort(key=lambda point: point["length"])
    return series


def plot_scaling(series, path, title):
    """Grouped bars over the sequence length: SQNR against FP32 SDPA on the left (methods that
    carry accuracy records), dense-equivalent throughput on the right."""
    import matplotlib

    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    lengths = sorted({point["length"] for points in series.values() for point in points})
    tick = lambda n: f"{n // 1024}K" if n % 1024 == 0 else str(n)
    figure, (left, right) = plt.subplots(1, 2, figsize=(15, 5.5))
    panels = ((left, "sqnr_db", "SQNR vs FP32 SDPA (dB, higher is better)", "Accuracy", "{:.1f}"),
              (right, "tops", "Dense-equivalent throughput (TOP/s)", "Speed", "{:.0f}"))
    for axis, metric, ylabel, name, text in panels:
        shown = {label: points for label, points in series.items() if any(p[metric] is not None for p in points)}
        width = 0.8 / max(1, len(shown))
        for index, (label, points) in enumerate(sorted(shown.items())):
            by_length = {p["length"]: p[metric] for p in points}
            heights = [by_length.get(n) or 0.0 for n in lengths]
            places = [x + (index - (len(shown) - 1) / 2) * width for x in range(len(lengths))]
            bars = axis.bar(places, heights, width, label=label, edgecolor="black", linewidth=0.8)
            for bar, height in zip(bars, heights):
                if height:
                    axis.annotate(text.format(height), (bar.get_x() + bar.get_width() / 2, height), xytext=(0, 4),
                                  textcoords="offset points", ha="center", va="bottom", rotation=90, fontsize=7)
        axis.set_xticks(range(len(lengths)), [tick(n) for n in lengths])
        axis.set_xlabel("Sequence length")
        axis.set_ylabel(ylabel)
        axis.set_title(name)
        axis.grid(axis="y", linewidth=0.5, alpha=0.6)
        axis.set_axisbelow(True)
        axis.margins(y=0.18)
        if shown:
            axis.legend(fontsize=7, loc="upper center", bbox_to_anchor=(0.5, -0.12), ncol=2 if len(shown) > 4 else len(shown))
    figure.suptitle(title)
    figure.tight_layout()
    path.parent.mkdir(parents=True, exist_ok=True)
    figure.savefig(path, dpi=130)
    plt.close(figure)


def kernel_time(torch, risa, packed, calls, warmup=2):
    """Milliseconds per launch of the attention kernel on prepared operands (events on the launch stream)."""
    stream = torch.cuda.current_stream()
    for _ in range(warmup):
        risa.int8_attention_from_prequantized(packed)
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record(stream)
    for _ in range(calls):
        risa.int8_attention_from_prequantized(packed)
    end.record(stream)
    end.synchronize()
    return begin.elapsed_time(end) / calls


def workload_clock(torch, risa, args, device):
    """The dense kernel on random and on all-zero operands, `--calls` launches each, twice over.  The
    instruction stream is the same (one data-dependent branch aside, taken in the first tiles of
    random data only), and so is the count of GPU clock cycles per launch (run under
    `rocprofv3 --pmc GRBM_GUI_ACTIVE --kernel-trace`); the time differs with the clock the part
    sustains while its matrix units switch real operands."""
    length = args.length or 32768
    q, k, v = make_inputs(torch, length, 0, device)
    operands = {
        "random": risa.prequantize_int8_attention(q, k, v, v_quantization=args.mode),
        "zeros": risa.prequantize_int8_attention(torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v),
                                                 v_quantization=args.mode),
    }
    rows = []
    for repeat in range(2):
        for name, packed in operands.items():
            rows.append({"operands": name, "repeat": repeat, "N": length, "calls": args.calls,
                         "kernel_ms": round(kernel_time(torch, risa, packed, args.calls, warmup=10), 4)})
    return rows


def cpu_baseline(length=1024, calls=15):
    """Oracle (numpy port of the quantised pipeline) on the host cores: the reference's own
    CPU-sized configuration (same heads and head dim as the headline, N=1024, seed 0,
    tensors drawn in the order q, k, v; about ten seconds of CPU work)."""
    import numpy as np
    import torch

    from oracle import pipeline

    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    generator = torch.Generator().manual_seed(0)
    shape_q = (SHAPE["batch"], SHAPE["q_heads"], length, SHAPE["head_dim"])
    shape_k = (SHAPE["batch"], SHAPE["kv_heads"], length, SHAPE["head_dim"])
    q = torch.randn(shape_q, generator=generator, dtype=torch.bfloat16).float().numpy()
    k = torch.randn(shape_k, generator=generator, dtype=torch.bfloat16).float().numpy()
    v = torch.randn(shape_k, generator=generator, dtype=torch.bfloat16).float().numpy()
    pipeline.int8_attention(q, k, v)  # warm-up
    samples = []
    for _ in range(calls):
        start = time.perf_counter()
        pipeline.int8_attention(q, k, v)
        samples.append(time.perf_counter() - start)
    seconds = statistics.median(samples)
    ops = dense_equivalent_ops(SHAPE["batch"], SHAPE["q_heads"], length, length, SHAPE["head_dim"])
    return {
        "value": ops / seconds / 1e12,
        "unit": "dense-equivalent TOPS",
        "ms": seconds * 1e3,
        "cores": threads,
        "kind": "port",
        "sample": f"numpy oracle, B=1 Hq=16 Hkv=4 N={length} D=128 bf16 absmax, median of {calls} calls",
    }


def dense_kernel_name(torch, length):
    """Which kernel an unmasked dense launch of this length takes (the 16-query kernel serves
    launches with no more 128-query workgroups than the GPU has compute units)."""
    workgroups = SHAPE["batch"] * SHAPE["q_heads"] * ((length + 127) // 128)
    units = torch.cuda.get_device_properties(0).multi_processor_count
    return "attention_narrow_kernel<128,128>" if workgroups <= units else "attention_kernel<128,128,fast>"


def write_records(torch, risa, args, rows):
    """One JSON file per run in the layout of reference benchmarks/common.py:321-360: per-seed
    records under `results` (read by the reference's report tool as they are), the summary rows
    of this run's JSON line under `summary`."""
    import hashlib
    from datetime import datetime, timezone

    from risaattention_amd import native

    digest = hashlib.sha256()
    for path in sorted((ROOT / "risaattention_amd").rglob("*")):
        if path.suffix in (".py", ".hip", ".hpp", ".h") or path.name == "Makefile":
            digest.update(path.relative_to(ROOT).as_posix().encode())
            digest.update(path.read_bytes())
    library = Path(native.library_path())
    config = {key: (str(value) if isinstance(value, Path) else value) for key, value in vars(args).items()
              if key not in ("output", "report", "csv", "markdown", "plot")}
    if args.baseline_library is not None:
        config["baseline_library_sha256"] = hashlib.sha256(Path(args.baseline_library).read_bytes()).hexdigest()
    paired = args.workload in ("sweep", "masked", "sparse_blocks", "mask_tiles")
    config["timing_order"] = "rotate-and-reverse" if paired else "back-to-back calls between two events"
    config["seeds"] = list(SEEDS) if paired else [0]
    payload = {
        "schema_version": 2,
        "suite": args.workload,
        "measured_at_utc": datetime.now(timezone.utc).isoformat(),
        "environment": {
            "gpu": torch.cuda.get_device_name(),
            "arch": torch.cuda.get_device_properties(0).gcnArchName,
            "hip": torch.version.hip,
            "versions": {"torch": torch.__version__},
            "package_path": risa.__file__,
            "source_sha256": digest.hexdigest(),
            "extension_sha256": hashlib.sha256(library.read_bytes()).hexdigest(),
        },
        "config": config,
        "reference": "FP32 PyTorch attention in query chunks",
        "results": RECORDS,
        "summary": rows if isinstance(rows, list) else [rows],
    }
    args.output.parent.mkdir(parents=True, exist_ok=True)
    args.output.write_text(json.dumps(payload, indent=2, allow_nan=True) + "\n")


def render_report(payload, csv_path=None):
    """Summary of a file written with --output (the role of reference benchmarks/report.py): one
    row per (case, method) with the median of the per-seed medians and the mean accuracy, as a
    Markdown table and optionally as CSV; suites without per-seed records print their summary rows."""
    import csv

    environment = payload["environment"]
    lines = [f"## {payload['suite']} — {environment['gpu']} ({environment.get('arch', '')}), {payload['measured_at_utc']}",
             f"timing: {payload['config'].get('timing_order')}, seeds {payload['config'].get('seeds')}"
             + (f", {payload['config'].get('samples')} samples per method and seed"
                if payload['config'].get('timing_order') == 'rotate-and-reverse' else "")
             + f"; reference: {payload['reference']}", ""]
    records = payload.get("results") or []
    if records and "timing" in records[0]:
        rows = summarize_records(records)
        names = ["case", "v_quantization", "stage", "seed_count", "median_ms", "p10_ms", "p90_ms", "nrmse", "sqnr_db",
                 "peak_incremental_mib", "coverage", "current_recall"]
        if csv_path is not None:
            csv_path.parent.mkdir(parents=True, exist_ok=True)
            with csv_path.open("w", newline="") as file:
                writer = csv.DictWriter(file, fieldnames=list(rows[0]))
                writer.writeheader()
                writer.writerows(rows)
    else:
        rows = payload.get("summary") or records
        names = [key for key, value in rows[0].items() if not isinstance(value, (list, dict))]
    def shown(value):
        return "" if value is None else f"{value:.5g}" if isinstance(value, float) else str(value)
    lines += ["| " + " | ".join(names) + " |", "|" + "---|" * len(names)]
    lines += ["| " + " | ".join(shown(row.get(name)) for name in names) + " |" for row in rows]
    return "\n".join(lines)


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=5)
    parser.add_argument("--length", type=int, default=None,
                        help="sequence length (default 32768 for dense; restricts sweep/sparse to one N)")
    parser.add_argument("--mode", default="absmax", choices=["absmax", "midpoint_affine"])
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-accuracy", action="store_true")
    parser.add_argument("--workload", default="dense",
                        choices=["dense", "sweep", "masked", "sparse", "sparse_blocks", "video", "prepare", "mask_tiles",
                                 "profile_ranges", "clock"],
                        help="dense = headline N=32K line (default); the others are the remaining benchmark "
                             "configurations of the reference, reported as one JSON line each")
    parser.add_argument("--samples", type=int, default=10, help="event-timed samples per method and seed (--workload)")
    parser.add_argument("--method-warmup", type=int, default=20, help="warm-up calls per method before its samples (--workload)")
    parser.add_argument("--no-side-measurements", action="store_true",
                        help="dense line only: skip config.sparse_reuse and config.masked")
    parser.add_argument("--output", type=Path, default=None, help="also write the records of a --workload run to this JSON file")
    parser.add_argument("--report", type=Path, default=None, help="print a file written with --output as a Markdown table and exit")
    parser.add_argument("--csv", type=Path, default=None, help="with --report: also write the summary rows as CSV")
    parser.add_argument("--markdown", type=Path, default=None, help="with --report: also write the table to this file")
    parser.add_argument("--plot", type=Path, default=None,
                        help="with --report: also draw SQNR and dense-equivalent TOPS over the sequence length (PNG)")
    parser.add_argument("--empty-fraction", action="append", type=float,
                        help="mask_tiles: fraction of key tiles hidden (repeatable; default 0, 0.25, 0.5, 0.75)")
    parser.add_argument("--mask-dtype", choices=("bool", "fp32", "both"), default="both", help="mask_tiles: mask element type")
    parser.add_argument("--v-modes", choices=("absmax", "midpoint_affine", "both"), default="both",
                        help="mask_tiles / profile_ranges: V quantisation modes to run")
    parser.add_argument("--baseline-library", type=Path, default=None,
                        help="mask_tiles: a second build of the C-ABI library to compare and time against")
    parser.add_argument("--stage", choices=("dense", "quantize", "attend"), default="dense", help="profile_ranges: what a range wraps")
    parser.add_argument("--calls", type=int, default=10, help="profile_ranges: ranges per V mode; clock: launches per operand set")
    parser.add_argument("--calibrate-copy", action="store_true",
                        help="only run a 1 GiB device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    args = parser.parse_args()
    if args.report is not None:
        payload = json.loads(args.report.read_text())
        table = render_report(payload, args.csv)
        if args.plot is not None:
            environment = payload["environment"]
            plot_scaling(scaling_series(payload.get("results") or []), args.plot,
                         f"{payload['suite']} - {environment['gpu']} ({environment.get('arch', '')})")
        if args.markdown is not None:
            args.markdown.parent.mkdir(parents=True, exist_ok=True)
            args.markdown.write_text(table + "\n")
        print(table)
        return
    if args.gpus != 1:
        print("bench.py measures one MI355X; this path uses no second GPU",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import risaattention_amd as risa
    from risaattention_amd import native

    native.library()
    if not risa.int8_attention_is_available():
        raise SystemExit("bench.py needs a gfx950 GPU and the built HIP extension")
    device = torch.device("cuda", 0)
    if args.calibrate_copy:
        source = torch.empty(1 << 30, dtype=torch.uint8, device=device).random_(0, 255)
        target = torch.empty_like(source)
        for _ in range(3):
            target.copy_(source)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "copy", "bytes_read": 1 << 30, "bytes_written": 1 << 30}))
        return
    if args.workload != "dense":
        runner = {"sweep": workload_sweep, "masked": workload_masked, "sparse": workload_sparse,
                  "video": workload_video, "prepare": workload_prepare,
                  "sparse_blocks": workload_sparse_blocks, "mask_tiles": workload_mask_tiles,
                  "profile_ranges": workload_profile_ranges, "clock": workload_clock}[args.workload]
        wall = time.perf_counter()
        rows = runner(torch, risa, args, device)
        if args.output is not None:
            write_records(torch, risa, args, rows)
        print(json.dumps({"metric": f"{args.workload} workload (see config.rows)", "value": None, "unit": "ms",
                          "n_gpus": 1, "steps": None, "warmup": None, "ms_per_step": None,
                          "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
                          "data": "synthetic", "wall_seconds": round(time.perf_counter() - wall, 1),
                          "config": {"workload": args.workload, "rows": rows}}))
        return
    length = args.length or 32768
    q, k, v = make_inputs(torch, length, 0, device)
    ops = dense_equivalent_ops(SHAPE["batch"], SHAPE["q_heads"], length, length, SHAPE["head_dim"])

    def step():
        return risa.int8_attention(q, k, v, v_quantization=args.mode)

    for _ in range(args.warmup):
        out = step()
    torch.cuda.synchronize()
    wall_start = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - wall_start) * 1e3 / args.steps

    # Attention kernel alone, timed with events on the launch stream; and once more on all-zero
    # operands: the same instructions in the same number of clock cycles, at the clock the part
    # holds when its multipliers switch no bits (see workload_clock).
    packed = risa.prequantize_int8_attention(q, k, v, v_quantization=args.mode)
    stream = torch.cuda.current_stream(device)
    kernel_ms = kernel_time(torch, risa, packed, args.steps)
    zero_ms = compiled_ms = None
    if not args.no_side_measurements:
        # the same launch through the compiler-scheduled tile loop (diagnostic switch of the library,
        # read at every launch): what the hand-scheduled loop is worth on this machine
        before = os.environ.get("RISA_COMPILED_LOOP")
        os.environ["RISA_COMPILED_LOOP"] = "1"
        try:
            compiled_ms = kernel_time(torch, risa, packed, args.steps)
        finally:
            if before is None:
                del os.environ["RISA_COMPILED_LOOP"]
            else:
                os.environ["RISA_COMPILED_LOOP"] = before
        zero_ms = kernel_time(torch, risa, risa.prequantize_int8_attention(
            torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v), v_quantization=args.mode), args.steps)
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record(stream)
    for _ in range(args.steps):
        risa.prequantize_int8_attention(q, k, v, v_quantization=args.mode)
    end.record(stream)
    end.synchronize()
    prepare_ms = begin.elapsed_time(end) / args.steps
    achieved_tops = ops / (kernel_ms * 1e-3) / 1e12

    result = {
        "metric": "dense-equivalent TOPS at N=32K Hq16/Hkv4/D128 BF16 (incl. Q/K/V preparation)",
        "value": ops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {
            "workload": f"dense int8_attention B=1 Hq=16 Hkv=4 N={length} D=128 bf16 {args.mode} non-causal",
            "attention_kernel_ms": kernel_ms,
            "prepare_ms": prepare_ms,
        },
        "roofline": {
            # The contract of this line names the roof the fraction is taken against; the
            # kernel's limiter on this hardware is the vector-instruction issue of the U8
            # softmax next to the matrix instructions (profiles/attention_dense_32k_counters.md).
            "bound": "mfma",
            "limited_by": "VALU issue of the softmax next to the MFMAs (they share the SIMD issue capacity), at the "
                          "clock the part sustains under this load: about 1.9 GHz against 2.4 GHz nominal "
                          "(profiles/attention_dense_32k_clock.md); kernel_ms_zero_inputs is the same launch on "
                          "all-zero operands, same cycle count at the full clock",
            "kernel_ms_compiled_loop": compiled_ms,
            "kernel_ms_compiled_loop_note": "RISA_COMPILED_LOOP=1: every tile through the compiler-scheduled loop of this "
                                            "build, which forms its copy offsets per tile and runs about 2.5 % behind the "
                                            "previous library's loop (an A/B of the two libraries on one machine: 5.44 "
                                            "against 5.15 ms)",
            "kernel_ms_zero_inputs": zero_ms,
            # same cycles at 2.4 GHz over the cycles at the sustained clock: an estimate of sustained / nominal clock
            "clock_ratio_estimate": None if zero_ms is None else zero_ms / kernel_ms,
            "achieved": achieved_tops,
            "peak": INT8_MFMA_PEAK_TOPS,
            "unit": "TOP/s",
            "frac": achieved_tops / INT8_MFMA_PEAK_TOPS,
            # not measured in this run: the figure recorded from rocprofv3 for this shape
            "traffic": ATTENTION_KERNEL_TRAFFIC_BYTES_32K if (length == 32768 and args.mode == "absmax") else None,
            "traffic_source": "recorded from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs "
                              "(profiles/attention_dense_32k_counters.md), bytes per launch",
            "kernel": dense_kernel_name(torch, length),
        },
    }
    if not args.no_side_measurements:
        del out
        result["config"]["sparse_reuse"] = sparse_blocks_case(
            torch, risa, length, args.mode, seeds=SEEDS, samples=10, method_warmup=3, device=device, with_quality=False)
        result["config"]["sparse_reuse"]["note"] = (
            "BASELINE config 4's own recipe (64 groups, centroid x 3) keeps 1.6 % of the tiles and is not this row: "
            "see --workload sparse")
        result["config"]["masked"] = workload_masked(torch, risa, args, device, dims=(128, 64), seeds=(0,), samples=4)
        if length == 32768:
            result["config"]["sweep"] = sweep_cells(torch, risa, device, skip=((32768, args.mode),))
        out = step()
    if not args.no_accuracy:
        reference = fp32_reference(torch, q, k, v)
        result["config"]["accuracy_vs_fp32_sdpa"] = accuracy(torch, out, reference)
        del reference
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
