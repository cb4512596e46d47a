#!/usr/bin/env python3
"""Headline benchmark: dense INT8 attention at N=32K, Hq16/Hkv4/D128, BF16, one MI355X.

A step is one ``int8_attention(q, k, v)`` call on inputs resident in HBM: Q/K/V
preparation plus the fused attention kernel, as the reference's latency figures
include quantisation (reference README.md:102-106).  The JSON line reports
dense-equivalent TOPS (4*B*Hq*Lq*Lk*D operations per call, reference
benchmarks/plot_scaling.py:66-75), the roofline fraction of the attention
kernel against the dense INT8 MFMA peak, and the numpy oracle timed on the host
cores on a bounded sample (N=1024) as the CPU baseline.
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
SHAPE = dict(batch=1, q_heads=16, kv_heads=4, head_dim=128)


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


def fp32_reference(torch, q, k, v, chunk=2048):
    """FP32 SDPA in query chunks (reference benchmarks/common.py:134-145)."""
    group = q.shape[1] // k.shape[1]
    kf = k.float().repeat_interleave(group, 1).transpose(-1, -2)
    vf = v.float().repeat_interleave(group, 1)
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    for start in range(0, q.shape[2], chunk):
        scores = q[:, :, start : start + chunk].float() @ kf * q.shape[-1] ** -0.5
        out[:, :, start : start + chunk] = torch.softmax(scores, dim=-1) @ vf
    return out


def accuracy(torch, actual, reference):
    error = actual.float() - reference
    rmse = error.pow(2).mean().sqrt().item()
    rms = reference.pow(2).mean().sqrt().item()
    nrmse = rmse / max(rms, 1e-12)
    return {"nrmse": nrmse, "sqnr_db": -20.0 * __import__("math").log10(max(nrmse, 1e-30))}


def cpu_baseline(length=1024, calls=3):
    """Oracle (numpy port of the quantised pipeline) on the host cores, N=1024."""
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


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=5)
    parser.add_argument("--length", type=int, default=32768)
    parser.add_argument("--mode", default="absmax", choices=["absmax", "midpoint_affine"])
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-accuracy", action="store_true")
    parser.add_argument("--calibrate-copy", action="store_true",
                        help="only run a 1 GiB device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py measures one MI355X; this path uses no second GPU (see DESIGN.md on sharding)",
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
    length = args.length
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

    # Attention kernel alone, timed with events on the launch stream.
    packed = risa.prequantize_int8_attention(q, k, v, v_quantization=args.mode)
    stream = torch.cuda.current_stream(device)
    for _ in range(2):
        risa.int8_attention_from_prequantized(packed)
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record(stream)
    for _ in range(args.steps):
        risa.int8_attention_from_prequantized(packed)
    end.record(stream)
    end.synchronize()
    kernel_ms = begin.elapsed_time(end) / args.steps
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
            "bound": "mfma",
            "achieved": achieved_tops,
            "peak": INT8_MFMA_PEAK_TOPS,
            "unit": "TOP/s",
            "frac": achieved_tops / INT8_MFMA_PEAK_TOPS,
            "traffic": None,
            "kernel": "attention_kernel<128,128,fast>",
        },
    }
    if not args.no_accuracy:
        reference = fp32_reference(torch, q, k, v)
        result["config"]["accuracy_vs_fp32_sdpa"] = accuracy(torch, out, reference)
        del reference
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
