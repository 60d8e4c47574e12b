#!/usr/bin/env python3
"""Benchmark of the EXL3 trellis GEMV hot path on one MI355X.

Workload (BASELINE.json configs[1] at the bit rate the metric is quoted on): the
dense 27B-shaped decode linear set at batch 1, 4 bpw, mul1 codebook — q_proj
5120x6144, k/v_proj 5120x1024, o_proj 6144x5120, gate/up 5120x17408, down
17408x5120 — fp16 activations N(0,1), uniform random trellis words, suh/svh
random signs times lognormal(0,0.1).  One step = the seven linears of one layer in
four launches: q/k/v as one sliced multi-linear (berth_ops_mgemm, as the
reference bundles them), o_proj (berth_exl3_linear), gate+up as one multi-linear,
down_proj.  Steps rotate
over `--layers` distinct weight sets (default 8 = 1.36 GB) so that reads come
from HBM, not from the 256 MB memory-side cache.  Inputs are resident in HBM
before the timed region.

value = algorithmic bytes of the step / time, in GB/s (the metric's unit);
roofline.achieved is the same quantity for the dominant kernel (all seven
launches are the one GEMV kernel), against the 8 TB/s HBM peak.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per GEMV launch of the default workload, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs scaled by a 1 GiB copy (profiles/exl3_gemv_4bpw_batch1_27b_linear_set.md)
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {4: int((24589 + 428) * 1024)}
ORDER = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
OUT_FP32 = {"q_proj": False, "k_proj": False, "v_proj": False, "o_proj": True,
            "gate_proj": False, "up_proj": False, "down_proj": True}


def linear_bytes(K, N, bits, m, out_bytes):
    """Algorithmic bytes of one linear on m rows: packed trellis + suh + svh +
    activation in + output out."""
    return K * N * bits // 8 + 2 * K + 2 * N + 2 * m * K + out_bytes * m * N


def cpu_baseline(bits: int, seconds: float):
    """The CPU oracle's decode-on-the-fly GEMV (a port: the reference has no CPU
    trellis path), timed on this host's cores on a bounded sample."""
    from berth_amd import synth
    from oracle import oracle as O
    K, N = synth.SHAPES_27B["q_proj"]
    tr, suh, svh = synth.linear(11, K, N, bits)
    x = synth.activations(12, 1, K)
    O.gemv_fused(x, tr, suh, svh, K, N, bits, 2, out_fp32=False)       # warm (builds the state table)
    reps, t0 = 0, time.perf_counter()
    while True:
        O.gemv_fused(x, tr, suh, svh, K, N, bits, 2, out_fp32=False)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= seconds or reps >= 200:
            break
    nbytes = linear_bytes(K, N, bits, 1, 2) * reps
    return {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": O.num_threads(), "kind": "port",
            "sample": f"{reps} x q_proj {K}x{N} {bits} bpw batch-1 decode-on-the-fly GEMV in {dt:.1f} s "
                      f"({K * N * reps / dt / 1e6:.0f} M weights/s)"}


def moe_bench(gpu, steps: int, warmup: int):
    """BASELINE.json configs[3]: hidden 2048, 128 experts, top-8 softmax routing,
    expert intermediate 768, 4 bpw, router fp16 N(0, 0.02); batch 1 and 64.  One
    call = route + permute + grouped gate/up + SiLU gate + grouped down + combine."""
    import torch

    from berth_amd import synth
    from berth_amd.device import Exl3Linear
    from berth_amd.moe import MoeLayer

    H, E, k, I, bits = 2048, 128, 8, 768, 4
    layers = []
    for li in range(2):
        experts = []
        for e in range(E):
            s = 100000 * (li + 1) + 10 * e
            experts.append(tuple(Exl3Linear(gpu, f"layers.{li}.experts.{e}.{n}", *synth.linear(s + 3 * j, *shape, bits))
                                 for j, (n, shape) in enumerate((("gate_proj", (H, I)), ("up_proj", (H, I)),
                                                                 ("down_proj", (I, H))))))
        layers.append(MoeLayer(gpu, synth.router_weight(77 + li, H, E), experts, k))
    expert_bytes = 3 * H * I * bits // 8 + 2 * (2 * (H + I) + (I + H))
    res = {}
    for T in (1, 64):
        xs = [gpu.upload(synth.activations(300 + i, T, H).view(np.uint16)) for i in range(16)]
        out = torch.zeros((T, H), dtype=torch.float32, device=gpu.device)
        idx = torch.zeros((T, k), dtype=torch.int32, device=gpu.device)
        hit = 0
        for i in range(16):
            layers[i % 2].forward(gpu, xs[i], out, T, idx)
            hit += len(np.unique(idx.cpu().numpy()))
        hit /= 16.0
        for i in range(warmup):
            layers[i % 2].forward(gpu, xs[i % 16], out, T)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            layers[i % 2].forward(gpu, xs[i % 16], out, T)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        nbytes = 2 * H * E + hit * expert_bytes + 2 * T * H + 4 * T * H
        res[f"T{T}"] = {"us_per_layer": round(dt / steps * 1e6, 2), "us_per_token": round(dt / steps / T * 1e6, 3),
                        "experts_hit": round(hit, 1), "algorithmic_GBps": round(nbytes * steps / dt / 1e9, 1)}
    res["config"] = "hidden 2048, 128 experts, top-8, intermediate 768, 4 bpw, mul1"
    return res


def prefill_bench(gpu, layers, bits: int, rows: int, steps: int):
    """BASELINE.json configs[2]: the same 27B-shaped linears at `rows` = 512 tokens,
    fp16 activations N(0,1), fp16/fp32 outputs with fp32 accumulation, through
    berth_prefill_exl3_linear (Hadamard pre-pass + decode-in-GEMM MFMA kernel)."""
    import torch

    from berth_amd import synth
    from berth_amd.device import RowScratch
    from berth_amd.kernels import OutDtype

    scratch = RowScratch(gpu, rows, 17408, 17408)
    xin = {K: gpu.upload(synth.activations(9, rows, K).view(np.uint16)) for K in (5120, 6144, 17408)}
    outs = {n: torch.zeros((rows, synth.SHAPES_27B[n][1]), dtype=torch.float32 if OUT_FP32[n] else torch.float16,
                           device=gpu.device) for n in ORDER}
    flops = sum(2.0 * rows * K * N for K, N in (synth.SHAPES_27B[n] for n in ORDER))

    def step(i):
        lin = layers[i % len(layers)]
        for n in ORDER:
            l = lin[n]
            l.forward_rows(gpu, scratch, xin[l.size_k], outs[n], rows, OutDtype.F32 if OUT_FP32[n] else OutDtype.F16)

    for i in range(3):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    return {"rows": rows, "ms_per_layer_set": round(dt * 1e3, 3), "tflops": round(flops / dt / 1e12, 1),
            "mfma_peak_tflops": 2500.0, "frac_of_fp16_mfma_peak": round(flops / dt / 2.5e15, 4),
            "tokens_per_s": round(rows / dt, 0)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=8)
    ap.add_argument("--bits", type=int, default=4)
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-moe", action="store_true")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--unfused", action="store_true", help="seven separate launches instead of four")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain 1 GiB device copy kernel a few times (reference reading for "
                         "the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path is single-GPU by design); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from berth_amd import kernels as Kn
    from berth_amd import synth
    from berth_amd.device import Exl3Linear, Exl3MultiLinear, Gpu
    from berth_amd.kernels import OutDtype

    Kn.load()
    gpu = Gpu(0)
    bits = args.bits

    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device=gpu.device)     # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4,
                                               "launches": 4}}))
        return

    layers = []
    for li in range(args.layers):
        lin = {}
        for j, name in enumerate(ORDER):
            K, N = synth.SHAPES_27B[name]
            tr, suh, svh = synth.linear(1000 * li + 10 * j, K, N, bits)
            lin[name] = Exl3Linear(gpu, f"layers.{li}.{name}", tr, suh, svh)
        if not args.unfused:
            lin["qkv"] = Exl3MultiLinear(gpu, [lin["q_proj"], lin["k_proj"], lin["v_proj"]])
            lin["gate_up"] = Exl3MultiLinear(gpu, [lin["gate_proj"], lin["up_proj"]])
        layers.append(lin)

    xin = {K: gpu.upload(synth.activations(5, 1, K).view(np.uint16)) for K in (5120, 6144, 17408)}
    outs = {name: torch.zeros(synth.SHAPES_27B[name][1], dtype=torch.float32 if OUT_FP32[name] else torch.float16,
                              device=gpu.device) for name in ORDER}

    step_bytes = sum(linear_bytes(*synth.SHAPES_27B[n], bits, 1, 4 if OUT_FP32[n] else 2) for n in ORDER)

    f16, f32 = OutDtype.F16, OutDtype.F32
    launches_per_step = len(ORDER) if args.unfused else 4

    def step(i):
        lin = layers[i % len(layers)]
        if args.unfused:
            for name in ORDER:
                l = lin[name]
                l.forward(gpu, xin[l.size_k], outs[name], f32 if OUT_FP32[name] else f16)
            return
        lin["qkv"].forward(gpu, xin[5120], [outs["q_proj"], outs["k_proj"], outs["v_proj"]], f16)
        lin["o_proj"].forward(gpu, xin[6144], outs["o_proj"], f32)
        lin["gate_up"].forward(gpu, xin[5120], [outs["gate_proj"], outs["up_proj"]], f16)
        lin["down_proj"].forward(gpu, xin[17408], outs["down_proj"], f32)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(args.steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ev_ms = e0.elapsed_time(e1)
    ms_per_step = wall_ms / args.steps
    value = step_bytes * args.steps / (wall_ms * 1e-3) / 1e9

    launches = args.steps * launches_per_step
    avg_launch_us = ev_ms * 1e3 / launches
    achieved = step_bytes * args.steps / (ev_ms * 1e-3) / 1e9

    line = {
        "metric": "trellis GEMV HBM GB/s at 4 bpw, batch 1",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"27B-shaped decode linear set (q,k,v,o,gate,up,down), batch 1, {bits} bpw, mul1",
                   "layers_rotated": len(layers), "bytes_per_step": step_bytes,
                   "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get(bits) if len(layers) == 8 and not args.unfused else None,
                     "kernel": Kn.last_launch().split(" grid=")[0],
                     "avg_launch_us": round(avg_launch_us, 3),
                     "bytes_per_launch": step_bytes // launches_per_step},
    }
    if not args.no_prefill:
        line["prefill_gemm"] = prefill_bench(gpu, layers, bits, 512, 10)
    if not args.no_moe:
        del layers
        torch.cuda.empty_cache()
        line["moe_layer"] = moe_bench(gpu, max(20, args.steps // 2), max(5, args.warmup // 2))
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(bits, args.cpu_seconds)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
