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
over `--layers` distinct weight sets (default 10 = 1.7 GB) so that reads come
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
# Figures of the default workload that only a profiler run can give, each tied to the launches
# it was taken on (profiles/exl3_gemv_4bpw_batch1_27b_linear_set.md): HBM bytes per launch from
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a 1 GiB copy, and vector instructions per
# weight from --pmc SQ_INSTS_VALU (wave instructions * 64 lanes / weights).  bench.py prints them
# only when the launches of the run are the ones the profile was taken on.
PROFILE = {
    4: {"launches": ["sliced x8 by value exl3_gemv_stream_kernel<4,2,table=0x0>",
                     "exl3_gemv_stream_kernel<4,2,table=0x0>",
                     "sliced x2 by value exl3_gemv_stream_kernel<4,2,table=0x0>",
                     "exl3_gemv_stream_kernel<4,2,table=0x0>"],
        "traffic_bytes_per_launch": int((42265 + 892) * 1024),
        "valu_instr_per_weight": 5.0},
}
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
        if dt >= seconds:
            break
    nbytes = linear_bytes(K, N, bits, 1, 2) * reps
    res = {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": O.num_threads(), "kind": "port",
           "sample": f"{reps} x q_proj {K}x{N} {bits} bpw batch-1 decode-on-the-fly GEMV in {dt:.1f} s "
                     f"({K * N * reps / dt / 1e6:.0f} M weights/s)"}

    def timed(fn, budget):
        fn()
        n, t0 = 0, time.perf_counter()
        while True:
            fn()
            n += 1
            el = time.perf_counter() - t0
            if el >= budget:
                return el / n, n

    # the other CPU figures of the same port, a few seconds each: BASELINE configs[0]
    # (4096 x 4096, 4 bpw) as a GEMV and as a dequantisation, configs[3] at one token
    k0 = 4096
    tr0, suh0, svh0 = synth.linear(13, k0, k0, 4)
    x0 = synth.activations(14, 1, k0)
    t_gemv0, n_gemv0 = timed(lambda: O.gemv_fused(x0, tr0, suh0, svh0, k0, k0, 4, 2, out_fp32=False), 2.0)
    t_deq, n_deq = timed(lambda: O.dequant(tr0, k0, k0, 4, 2), 2.0)
    H, E, topk, I = 2048, 128, 8, 768
    distinct = [tuple(synth.linear(2000 + 10 * e + 3 * j, *shape, 4) for j, shape in enumerate(((H, I), (H, I), (I, H))))
                for e in range(8)]
    experts = [distinct[e % 8] for e in range(E)]       # 8 distinct synthetic experts repeated: timing only
    wr = synth.router_weight(15, H, E)
    xm = synth.activations(16, 1, H)
    t_moe, n_moe = timed(lambda: O.moe_layer(xm, wr, experts, topk, I, 4, 2), 3.0)
    res["also"] = {
        "config0_gemv_ms": round(t_gemv0 * 1e3, 3), "config0_gemv_GBps": round(linear_bytes(k0, k0, 4, 1, 2) / t_gemv0 / 1e9, 3),
        "config0_dequant_Gweights_per_s": round(k0 * k0 / t_deq / 1e9, 3),
        "moe_config3_one_token_us_per_token": round(t_moe * 1e6, 1),
        "sample": f"{n_gemv0} GEMVs and {n_deq} dequantisations of 4096x4096 at 4 bpw, {n_moe} one-token MoE layers "
                  f"(128 experts, top-8; 8 distinct synthetic experts repeated)"}
    return res


def time_steps(gpu, step, steps: int, warmup: int, graph: bool = True, run=None):
    """Time exactly `steps` steps two ways: launched one by one (eager), and recorded once into
    a HIP graph that holds all `steps` steps and is replayed (the library's launches keep no
    host state between calls, so a recorded step replays bit for bit).  Each way: (wall ms,
    device ms between two events on the launch stream).  The graph pair is None when recording
    is switched off.  `run(n)`, when given, issues n steps on the current stream from compiled
    code (bench_native.hip), as the reference's engine does; otherwise step(i) is called from
    this interpreter, whose own time per call then shows in the eager wall time."""
    import torch

    def timed(go):
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        go()
        e1.record()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3, e0.elapsed_time(e1)

    issue = run if run is not None else (lambda n: [step(i) for i in range(n)])
    for i in range(warmup):
        step(i)
    issue(max(1, warmup))
    eager = sorted((timed(lambda: issue(steps)) for _ in range(3)), key=lambda t: t[0])[1]
    if not graph:
        return eager, None
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=gpu.device)
    side.wait_stream(torch.cuda.current_stream(gpu.device))
    with torch.cuda.stream(side):
        step(0)
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=side):
            issue(steps)
    torch.cuda.current_stream(gpu.device).wait_stream(side)
    g.replay()                                          # untimed: the first replay uploads the graph
    runs = sorted((timed(g.replay) for _ in range(3)), key=lambda t: t[1])
    return eager, runs[1]                               # the median of three replays


class NativeCalls:
    """A prepared sequence of C-ABI calls (bench_native.hip's BenchCall records) that
    berth_bench_run issues on the current stream: `per_step` calls per step, rotating over
    `distinct` steps."""

    def __init__(self, gpu, per_step: int):
        import ctypes

        class BenchCall(ctypes.Structure):
            _fields_ = [("kind", ctypes.c_int), ("i", ctypes.c_int * 12), ("p", ctypes.c_void_p * 12)]

        self._type, self._calls, self._keep = BenchCall, [], []
        self.gpu, self.per_step, self.lib, self._array = gpu, per_step, native(), None

    def linear(self, lin, a, c, out_fp32: bool):
        from berth_amd.device import ptr
        call = self._type()
        call.kind = 0
        for j, v in enumerate((ptr(a), ptr(lin.trellis), ptr(c), ptr(lin.suh), ptr(lin.a_had), ptr(lin.svh))):
            call.p[j] = v
        for j, v in enumerate((1, lin.size_k, lin.size_n, lin.k_bits, int(lin.codebook), int(out_fp32))):
            call.i[j] = v
        self._calls.append(call)

    def bundle(self, multi, a, outs, out_fp32: bool):
        """One sliced multi-linear with its lists by value (Exl3MultiLinear's host copies)."""
        from berth_amd.device import ptr
        from berth_amd.kernels import OutDtype
        multi.forward(self.gpu, a, outs, OutDtype.F32 if out_fp32 else OutDtype.F16)     # fixes the output list
        h = multi._h
        call = self._type()
        call.kind = 1 if multi.host_lists else 2
        lists = (h["b"], h["suh"], h["svh"], h["size_n"], multi._h_c, h["stride"], h["src"]) if multi.host_lists else None
        if lists is None:
            dv = (multi.b_list, multi.suh_list, multi.svh_list, multi.size_n_list, multi._c_ptrs, multi.n_stride_list,
                  multi.had_src_list)
            addr = [ptr(t) for t in dv]
            self._keep.append(dv)
        else:
            addr = [x.ctypes.data for x in lists]
            self._keep.append(lists)
        for j, v in enumerate((ptr(a), addr[0], ptr(outs[0]), addr[1], ptr(multi.a_had), addr[2], addr[3], addr[4],
                               addr[5], addr[6])):
            call.p[j] = v
        for j, v in enumerate((1, multi.size_k, multi.width, multi.k_bits, int(multi.codebook), int(out_fp32), 1,
                               multi.slices, len(multi.sources))):
            call.i[j] = v
        self._calls.append(call)

    def mlp(self, layer, x, y):
        """berth_exl3_mlp on one row (MlpLayer's buffers)."""
        import ctypes
        from berth_amd.device import ptr
        from berth_amd.kernels import Exl3Lin
        layer.forward(self.gpu, x, y, fused=True)           # allocates the layer's rotated-input buffers
        lins = (Exl3Lin * 3)(*[Exl3Lin(ptr(l.trellis), ptr(l.suh), ptr(l.svh)) for l in (layer.gate, layer.up, layer.down)])
        self._keep.append(lins)
        call = self._type()
        call.kind = 3
        for j, v in enumerate((ptr(x), ctypes.addressof(lins), ptr(layer.g), ptr(layer.u), ptr(layer.x_had),
                               ptr(layer.act_had), ptr(y))):
            call.p[j] = v
        for j, v in enumerate((1, layer.hidden, layer.intermediate, layer.gate.k_bits, int(layer.gate.codebook))):
            call.i[j] = v
        self._calls.append(call)

    def mlp_block(self, layer, x32, res, res_out, norm_w, y):
        """berth_exl3_mlp_block on one row (epsilon 1e-6, bias 1, scale 1, bf16 norm weight)."""
        import ctypes
        from berth_amd.device import ptr
        from berth_amd.kernels import Exl3Lin, RmsNorm
        layer.forward_block(self.gpu, x32, res, res_out, norm_w, y)      # allocates the layer's scratch
        lins = (Exl3Lin * 3)(*[Exl3Lin(ptr(l.trellis), ptr(l.suh), ptr(l.svh)) for l in (layer.gate, layer.up, layer.down)])
        norm = RmsNorm(ptr(norm_w), 1e-6, 1.0, 1.0, 1)
        self._keep += [lins, norm]
        call = self._type()
        call.kind = 5
        for j, v in enumerate((ptr(x32), ptr(res), ptr(res_out), ctypes.addressof(norm), ctypes.addressof(lins),
                               ptr(layer.h_norm), ptr(layer.g), ptr(layer.u), ptr(layer.x_had), ptr(layer.act_had), ptr(y))):
            call.p[j] = v
        for j, v in enumerate((1, layer.hidden, layer.intermediate, layer.gate.k_bits, int(layer.gate.codebook))):
            call.i[j] = v
        self._calls.append(call)

    def raw(self, kind: int, pointers, ints):
        from berth_amd.device import ptr
        call = self._type()
        call.kind = kind
        for j, t in enumerate(pointers):
            call.p[j] = ptr(t)
        for j, v in enumerate(ints):
            call.i[j] = v
        self._calls.append(call)

    def silu_mul(self, gate, up, out, numel: int):
        from berth_amd.device import ptr
        call = self._type()
        call.kind = 4
        for j, v in enumerate((ptr(gate), ptr(up), ptr(out))):
            call.p[j] = v
        call.i[0] = numel
        self._calls.append(call)

    def run(self, steps: int):
        import ctypes
        if self._array is None:
            self._array = (self._type * len(self._calls))(*self._calls)
        rc = self.lib.berth_bench_run(ctypes.addressof(self._array), self.per_step, len(self._calls) // self.per_step,
                                      steps, self.gpu.raw_stream())
        if rc != 0:
            from berth_amd import kernels as Kn
            raise RuntimeError(f"native step loop: call {rc - 1} failed: {Kn.last_error() or Kn.ops.last_error()}")


def native():
    """libberth_bench.so: bench.py's own compiled helpers (bench_native.hip)."""
    import ctypes
    lib = ctypes.CDLL(os.path.join(ROOT, "libberth_bench.so"))
    lib.berth_probe_valu.restype = ctypes.c_int
    lib.berth_probe_valu.argtypes = [ctypes.c_double, ctypes.POINTER(ctypes.c_double)]
    lib.berth_bench_run.restype = ctypes.c_int
    lib.berth_bench_run.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    return lib


def valu_ceiling(bits: int, instr_per_weight):
    """The vector-ALU bound of the decode, measured live: lane-instructions per second of the
    decode's instruction mix, from an idle device (the clock a 10 - 30 us launch sees) and after
    250 ms of back-to-back launches (the clock a long launch settles at), over the vector
    instructions the GEMV kernel issues per weight (from the profile; None when the run's
    launches are not the profile's)."""
    import ctypes
    out = (ctypes.c_double * 2)()
    if native().berth_probe_valu(250.0, out) != 0:
        return None
    cus = 256
    res = {"unit": "T lane-instr/s", "instr_per_weight": instr_per_weight}
    for name, rate in (("boost", out[0]), ("sustained", out[1])):
        d = {"lane_instr_per_s": round(rate / 1e12, 2), "implied_clock_GHz": round(rate / (cus * 64) / 1e9, 3)}
        if instr_per_weight:
            d["weights_per_s"] = round(rate / instr_per_weight / 1e12, 2)
            d["implied_GBps"] = round(rate / instr_per_weight * bits / 8 / 1e9, 1)
            d["implied_frac_of_hbm_peak"] = round(rate / instr_per_weight * bits / 8 / 1e9 / HBM_PEAK_GBS, 4)
        res[name] = d
    return res


def moe_plan_bytes(H: int, E: int, k: int, I: int, bits: int, shared_I: int = 0):
    """Bytes of one MoE layer by the reference's placement model (crates/berth-plan/src/place.rs:345-376),
    through the planner this build ships: the layer's tensors are listed under the names a checkpoint
    gives them, `is_routed_expert` splits them into backbone (router, shared expert) and expert pool, and
    `bytes_moved` = backbone + pool * k / E is what one decoded token reads.  Returns (backbone, pool,
    bytes_moved).  A configuration without a shared expert lists none of its tensors; the plan record
    still needs a non-zero width for it."""
    from berth_amd import plan as P

    def linear_bytes(kk, nn):                      # trellis + fp16 suh + svh
        return kk * nn * bits // 8 + 2 * (kk + nn)

    mlp = "model.language_model.layers.0.mlp"
    tensors = [(f"{mlp}.gate.weight", 2 * H * E)]
    for e in range(E):
        tensors += [(f"{mlp}.experts.{e}.gate_proj", linear_bytes(H, I)), (f"{mlp}.experts.{e}.up_proj", linear_bytes(H, I)),
                    (f"{mlp}.experts.{e}.down_proj", linear_bytes(I, H))]
    if shared_I:
        tensors += [(f"{mlp}.shared_expert.gate_proj", linear_bytes(H, shared_I)),
                    (f"{mlp}.shared_expert.up_proj", linear_bytes(H, shared_I)),
                    (f"{mlp}.shared_expert.down_proj", linear_bytes(shared_I, H))]
    shape = P.ModelShape(P.ARCH_QWEN3_5_MOE, 1, [P.LayerKind.FULL_ATTENTION], H, 256, 16, 2, P.GdnDims(16, 32, 128, 128, 4),
                         P.MoeDims(E, k, I, shared_I or I), 248_320)
    listed = P.TensorBytes(tensors)
    placed = P.place(P.build_plan(shape), listed)
    pool = sum(b for n, b in listed.tensors if P.is_routed_expert(n))
    return listed.total() - pool, pool, placed.bytes_moved


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
    backbone, pool, moved = moe_plan_bytes(H, E, k, I, bits)
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
        eager_us = dt / steps * 1e6
        launch = "eager"
        # the same 16 calls recorded once into a HIP graph and replayed (the library's launches
        # keep no host state between calls, so a recorded layer replays bit for bit)
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(device=gpu.device)
        side.wait_stream(torch.cuda.current_stream(gpu.device))
        with torch.cuda.stream(side):
            for i in range(16):
                layers[i % 2].forward(gpu, xs[i], out, T)
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for i in range(16):
                    layers[i % 2].forward(gpu, xs[i], out, T)
        torch.cuda.current_stream(gpu.device).wait_stream(side)
        replays = max(2, steps // 16)
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        graph_us = (time.perf_counter() - t0) / (replays * 16) * 1e6
        if graph_us < eager_us:
            dt, launch = graph_us * 1e-6 * steps, "hip graph of 16 layers"
        # one token: the placement model's bytes_moved; a batch reads each expert it hits once
        weights = moved if T == 1 else backbone + pool * hit / E
        nbytes = weights + 2 * T * H + 4 * T * H
        res[f"T{T}"] = {"us_per_layer": round(dt / steps * 1e6, 2), "us_per_token": round(dt / steps / T * 1e6, 3),
                        "experts_hit": round(hit, 1), "algorithmic_GBps": round(nbytes * steps / dt / 1e9, 1),
                        "launch": launch, "eager_us_per_layer": round(eager_us, 2)}
    res["config"] = "hidden 2048, 128 experts, top-8, intermediate 768, 4 bpw, mul1"
    res["bytes_model"] = {"backbone": backbone, "expert_pool": pool, "bytes_moved_per_token": moved,
                          "source": "berth_amd.plan.place (place.rs:345-376)"}
    return res


def moe_large_bench(gpu, steps: int, resident_layers: int = 48):
    """BASELINE.json configs[4]: hidden 2048, 512 experts top-10 plus one always-on
    shared expert, intermediate 512, 3 bpw, 256 tokens, router logits biased so
    that expert popularity is Zipf(1.1); the weights of 48 such layers (29 GB)
    stay resident in HBM and the steps rotate over them.  Weights are generated
    on the device (uniform random trellis words, sign x lognormal(0, 0.1) scales)."""
    import torch

    from berth_amd import synth
    from berth_amd.device import Exl3Linear
    from berth_amd.moe import MoeLayer

    T, H, E, k, I, bits = 256, 2048, 512, 10, 512, 3
    g = torch.Generator(device=gpu.device)
    g.manual_seed(4242)
    words = (H // 16) * (I // 16) * 16 * bits          # u16 words of one expert linear
    a_had = torch.zeros(H, dtype=torch.float16, device=gpu.device)

    def scales(n):
        sign = torch.randint(0, 2, (n,), generator=g, device=gpu.device).float() * 2 - 1
        return (sign * torch.exp(0.1 * torch.randn(n, generator=g, device=gpu.device))).half()

    layers = []
    for li in range(resident_layers):
        slab = torch.randint(0, 65536, ((E + 1) * 3, words), generator=g, device=gpu.device,
                             dtype=torch.int32).to(torch.int16)
        su = scales((E + 1) * 3 * H).view((E + 1) * 3, H)      # rows of H; the I-sized vectors use a prefix
        sv = scales((E + 1) * 3 * H).view((E + 1) * 3, H)
        experts = []
        for e in range(E + 1):
            trio = []
            for j, (kk, nn) in enumerate(((H, I), (H, I), (I, H))):
                r = 3 * e + j
                trio.append(Exl3Linear.from_device(f"layers.{li}.experts.{e}.{j}", slab[r], su[r, :kk], sv[r, :nn],
                                                   bits, a_had=a_had))
            experts.append(tuple(trio))
        layers.append(MoeLayer(gpu, synth.router_weight(900 + li, H, E), experts[:E], k, shared=experts[E],
                               bias=synth.zipf_bias(950 + li, E)))
    resident = sum(l.trellis_bytes() for l in layers)
    xs = [gpu.upload(synth.activations(700 + i, T, H).view(np.uint16)) for i in range(8)]
    out = torch.zeros((T, H), dtype=torch.float32, device=gpu.device)
    idx = torch.zeros((T, k), dtype=torch.int32, device=gpu.device)
    hit, hottest = 0.0, 0
    for i in range(8):
        layers[i % len(layers)].forward(gpu, xs[i], out, T, idx)
        c = np.bincount(idx.cpu().numpy().ravel(), minlength=E)
        hit += float((c > 0).sum()) / 8
        hottest = max(hottest, int(c.max()))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        layers[i % len(layers)].forward(gpu, xs[i % 8], out, T)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    eager_us, launch = dt * 1e6, "eager"
    # one pass over the resident layers recorded into a HIP graph and replayed
    n = len(layers)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=gpu.device)
    side.wait_stream(torch.cuda.current_stream(gpu.device))
    with torch.cuda.stream(side):
        for i in range(n):
            layers[i].forward(gpu, xs[i % 8], out, T)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for i in range(n):
                layers[i].forward(gpu, xs[i % 8], out, T)
    torch.cuda.current_stream(gpu.device).wait_stream(side)
    replays = max(2, steps // n)
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(replays):
        graph.replay()
    torch.cuda.synchronize()
    graph_dt = (time.perf_counter() - t0) / (replays * n)
    if graph_dt < dt:
        dt, launch = graph_dt, f"hip graph of {n} layers"
    backbone, pool, moved = moe_plan_bytes(H, E, k, I, bits, shared_I=I)
    nbytes = backbone + pool * hit / E + 2 * T * H + 4 * T * H
    flops = 2.0 * (T * k + T) * 3 * H * I
    return {"config": "hidden 2048, 512 experts top-10 + shared expert, intermediate 512, 3 bpw, 256 tokens, "
                      "Zipf(1.1) router bias, mul1",
            "resident_layers": len(layers), "resident_weight_GB": round(resident / 1e9, 2),
            "us_per_layer": round(dt * 1e6, 1), "us_per_token": round(dt / T * 1e6, 3),
            "launch": launch, "eager_us_per_layer": round(eager_us, 1),
            "experts_hit": round(hit, 1), "hottest_expert_rows": hottest,
            "bytes_model": {"backbone": backbone, "expert_pool": pool, "bytes_moved_per_token": moved,
                            "source": "berth_amd.plan.place (place.rs:345-376)"},
            "algorithmic_GBps": round(nbytes / dt / 1e9, 1), "tflops": round(flops / dt / 1e12, 2)}


def bpw_sweep(gpu, rates, steps: int, nlayers: int = 8):
    """BASELINE.json configs[1] at the other bit rates of its sweep: the same four
    launches per step over device-generated weights, GB/s of algorithmic bytes."""
    import torch

    from berth_amd import synth
    from berth_amd.device import Exl3Linear, Exl3MultiLinear
    from berth_amd.kernels import OutDtype

    g = torch.Generator(device=gpu.device)
    g.manual_seed(99)
    xin = {K: gpu.upload(synth.activations(5, 1, K).view(np.uint16)) for K in (5120, 6144, 17408)}
    outs = {n: torch.zeros(synth.SHAPES_27B[n][1], dtype=torch.float32 if OUT_FP32[n] else torch.float16,
                           device=gpu.device) for n in ORDER}
    res = {}
    for bits in rates:
        layers = []
        for li in range(nlayers):
            lin = {}
            for name in ORDER:
                K, N = synth.SHAPES_27B[name]
                tr = torch.randint(0, 65536, (K * N * bits // 16,), generator=g, device=gpu.device,
                                   dtype=torch.int32).to(torch.int16)
                sc = [((torch.randint(0, 2, (n,), generator=g, device=gpu.device).float() * 2 - 1)
                       * torch.exp(0.1 * torch.randn(n, generator=g, device=gpu.device))).half() for n in (K, N)]
                lin[name] = Exl3Linear.from_device(f"layers.{li}.{name}", tr, sc[0], sc[1], bits)
            lin["qkv"] = Exl3MultiLinear(gpu, [lin["q_proj"], lin["k_proj"], lin["v_proj"]])
            lin["gate_up"] = Exl3MultiLinear(gpu, [lin["gate_proj"], lin["up_proj"]])
            layers.append(lin)

        def step(i):
            lin = layers[i % nlayers]
            lin["qkv"].forward(gpu, xin[5120], [outs["q_proj"], outs["k_proj"], outs["v_proj"]], OutDtype.F16)
            lin["o_proj"].forward(gpu, xin[6144], outs["o_proj"], OutDtype.F32)
            lin["gate_up"].forward(gpu, xin[5120], [outs["gate_proj"], outs["up_proj"]], OutDtype.F16)
            lin["down_proj"].forward(gpu, xin[17408], outs["down_proj"], OutDtype.F32)

        calls = NativeCalls(gpu, 4)
        for lin in layers:
            calls.bundle(lin["qkv"], xin[5120], [outs["q_proj"], outs["k_proj"], outs["v_proj"]], False)
            calls.linear(lin["o_proj"], xin[6144], outs["o_proj"], True)
            calls.bundle(lin["gate_up"], xin[5120], [outs["gate_proj"], outs["up_proj"]], False)
            calls.linear(lin["down_proj"], xin[17408], outs["down_proj"], True)
        (e_wall, e_dev), graphed = time_steps(gpu, step, steps, 10, run=calls.run)
        dt = e_wall * 1e-3 / steps                      # eager, issued from compiled code: the headline's mode
        nbytes = sum(linear_bytes(*synth.SHAPES_27B[n], bits, 1, 4 if OUT_FP32[n] else 2) for n in ORDER)
        res[f"{bits}bpw"] = {"GBps": round(nbytes / dt / 1e9, 1), "us_per_step": round(dt * 1e6, 2),
                             "frac_of_hbm_peak": round(nbytes / dt / 1e9 / HBM_PEAK_GBS, 4),
                             "Gweights_per_s": round(340787200 / dt / 1e9, 1), "launch": "eager",
                             "eager_device_us_per_step": round(e_dev * 1e3 / steps, 2),
                             "graph_device_us_per_step": None if graphed is None else round(graphed[1] * 1e3 / steps, 2)}
        del calls
        del layers
        torch.cuda.empty_cache()
    return res


def lm_head_bench(gpu, steps: int):
    """The largest single GEMV of the 27B checkpoint: lm_head, K = 5120, N = 248320
    at 6 bpw with the mul1 codebook and fp16 logits (trellis [320, 15520, 96],
    953,548,800 bytes: crates/berth-exl3/tests/qwen38_27b.rs:66-76,
    crates/berth-kernels/csrc/gemm_k6.cu:1-3).  Two device-generated copies are
    alternated so that no launch finds its weights in a cache."""
    import torch

    from berth_amd import synth
    from berth_amd.device import Exl3Linear
    from berth_amd.kernels import OutDtype

    K, N, bits = 5120, 248320, 6
    g = torch.Generator(device=gpu.device)
    g.manual_seed(606)
    heads = []
    for li in range(2):
        tr = torch.randint(0, 65536, (K * N * bits // 16,), generator=g, device=gpu.device,
                           dtype=torch.int32).to(torch.int16)
        sc = [((torch.randint(0, 2, (n,), generator=g, device=gpu.device).float() * 2 - 1)
               * torch.exp(0.1 * torch.randn(n, generator=g, device=gpu.device))).half() for n in (K, N)]
        heads.append(Exl3Linear.from_device(f"lm_head.{li}", tr, sc[0], sc[1], bits))
    x = gpu.upload(synth.activations(6, 1, K).view(np.uint16))
    out = torch.zeros(N, dtype=torch.float16, device=gpu.device)
    for i in range(4):
        heads[i % 2].forward(gpu, x, out, OutDtype.F16)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        heads[i % 2].forward(gpu, x, out, OutDtype.F16)
    e1.record()
    torch.cuda.synchronize()
    dt = e0.elapsed_time(e1) * 1e-3 / steps
    nbytes = linear_bytes(K, N, bits, 1, 2)
    from berth_amd import kernels as Kn
    return {"config": "K 5120, N 248320, 6 bpw, mul1, batch 1, fp16 logits", "bytes": nbytes,
            "us_per_launch": round(dt * 1e6, 1), "GBps": round(nbytes / dt / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / dt / 1e9 / HBM_PEAK_GBS, 4),
            "Gweights_per_s": round(K * N / dt / 1e9, 1), "kernel": Kn.last_launch()}


def mlp_block_bench(gpu, layers, bits: int, steps: int):
    """One dense MLP block of the 27B shapes (hidden 5120, intermediate 17408) for one
    token: berth_exl3_mlp (gate and up in one launch, SiLU gating inside the down
    projection: two launches) beside the reference's four calls
    (crates/berth-engine/src/mlp.rs:118-150), rotating over the resident layers."""
    import torch

    from berth_amd import synth
    from berth_amd.device import MlpLayer

    H, I = synth.SHAPES_27B["gate_proj"]
    mlps = [MlpLayer(gpu, lin["gate_proj"], lin["up_proj"], lin["down_proj"]) for lin in layers]
    x = gpu.upload((synth.activations(11, 1, H).astype(np.float32) / np.sqrt(H)).astype(np.float16).view(np.uint16))
    y = torch.zeros(H, dtype=torch.float32, device=gpu.device)
    nbytes = 2 * linear_bytes(H, I, bits, 1, 2) + linear_bytes(I, H, bits, 1, 4)
    res = {"config": f"hidden {H}, intermediate {I}, {bits} bpw, mul1, batch 1", "bytes": nbytes,
           "launch": "eager, issued by the compiled host loop"}
    # the block with the glue either side of it: residual add + RMS norm ahead, residual add behind
    x32 = torch.randn(H, device=gpu.device, dtype=torch.float32)
    resid = torch.randn(H, device=gpu.device, dtype=torch.float32)
    res_out = torch.zeros_like(resid)
    h16 = torch.zeros(H, dtype=torch.float16, device=gpu.device)
    norm_w = torch.zeros(H, dtype=torch.int16, device=gpu.device)          # bf16 zeros: weight + 1 = 1
    for name, fused in (("one_call", True), ("four_calls", False), ("block_one_call", "block"),
                        ("block_norm_mlp_add_calls", "glue")):
        calls = NativeCalls(gpu, {True: 1, False: 4, "block": 1, "glue": 3}[fused])
        for m in mlps:
            if fused == "block":
                calls.mlp_block(m, x32, resid, res_out, norm_w, y)
            elif fused == "glue":
                calls.raw(6, (x32, norm_w, h16, res_out), (1, H))           # rms_norm_res_in (in place on res_out)
                calls.mlp(m, h16, y)
                calls.raw(7, (y, res_out, y), (H,))                         # add_f32
            elif fused:
                calls.mlp(m, x, y)
            else:
                calls.linear(m.gate, x, m.g, False)
                calls.linear(m.up, x, m.u, False)
                calls.silu_mul(m.g, m.u, m.u, I)
                calls.linear(m.down, m.u, y, True)
        calls.run(len(mlps))
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            calls.run(steps)
            e1.record()
            torch.cuda.synchronize()
            dt = e0.elapsed_time(e1) * 1e-3 / steps
            best = dt if best is None else min(best, dt)
        dt = best
        res[name] = {"us_per_block": round(dt * 1e6, 2), "GBps": round(nbytes / dt / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / dt / 1e9 / HBM_PEAK_GBS, 4)}
    return res


def prefill_bench(gpu, layers, bits: int, rows: int, steps: int):
    """BASELINE.json configs[2]: the same 27B-shaped linears at `rows` = 512 tokens,
    fp16 activations N(0,1), fp16/fp32 outputs with fp32 accumulation: seven calls of
    berth_prefill_exl3_linear (Hadamard pre-pass + decode-in-GEMM MFMA kernel), and the same
    work with q/k/v and gate/up as bundles (berth_ops_mgemm: one rotation launch and one dense
    MFMA launch per bundle), which is what the decode benchmark's four launches do at one row."""
    import torch

    from berth_amd import synth
    from berth_amd.device import RowScratch
    from berth_amd.kernels import OutDtype

    scratch = RowScratch(gpu, rows, 17408, 17408)
    xin = {K: gpu.upload(synth.activations(9, rows, K).view(np.uint16)) for K in (5120, 6144, 17408)}
    outs = {n: torch.zeros((rows, synth.SHAPES_27B[n][1]), dtype=torch.float32 if OUT_FP32[n] else torch.float16,
                           device=gpu.device) for n in ORDER}
    flops = sum(2.0 * rows * K * N for K, N in (synth.SHAPES_27B[n] for n in ORDER))

    def step_seven(i):
        lin = layers[i % len(layers)]
        for n in ORDER:
            l = lin[n]
            l.forward_rows(gpu, scratch, xin[l.size_k], outs[n], rows, OutDtype.F32 if OUT_FP32[n] else OutDtype.F16)

    def step_bundles(i):
        # q/k/v and gate/up share their inputs: each group is one berth_ops_mgemm call (lists by value)
        lin = layers[i % len(layers)]
        lin["qkv"].forward(gpu, xin[5120], [outs["q_proj"], outs["k_proj"], outs["v_proj"]], OutDtype.F16, rows)
        l = lin["o_proj"]
        l.forward_rows(gpu, scratch, xin[l.size_k], outs["o_proj"], rows, OutDtype.F32 if OUT_FP32["o_proj"] else OutDtype.F16)
        lin["gate_up"].forward(gpu, xin[5120], [outs["gate_proj"], outs["up_proj"]], OutDtype.F16, rows)
        l = lin["down_proj"]
        l.forward_rows(gpu, scratch, xin[l.size_k], outs["down_proj"], rows,
                       OutDtype.F32 if OUT_FP32["down_proj"] else OutDtype.F16)

    def timed(step):
        for i in range(3):
            step(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            step(i)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        eager_ms, launch = dt * 1e3, "eager"
        # one pass over the rotated weight sets recorded into a HIP graph and replayed
        n = len(layers)
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(device=gpu.device)
        side.wait_stream(torch.cuda.current_stream(gpu.device))
        with torch.cuda.stream(side):
            for i in range(n):
                step(i)
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for i in range(n):
                    step(i)
        torch.cuda.current_stream(gpu.device).wait_stream(side)
        replays = max(2, steps // n)
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        graph_dt = (time.perf_counter() - t0) / (replays * n)
        if graph_dt < dt:
            dt, launch = graph_dt, f"hip graph of {n} layer sets"
        return dt, eager_ms, launch

    seven_dt, seven_eager_ms, seven_launch = timed(step_seven)
    bundled = all("qkv" in lin and "gate_up" in lin for lin in layers) and all(
        not OUT_FP32[n] for n in ("q_proj", "k_proj", "v_proj", "gate_proj", "up_proj"))
    if bundled:
        dt, eager_ms, launch = timed(step_bundles)
        calls = "four calls: q/k/v and gate/up as berth_ops_mgemm bundles, o and down berth_prefill_exl3_linear"
    else:
        dt, eager_ms, launch = seven_dt, seven_eager_ms, seven_launch
        calls = "seven calls of berth_prefill_exl3_linear"

    # Beside it: the vendor library's dense fp16 GEMM (torch.matmul) on already
    # decoded fp16 weights of the same seven shapes.  It reads 4x the weight bytes
    # and decodes nothing; it shows what a plain MFMA GEMM reaches at 512 rows of
    # these shapes on this device, i.e. the practical ceiling for the fused kernel.
    dense_us = 0.0
    for n in ORDER:
        Kk, N = synth.SHAPES_27B[n]
        a = torch.randn((rows, Kk), device=gpu.device, dtype=torch.float16)
        ws = [torch.randn((Kk, N), device=gpu.device, dtype=torch.float16) for _ in range(3)]
        c = torch.empty((rows, N), device=gpu.device, dtype=torch.float16)
        for i in range(3):
            torch.matmul(a, ws[i], out=c)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(12):
            torch.matmul(a, ws[i % 3], out=c)
        e1.record()
        torch.cuda.synchronize()
        dense_us += e0.elapsed_time(e1) / 12 * 1e3
        del a, ws, c
    torch.cuda.empty_cache()
    return {"rows": rows, "ms_per_layer_set": round(dt * 1e3, 3), "tflops": round(flops / dt / 1e12, 1),
            "mfma_peak_tflops": 2500.0, "frac_of_fp16_mfma_peak": round(flops / dt / 2.5e15, 4),
            "tokens_per_s": round(rows / dt, 0), "launch": launch, "calls": calls,
            "eager_ms_per_layer_set": round(eager_ms, 3),
            "seven_calls": {"ms_per_layer_set": round(seven_dt * 1e3, 3), "tflops": round(flops / seven_dt / 1e12, 1),
                            "launch": seven_launch},
            "vendor_dense_fp16_gemm": {"what": "torch.matmul on decoded fp16 weights, same shapes and rows",
                                       "ms_per_layer_set": round(dense_us * 1e-3, 3),
                                       "tflops": round(flops / dense_us / 1e6, 1)}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=10)
    ap.add_argument("--bits", type=int, default=4)
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-moe", action="store_true")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-lm-head", action="store_true")
    ap.add_argument("--no-mlp", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only")
    ap.add_argument("--no-valu", action="store_true", help="skip the vector-ALU rate probe")
    ap.add_argument("--moe-resident-layers", type=int, default=48)
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

    # the launch texts of one step, in order (what the profile's figures are tied to)
    launch_texts = []
    lin = layers[0]
    if args.unfused:
        for name in ORDER:
            lin[name].forward(gpu, xin[lin[name].size_k], outs[name], f32 if OUT_FP32[name] else f16)
            launch_texts.append(Kn.last_launch())
    else:
        lin["qkv"].forward(gpu, xin[5120], [outs["q_proj"], outs["k_proj"], outs["v_proj"]], f16)
        launch_texts.append(Kn.ops.last_launch())
        lin["o_proj"].forward(gpu, xin[6144], outs["o_proj"], f32)
        launch_texts.append(Kn.last_launch())
        lin["gate_up"].forward(gpu, xin[5120], [outs["gate_proj"], outs["up_proj"]], f16)
        launch_texts.append(Kn.ops.last_launch())
        lin["down_proj"].forward(gpu, xin[17408], outs["down_proj"], f32)
        launch_texts.append(Kn.last_launch())
    kernels_run = [t.split(" grid=")[0] for t in launch_texts]
    prof = PROFILE.get(bits)
    prof_applies = bool(prof) and not args.unfused and kernels_run == prof["launches"]

    # the same steps as prepared C-ABI calls for the compiled launch loop
    calls = NativeCalls(gpu, launches_per_step)
    for lin in layers:
        if args.unfused:
            for name in ORDER:
                calls.linear(lin[name], xin[lin[name].size_k], outs[name], OUT_FP32[name])
        else:
            calls.bundle(lin["qkv"], xin[5120], [outs["q_proj"], outs["k_proj"], outs["v_proj"]], False)
            calls.linear(lin["o_proj"], xin[6144], outs["o_proj"], True)
            calls.bundle(lin["gate_up"], xin[5120], [outs["gate_proj"], outs["up_proj"]], False)
            calls.linear(lin["down_proj"], xin[17408], outs["down_proj"], True)

    (eager_wall_ms, eager_ev_ms), graphed = time_steps(gpu, step, args.steps, args.warmup, graph=not args.no_graph,
                                                       run=calls.run)
    # The headline is the eager figure: launches issued one by one from compiled code, as the
    # reference's engine issues them.  The graph replay of the same launches is reported beside it.
    ms_per_step = eager_wall_ms / args.steps
    value = step_bytes * args.steps / (eager_wall_ms * 1e-3) / 1e9
    launches = args.steps * launches_per_step
    avg_launch_us = eager_ev_ms * 1e3 / launches
    achieved = step_bytes * args.steps / (eager_ev_ms * 1e-3) / 1e9

    def leg(pair):
        return {"GBps": round(step_bytes * args.steps / (pair[0] * 1e-3) / 1e9, 1),
                "us_per_step": round(pair[0] * 1e3 / args.steps, 2),
                "device_us_per_step": round(pair[1] * 1e3 / args.steps, 2),
                "frac_of_hbm_peak": round(step_bytes * args.steps / (pair[1] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

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
                   "launch": "eager: one C-ABI call per launch, issued by a compiled host loop (bench_native.hip)",
                   "launches_per_step": launch_texts,
                   "eager": leg((eager_wall_ms, eager_ev_ms)),
                   "graph": None if graphed is None else leg(graphed),
                   "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2)},
        # priced against the HBM peak, as the metric asks; what limits the kernel is the vector
        # ALU's decode arithmetic (limited_by, valu_ceiling), not the memory system
        "roofline": {"bound": "hbm", "limited_by": "vector ALU (trellis decode arithmetic)",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": prof["traffic_bytes_per_launch"] if prof_applies else None,
                     "profile_applies": prof_applies,
                     "kernel": kernels_run[-1],
                     "avg_launch_us": round(avg_launch_us, 3),
                     "bytes_per_launch": step_bytes // launches_per_step,
                     "valu_ceiling": None if args.no_valu else valu_ceiling(
                         bits, prof["valu_instr_per_weight"] if prof_applies else None)},
    }
    if not args.no_sweep:
        line["bpw_sweep"] = bpw_sweep(gpu, [b for b in (2, 3, 4, 5) if b != bits], max(20, args.steps // 2))
        line["bpw_sweep"][f"{bits}bpw"] = {"GBps": line["value"], "us_per_step": round(ms_per_step * 1e3, 2),
                                          "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
                                          "Gweights_per_s": round(340787200 / ms_per_step / 1e6, 1)}
    if not args.no_mlp:
        line["mlp_block"] = mlp_block_bench(gpu, layers, bits, args.steps)
    if not args.no_prefill:
        line["prefill_gemm"] = prefill_bench(gpu, layers, bits, 512, 10)
    if not args.no_moe or not args.no_lm_head:
        del layers
        torch.cuda.empty_cache()
    if not args.no_lm_head:
        line["lm_head"] = lm_head_bench(gpu, 40)
        torch.cuda.empty_cache()
    if not args.no_moe:
        line["moe_layer"] = moe_bench(gpu, max(20, args.steps // 2), max(5, args.warmup // 2))
        torch.cuda.empty_cache()
        line["moe_large_layer"] = moe_large_bench(gpu, 96, args.moe_resident_layers)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(bits, args.cpu_seconds)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
