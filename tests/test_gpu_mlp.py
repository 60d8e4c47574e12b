"""The dense MLP block in one call (berth_exl3_mlp: gate and up in one launch, SiLU
gating inside the down projection) against the CPU oracle, stage by stage, and
against the reference's four-call sequence (crates/berth-engine/src/mlp.rs:118-150)."""
import os
import subprocess

import numpy as np
import pytest
import torch

from berth_amd import kernels as K
from berth_amd import synth
from berth_amd.device import Exl3Linear, Gpu, MlpLayer
from oracle import oracle as O
from tests.gpu_util import close, host_f16, host_u16

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "berth_amd", "lib", "berth_host_check")


def _layer(gpu, H, I, bits, seed, rows):
    lins = [synth.linear(seed, H, I, bits), synth.linear(seed + 3, H, I, bits), synth.linear(seed + 6, I, H, bits)]
    mlp = MlpLayer(gpu, *(Exl3Linear(gpu, n, *l) for n, l in zip(("gate", "up", "down"), lins)), max_rows=rows)
    return lins, mlp


@pytest.mark.parametrize("rows,H,I,bits", [(1, 256, 384, 4), (3, 256, 384, 3), (8, 256, 384, 4), (1, 1024, 2816, 4),
                                           (2, 2048, 768, 2), (20, 256, 384, 4), (40, 512, 256, 5)])
def test_fused_mlp_stage_by_stage(rows, H, I, bits):
    launch = run_mlp_block(rows, H, I, bits)
    if rows <= 8:
        assert launch.count("exl3_gemv_kernel") == 2 and "pair" in launch and ",silu>" in launch
    elif I >= H:
        # gate and up as one bundle (one rotation launch, one dense launch), then the down projection
        assert launch.count("exl3_gemm_kernel") == 2 and "had_r_128_slabs_kernel" in launch and "silu_mul" in launch
    else:
        assert launch.count("exl3_gemm_kernel") == 3 and "silu_mul" in launch


def run_mlp_block(rows, H, I, bits):
    """One berth_exl3_mlp call checked stage by stage against the oracle; returns the launch text."""
    gpu = Gpu(0)
    (gate, up, down), mlp = _layer(gpu, H, I, bits, 9000 + rows, rows)
    x = (synth.activations(9100 + rows, rows, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    y = torch.zeros((rows, H), dtype=torch.float32, device=gpu.device)
    mlp.forward(gpu, gpu.upload(x.view(np.uint16)), y, rows=rows)
    gpu.synchronize()
    launch = K.last_launch()

    g_want, xh_want = O.linear(x, *gate, H, I, bits, 2)
    u_want, _ = O.linear(x, *up, H, I, bits, 2)
    g_got = host_f16(mlp.g)[:rows * I].reshape(rows, I)
    assert close(g_got, g_want.reshape(rows, I))[0] == 0
    if rows <= 8 or I >= H:
        # the rotated input is the gate's (its suh); above 8 rows with intermediate < hidden the up
        # projection, a launch of its own then, rewrites it with its own
        assert np.array_equal(host_u16(mlp.x_had)[:rows * H], xh_want.view(np.uint16).ravel())
    if rows <= 8:
        u_got = host_f16(mlp.u)[:rows * I].reshape(rows, I)
        assert close(u_got, u_want.reshape(rows, I))[0] == 0
        act = O.silu_mul(g_got, u_got).reshape(rows, I)            # from the GPU's own gate / up outputs
        # the activation the down projection formed, seen through its rotated copy: bit-exact
        assert np.array_equal(host_u16(mlp.act_had)[:rows * I],
                              O.had_rows_f16(act, down[1], True).view(np.uint16).ravel())
    else:
        act = host_f16(mlp.u)[:rows * I].reshape(rows, I)          # up_out holds the activation
        assert close(act, O.silu_mul(g_want, u_want).reshape(rows, I), rtol=4e-3, atol=2e-3)[0] == 0
    y_want, _ = O.linear(act, *down, I, H, bits, 2, out_fp32=True)
    assert close(y.cpu().numpy(), y_want.reshape(rows, H))[0] == 0
    return launch


def test_fused_mlp_equals_the_four_call_sequence_up_to_summation_order():
    gpu = Gpu(0)
    H, I = 1024, 2816
    _, mlp = _layer(gpu, H, I, 4, 9500, 1)
    x = (synth.activations(9501, 1, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    dx = gpu.upload(x.view(np.uint16))
    y_fused = torch.zeros(H, dtype=torch.float32, device=gpu.device)
    y_calls = torch.zeros(H, dtype=torch.float32, device=gpu.device)
    mlp.forward(gpu, dx, y_fused)
    mlp.forward(gpu, dx, y_calls, fused=False)
    gpu.synchronize()
    a, b = y_fused.cpu().numpy(), y_calls.cpu().numpy()
    assert np.abs(a - b).max() <= 2e-3 * np.abs(b).max()


@pytest.mark.parametrize("rows", [1, 5])
def test_cpp_mlp_forward_fused(tmp_path, rows):
    H, I, bits = 256, 384, 3
    trio = dict(gate=synth.linear(5000, H, I, bits), up=synth.linear(5003, H, I, bits), down=synth.linear(5006, I, H, bits))
    x = (synth.activations(5100 + rows, rows, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    for name, (tr, suh, svh) in trio.items():
        tr.tofile(tmp_path / f"{name}.trellis.bin")
        suh.view(np.uint16).tofile(tmp_path / f"{name}.suh.bin")
        svh.view(np.uint16).tofile(tmp_path / f"{name}.svh.bin")
    x.view(np.uint16).tofile(tmp_path / "x.bin")
    (tmp_path / "meta.txt").write_text(f"{H} {I} {rows} 1\n")
    r = subprocess.run([EXE, "mlp", str(tmp_path)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "fused=1" in r.stdout and "pair" in r.stdout, r.stdout + r.stderr
    y = np.fromfile(tmp_path / "y.bin", dtype=np.float32).reshape(rows, H)
    g, _ = O.linear(x, *trio["gate"], H, I, bits, 2)
    u, _ = O.linear(x, *trio["up"], H, I, bits, 2)
    want, _ = O.linear(O.silu_mul(g, u).reshape(rows, I), *trio["down"], I, H, bits, 2, out_fp32=True)
    assert np.abs(y - want.reshape(rows, H)).max() <= 2e-3 * np.abs(want).max()


def _block_inputs(gpu, H, rows, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, H)).astype(np.float32)
    res = (3.0 * rng.standard_normal((rows, H))).astype(np.float32)
    w = (0.1 * rng.standard_normal(H)).astype(np.float32)
    w_bf16 = (w.view(np.uint32) >> 16).astype(np.uint16)          # truncated: any bf16 pattern will do
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu.device)
    return up(x), up(res), torch.from_numpy(w_bf16.view(np.int16)).to(gpu.device)


@pytest.mark.parametrize("rows,H,I,bits,fused", [(1, 2048, 12288, 3, "both"), (1, 1024, 2816, 4, "none"),
                                                  (3, 256, 384, 4, "none"), (20, 256, 384, 4, "none")])
def test_mlp_block_call_equals_norm_mlp_add_as_separate_calls(rows, H, I, bits, fused):
    """berth_exl3_mlp_block against berth_ops_rms_norm_res_in -> berth_exl3_mlp -> berth_ops_add_f32
    on the same inputs: the residual stream, the rotated input of gate / up (hence the norm's
    fp16 output) and the gate / up outputs bit for bit; the block's output bit for bit where
    the launches are the same, and within the summation-order bound otherwise."""
    from berth_amd.device import ptr
    gpu = Gpu(0)
    _, mlp = _layer(gpu, H, I, bits, 9700 + rows, rows)
    x, res, w = _block_inputs(gpu, H, rows, 9800 + rows)
    eps = 1e-6
    # the separate calls
    res_ref = res.clone()
    h = torch.zeros((rows, H), dtype=torch.float16, device=gpu.device)
    K.ops.rms_norm_res_in(ptr(x), ptr(w), ptr(h), ptr(res_ref), rows, H, eps, 1.0, 1.0, True, gpu.raw_stream())
    y_ref = torch.zeros((rows, H), dtype=torch.float32, device=gpu.device)
    mlp.forward(gpu, h, y_ref, rows=rows)
    K.ops.add_f32(ptr(y_ref), ptr(res_ref), ptr(y_ref), rows * H, gpu.raw_stream())
    gpu.synchronize()
    xh_ref, g_ref, u_ref = host_u16(mlp.x_had)[:rows * H].copy(), host_u16(mlp.g)[:rows * I].copy(), host_u16(mlp.u)[:rows * I].copy()
    mlp.x_had.zero_(); mlp.g.zero_(); mlp.u.zero_()
    # the block call
    res_out = torch.zeros_like(res)
    y = torch.zeros((rows, H), dtype=torch.float32, device=gpu.device)
    mlp.forward_block(gpu, x, res, res_out, w, y, epsilon=eps, rows=rows)
    gpu.synchronize()
    launch = K.last_launch()
    assert ("pair,norm" in launch) == (fused == "both") and ("+residual" in launch) == (fused == "both"), launch
    assert np.array_equal(res_out.cpu().numpy().view(np.uint32), res_ref.cpu().numpy().view(np.uint32))
    if rows <= 8:
        assert np.array_equal(host_u16(mlp.x_had)[:rows * H], xh_ref)
        assert np.array_equal(host_u16(mlp.g)[:rows * I], g_ref) and np.array_equal(host_u16(mlp.u)[:rows * I], u_ref)
    a, b = y.cpu().numpy(), y_ref.cpu().numpy()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), float(np.abs(a - b).max())
