"""GPU parity of the MoE layer against the CPU oracle, through the C ABI.
Bars: logits, top-k expert indices, offsets and the permutation are bit-exact;
routing weights within 1e-5; layer outputs within rtol 2e-3 / atol 1e-3."""
import numpy as np
import pytest
import torch

from berth_amd import kernels as K
from berth_amd import synth
from berth_amd.device import Exl3Linear, Gpu
from berth_amd.device import InputError
from berth_amd.moe import MoeLayer
from oracle import oracle as O
from tests.gpu_util import DEV, close, dev, knobs

pytestmark = pytest.mark.gpu


def _route(x, wr, k, bias=None, renorm=True):
    T, H = x.shape
    E = wr.shape[1]
    d_x, d_w = dev(x.view(np.uint16)), dev(wr.view(np.uint16))
    d_b = None if bias is None else torch.from_numpy(bias).to(DEV)
    idx = torch.zeros((T, k), dtype=torch.int32, device=DEV)
    w = torch.zeros((T, k), dtype=torch.float32, device=DEV)
    logits = torch.zeros((T, E), dtype=torch.float32, device=DEV)
    parts = torch.zeros(T * ((H + 63) // 64) * E, dtype=torch.float32, device=DEV)
    K.moe.route(d_x.data_ptr(), d_w.data_ptr(), None if d_b is None else d_b.data_ptr(), idx.data_ptr(),
                w.data_ptr(), logits.data_ptr(), parts.data_ptr(), T, H, E, k, renorm)
    torch.cuda.synchronize()
    return idx.cpu().numpy(), w.cpu().numpy(), logits.cpu().numpy()


@pytest.mark.parametrize("T,H,E,k", [(1, 2048, 128, 8), (64, 2048, 128, 8), (5, 200, 16, 4), (3, 130, 7, 7),
                                     (256, 2048, 512, 10), (9, 64, 300, 10)])
def test_route_bit_exact(T, H, E, k):
    x = synth.activations(T + H, T, H)
    wr = synth.router_weight(E, H, E)
    bias = synth.zipf_bias(3, E) if E == 512 else None
    idx, w, logits = _route(x, wr, k, bias=bias)
    oi, ow, ol = O.moe_route(x, wr, k, bias=bias, want_logits=True)
    assert np.array_equal(logits.view(np.uint32), ol.view(np.uint32))
    assert np.array_equal(idx, oi)
    assert np.allclose(w, ow, rtol=1e-5, atol=1e-7)


def test_route_ties_and_no_renorm():
    H, E = 64, 8
    x = np.ones((2, H), dtype=np.float16)
    wr = np.zeros((H, E), dtype=np.float16)
    idx, w, _ = _route(x, wr, 3)
    assert idx.tolist() == [[0, 1, 2], [0, 1, 2]] and np.allclose(w, 1 / 3)
    wr[:, 5] = 1.0
    idx, w, _ = _route(x, wr, 2, renorm=False)
    oi, ow = O.moe_route(x, wr, 2, renorm=False)
    assert np.array_equal(idx, oi) and np.allclose(w, ow, rtol=1e-5, atol=1e-9)


def test_permute_matches_oracle():
    rng = np.random.default_rng(4)
    for T, k, E in [(1, 8, 128), (64, 8, 128), (256, 10, 512), (7, 3, 5)]:
        idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        d_idx = torch.from_numpy(idx).to(DEV)
        off = torch.zeros(E + 1, dtype=torch.int32, device=DEV)
        perm = torch.zeros(T * k, dtype=torch.int32, device=DEV)
        inv = torch.zeros(T * k, dtype=torch.int32, device=DEV)
        scratch = torch.zeros(K.moe.permute_scratch_bytes(T, k, E), dtype=torch.uint8, device=DEV)
        K.moe.permute(d_idx.data_ptr(), off.data_ptr(), perm.data_ptr(), inv.data_ptr(), scratch.data_ptr(), T, k, E)
        torch.cuda.synchronize()
        ooff, operm = O.moe_permute(idx, E)
        assert np.array_equal(off.cpu().numpy(), ooff)
        assert np.array_equal(perm.cpu().numpy(), operm)
        assert np.array_equal(inv.cpu().numpy()[operm], np.arange(T * k))


def _make_layer(gpu, seed, H, E, I, bits, shared_I=0, router_scale=1.0):
    experts_np, experts = [], []
    for e in range(E):
        s = seed + 10 * e
        trio = (synth.linear(s, H, I, bits), synth.linear(s + 3, H, I, bits), synth.linear(s + 6, I, H, bits))
        experts_np.append(trio)
        experts.append(tuple(Exl3Linear(gpu, f"experts.{e}.{n}", *lin)
                             for n, lin in zip(("gate_proj", "up_proj", "down_proj"), trio)))
    shared_np = shared = None
    if shared_I:
        s = seed + 99991
        shared_np = (synth.linear(s, H, shared_I, bits), synth.linear(s + 3, H, shared_I, bits),
                     synth.linear(s + 6, shared_I, H, bits))
        shared = tuple(Exl3Linear(gpu, f"shared_expert.{n}", *lin)
                       for n, lin in zip(("gate_proj", "up_proj", "down_proj"), shared_np))
    wr = (synth.router_weight(seed + 5, H, E).astype(np.float32) * router_scale).astype(np.float16)
    return wr, experts_np, experts, shared_np, shared


def _check_stages(layer, x, experts_np, shared_np, idx, w, out, T, H, E, k, I, bits, shared_I):
    """Each stage against the oracle on the SAME inputs the GPU stage consumed:
    gate/up outputs from the gathered tokens, down outputs from the GPU's own
    gate/up outputs, and the combine from the GPU's own down outputs."""
    offs = K.moe.workspace_offsets(T, H, E, k, I, shared_I)
    ws = layer._ws.cpu().numpy()
    P = T * k

    def view(name, dtype, shape):
        n = int(np.prod(shape)) * np.dtype(dtype).itemsize
        return ws[offs[name]:offs[name] + n].view(dtype).reshape(shape)

    perm = view("perm", np.int32, (P,))
    offsets = view("offsets", np.int32, (E + 1,))
    inv = view("inv", np.int32, (P,))
    ooff, operm = O.moe_permute(idx, E)
    assert np.array_equal(offsets, ooff) and np.array_equal(perm, operm)
    g = view("gate_out", np.float16, (P, I))
    u = view("up_out", np.float16, (P, I))
    slot = view("slot_out", np.float32, (P, H))
    for e in range(E):
        r0, r1 = int(offsets[e]), int(offsets[e + 1])
        if r0 == r1:
            continue
        xe = x[perm[r0:r1] // k]
        (gt, gs, gv), (ut, us, uv), (dt, ds, dv) = experts_np[e]
        want_g, _ = O.linear(xe, gt, gs, gv, H, I, bits, 2)
        want_u, _ = O.linear(xe, ut, us, uv, H, I, bits, 2)
        assert close(g[r0:r1], want_g)[0] == 0, ("gate", e)
        assert close(u[r0:r1], want_u)[0] == 0, ("up", e)
        a = O.silu_mul(g[r0:r1], u[r0:r1]).reshape(r1 - r0, I)
        want_d, _ = O.linear(a, dt, ds, dv, I, H, bits, 2, out_fp32=True)
        assert close(slot[r0:r1], want_d)[0] == 0, ("down", e)
    base = np.zeros((T, H), dtype=np.float32)
    if shared_np is not None:
        base = view("shared_out", np.float32, (T, H)).copy()
        # the always-on expert, stage by stage like the routed ones: its gate / up rows
        # (where the layer keeps them) against the oracle, its down row from the GPU's own
        # gate / up outputs
        sg_want, _ = O.linear(x, *shared_np[0], H, shared_I, bits, 2)
        su_want, _ = O.linear(x, *shared_np[1], H, shared_I, bits, 2)
        if shared_I == I:           # one more expert of the grouped launches: rows P .. P + T - 1
            sg = ws[offs["gate_out"] + P * I * 2:offs["gate_out"] + (P + T) * I * 2].view(np.float16).reshape(T, I)
            su = ws[offs["up_out"] + P * I * 2:offs["up_out"] + (P + T) * I * 2].view(np.float16).reshape(T, I)
            assert close(sg, sg_want)[0] == 0 and close(su, su_want)[0] == 0, "shared gate / up"
            act = O.silu_mul(sg, su).reshape(T, I)
        else:                       # a launch sequence of its own, with buffers of its own
            so = K.moe.workspace_shared_offsets(T, H, E, k, I, shared_I)
            sg = ws[so["shared_gate_out"]:so["shared_gate_out"] + T * shared_I * 2].view(np.float16).reshape(T, shared_I)
            su = ws[so["shared_up_out"]:so["shared_up_out"] + T * shared_I * 2].view(np.float16).reshape(T, shared_I)
            assert close(sg, sg_want)[0] == 0, "shared gate"
            if T <= 8:
                assert close(su, su_want)[0] == 0, "shared up"
                act = O.silu_mul(sg, su).reshape(T, shared_I)
            else:                   # the up buffer holds the activation by now
                act = su
                assert close(act, O.silu_mul(sg, su_want.astype(np.float16)).reshape(T, shared_I),
                             rtol=4e-3, atol=2e-3)[0] == 0, "shared activation"
        sd_want, _ = O.linear(act, *shared_np[2], shared_I, H, bits, 2, out_fp32=True)
        assert close(base, sd_want)[0] == 0, ("shared down", close(base, sd_want))
    acc = base.astype(np.float32)
    for j in range(k):
        acc = (np.float32(1) * acc + w[:, j:j + 1].astype(np.float32) * slot[inv.reshape(T, k)[:, j]]).astype(np.float32)
    assert np.allclose(out, acc, rtol=1e-5, atol=1e-5 * max(1.0, float(np.abs(acc).max())))


@pytest.mark.parametrize("T,H,E,k,I,bits,shared_I,scale", [
    (1, 256, 8, 2, 128, 4, 0, 1.0),
    (1, 256, 8, 2, 128, 4, 128, 1.0),       # one token, shared expert inside the grouped launches
    (1, 384, 8, 3, 128, 4, 256, 1.0),       # one token, shared expert as dense launches
    (4, 256, 8, 3, 256, 4, 128, 1.0),
    (40, 256, 4, 2, 128, 4, 0, 1.0),        # about 20 rows per expert
    (70, 256, 6, 2, 128, 3, 128, 30.0),     # skewed routing: one expert with several 32-row chunks
    (300, 128, 3, 1, 128, 4, 0, 50.0),      # long problem list
    (16, 2048, 16, 2, 768, 4, 0, 1.0),      # K large enough for split-K in the grouped GEMM
])
def test_moe_layer_matches_oracle(T, H, E, k, I, bits, shared_I, scale):
    gpu = Gpu(0)
    wr, experts_np, experts, shared_np, shared = _make_layer(gpu, 500 + T, H, E, I, bits, shared_I, scale)
    bias = synth.zipf_bias(7, E) if scale > 1 else None
    layer = MoeLayer(gpu, wr, experts, k, shared=shared, bias=bias)
    # tokens scaled like normalised hidden states, so that gate/up outputs are O(1)
    x = (synth.activations(900 + T, T, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    d_x = dev(x.view(np.uint16))
    out = torch.zeros((T, H), dtype=torch.float32, device=DEV)
    idx = torch.zeros((T, k), dtype=torch.int32, device=DEV)
    w = torch.zeros((T, k), dtype=torch.float32, device=DEV)
    layer.forward(gpu, d_x, out, T, idx, w)
    torch.cuda.synchronize()
    launch = K.moe.last_launch()
    want, oi, ow = O.moe_layer(x, wr, experts_np, k, I, bits, 2, bias=bias, shared=shared_np, shared_I=shared_I)
    assert np.array_equal(idx.cpu().numpy(), oi), launch
    assert np.allclose(w.cpu().numpy(), ow, rtol=1e-5, atol=1e-7)
    _check_stages(layer, x, experts_np, shared_np, oi, w.cpu().numpy(), out.cpu().numpy(), T, H, E, k, I, bits, shared_I)
    # end to end, the fp16 roundings of gate/up outputs differ in a few last bits
    # between two fp32 summation orders and propagate through down; bound the
    # whole-layer error relative to the output scale
    err = np.abs(out.cpu().numpy() - want)
    assert err.max() <= 2e-3 * np.abs(want).max(), (err.max(), np.abs(want).max(), launch)
    if T > 1 and T * k + (T if shared_I == I else 0) > 8:
        assert ("exl3_gemm_kernel" in launch or "exl3_gemm_mixed_kernel" in launch) and "exl3_gemv_kernel" not in launch
    else:
        assert "exl3_gemv_kernel" in launch and "exl3_gemm_" not in launch
    # a second call reuses the workspace and the self-resetting counters
    out2 = torch.zeros_like(out)
    layer.forward(gpu, d_x, out2, T)
    torch.cuda.synchronize()
    assert np.array_equal(out2.cpu().numpy().view(np.uint32), out.cpu().numpy().view(np.uint32))


def test_moe_config3_shape_decode_token():
    """hidden 2048, 128 experts, top-8, intermediate 768, 4 bpw, one token: the
    oracle runs only the 8 selected experts."""
    gpu = Gpu(0)
    H, E, k, I, bits = 2048, 128, 8, 768, 4
    wr, experts_np, experts, _, _ = _make_layer(gpu, 31, H, E, I, bits)
    layer = MoeLayer(gpu, wr, experts, k)
    x = (synth.activations(32, 1, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    out = torch.zeros((1, H), dtype=torch.float32, device=DEV)
    idx = torch.zeros((1, k), dtype=torch.int32, device=DEV)
    layer.forward(gpu, dev(x.view(np.uint16)), out, 1, idx)
    torch.cuda.synchronize()
    want, oi, ow = O.moe_layer(x, wr, experts_np, k, I, bits, 2)
    assert np.array_equal(idx.cpu().numpy(), oi)
    _check_stages(layer, x, experts_np, None, oi, ow, out.cpu().numpy(), 1, H, E, k, I, bits, 0)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-3 * np.abs(want).max()


def test_moe_config3_shape_batch64():
    """BASELINE configs[3] at 64 tokens (hidden 2048, 128 experts, top-8, intermediate 768,
    4 bpw) at full size: the whole layer against the oracle, stage by stage and end to end."""
    gpu = Gpu(0)
    T, H, E, k, I, bits = 64, 2048, 128, 8, 768, 4
    wr, experts_np, experts, _, _ = _make_layer(gpu, 61, H, E, I, bits)
    layer = MoeLayer(gpu, wr, experts, k)
    x = (synth.activations(62, T, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    out = torch.zeros((T, H), dtype=torch.float32, device=DEV)
    idx = torch.zeros((T, k), dtype=torch.int32, device=DEV)
    w = torch.zeros((T, k), dtype=torch.float32, device=DEV)
    layer.forward(gpu, dev(x.view(np.uint16)), out, T, idx, w)
    torch.cuda.synchronize()
    launch = K.moe.last_launch()
    want, oi, ow = O.moe_layer(x, wr, experts_np, k, I, bits, 2)
    assert np.array_equal(idx.cpu().numpy(), oi), launch
    assert len(np.unique(oi)) > 100                          # nearly every expert is hit
    assert np.allclose(w.cpu().numpy(), ow, rtol=1e-5, atol=1e-7)
    _check_stages(layer, x, experts_np, None, oi, w.cpu().numpy(), out.cpu().numpy(), T, H, E, k, I, bits, 0)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-3 * np.abs(want).max(), launch
    assert "exl3_gemm_kernel" in launch or "exl3_gemm_mixed_kernel" in launch


def test_moe_config4_shape_zipf_shared():
    """hidden 2048, 512 experts top-10 plus an always-on shared expert, intermediate
    512, 3 bpw, 256 tokens, Zipf(1.1)-biased router: skewed problem list (hot
    experts with several 32-row chunks, many cold experts with a row or none)."""
    gpu = Gpu(0)
    T, H, E, k, I, bits = 256, 2048, 512, 10, 512, 3
    # router scaled by sqrt(H) to compensate the 1/sqrt(H) token scale: same logits as N(0,1) tokens
    wr, experts_np, experts, shared_np, shared = _make_layer(gpu, 7000, H, E, I, bits, I, float(np.sqrt(H)))
    bias = synth.zipf_bias(41, E)
    layer = MoeLayer(gpu, wr, experts, k, shared=shared, bias=bias)
    x = (synth.activations(43, T, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    out = torch.zeros((T, H), dtype=torch.float32, device=DEV)
    idx = torch.zeros((T, k), dtype=torch.int32, device=DEV)
    w = torch.zeros((T, k), dtype=torch.float32, device=DEV)
    layer.forward(gpu, dev(x.view(np.uint16)), out, T, idx, w)
    torch.cuda.synchronize()
    want, oi, ow = O.moe_layer(x, wr, experts_np, k, I, bits, 2, bias=bias, shared=shared_np, shared_I=I)
    assert np.array_equal(idx.cpu().numpy(), oi)
    counts = np.bincount(oi.ravel(), minlength=E)
    assert counts.max() > 64 and (counts == 0).sum() > 0, "routing is not skewed"
    assert np.allclose(w.cpu().numpy(), ow, rtol=1e-5, atol=1e-7)
    _check_stages(layer, x, experts_np, shared_np, oi, w.cpu().numpy(), out.cpu().numpy(), T, H, E, k, I, bits, I)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-3 * np.abs(want).max()


_ONE_TOKEN_CASES = {"plain": (2048, 128, 8, 768, 4, 0), "folded": (512, 16, 4, 256, 3, 256),
                    "dense": (512, 16, 4, 256, 4, 384), "sixteen": (512, 32, 15, 256, 4, 256),
                    "seventeen": (512, 32, 16, 256, 2, 256)}


def _one_token_outputs():
    """One token through five layers (no shared expert, shared expert of the routed size,
    shared expert of another size, sixteen and seventeen problems per launch), twice each:
    output bits, the rows of the down projection and launch text."""
    gpu = Gpu(0)
    res = {}
    for name, (H, E, k, I, bits, shared_I) in _ONE_TOKEN_CASES.items():
        wr, _, experts, _, shared = _make_layer(gpu, 8100 + H + shared_I + k, H, E, I, bits, shared_I)
        layer = MoeLayer(gpu, wr, experts, k, shared=shared)
        outs, rows = [], []
        for rep in range(2):
            x = (synth.activations(77 + rep, 1, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
            out = torch.zeros((1, H), dtype=torch.float32, device=DEV)
            layer.forward(gpu, dev(x.view(np.uint16)), out, 1)
            torch.cuda.synchronize()
            outs.append(out.cpu().numpy().view(np.uint32))
            at = K.moe.workspace_offsets(1, H, E, k, I, shared_I)["slot_out"]
            rows.append(layer._ws.cpu().numpy()[at:at + k * H * 4].view(np.uint32).copy())
        res[name] = np.stack(outs)
        res[name + "_rows"] = np.stack(rows)
        res[name + "_launch"] = np.array(K.moe.last_launch())
    return res


def test_moe_one_token_combine_inside_down_projection(tmp_path):
    """With one token the last workgroup to finish a column block of the down projection
    combines it.  By default split-K and combine share one hand-over (up to sixteen problems
    per launch); BERTH_MOE_FOLD_COMBINE=1 keeps the two-stage form and =0 the separate combine
    launch (read once per process, so each in a process of its own).  All three give the same
    output bits and the same rows of the down projection."""
    import os
    import subprocess
    import sys

    here = _one_token_outputs()
    for name in _ONE_TOKEN_CASES:
        launch = str(here[name + "_launch"])
        assert "+combine" in launch and "moe_combine_kernel" not in launch, launch
        assert ("one hand-over" in launch) == (name != "seventeen"), launch
        assert here[name].any() and here[name + "_rows"].any()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for mode in ("0", "1"):
        path = str(tmp_path / f"mode{mode}.npz")
        code = ("import numpy as np, tests.test_gpu_moe as T\n"
                f"np.savez({path!r}, **T._one_token_outputs())\nprint('ok')\n")
        r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=600, cwd=root,
                           env=dict(os.environ, BERTH_MOE_FOLD_COMBINE=mode))
        assert r.returncode == 0 and "ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
        there = np.load(path)
        for name in _ONE_TOKEN_CASES:
            launch = str(there[name + "_launch"])
            if mode == "0":
                assert "moe_combine_kernel" in launch and "+combine" not in launch, launch
            else:
                assert "+combine" in launch and "one hand-over" not in launch, launch
            assert np.array_equal(here[name], there[name]), (mode, name)
            assert np.array_equal(here[name + "_rows"], there[name + "_rows"]), (mode, name)


def test_moe_128_row_problems_give_the_bits_of_32_row_problems():
    """From 256 rows on, an expert's rows beyond 32 run as problems of up to 128 rows in the same
    launch as the 32-row ones (BERTH_MOE_BIG_MIN: the smallest remainder that still becomes one;
    0 switches them off).  Every output element sums the same products in the same order either
    way, so the layer's bits do not depend on the setting."""
    gpu = Gpu(0)
    for T, H, E, k, I, bits, shared_I, scale in ((300, 128, 3, 1, 128, 4, 0, 50.0), (160, 256, 6, 2, 128, 3, 128, 30.0)):
        wr, _, experts, _, shared = _make_layer(gpu, 7300 + T, H, E, I, bits, shared_I, scale)
        x = (synth.activations(7400 + T, T, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
        d_x = dev(x.view(np.uint16))
        res = {}
        for big_min in (0, 33, 65, 128):
            with knobs(BERTH_MOE_BIG_MIN=big_min):
                layer = MoeLayer(gpu, wr, experts, k, shared=shared, bias=synth.zipf_bias(7, E))
                out = torch.zeros((T, H), dtype=torch.float32, device=DEV)
                layer.forward(gpu, d_x, out, T)
                torch.cuda.synchronize()
                launch = K.moe.last_launch()
                assert ("exl3_gemm_mixed_kernel" in launch) == (big_min > 0), launch
                res[big_min] = out.cpu().numpy().view(np.uint32).copy()
        for big_min in (33, 65, 128):
            assert np.array_equal(res[big_min], res[0]), big_min


@pytest.mark.parametrize("T,H,E,k,I,bits,shared_I", [
    (1, 256, 8, 2, 128, 4, 128),         # one token, the shared expert inside the grouped launches
    (1, 384, 8, 3, 128, 4, 256),         # one token, the shared expert as dense launches
    (5, 256, 8, 2, 128, 3, 128),
    (40, 256, 4, 2, 128, 4, 256),        # the MFMA path
])
def test_moe_layer_with_a_gate_on_the_shared_expert(T, H, E, k, I, bits, shared_I):
    """berth_moe_layer_gated: the always-on expert's row is scaled by sigmoid(x . w) before the
    routed experts are added; routing and every stage ahead of the combine are untouched."""
    gpu = Gpu(0)
    wr, experts_np, experts, shared_np, shared = _make_layer(gpu, 6600 + T, H, E, I, bits, shared_I)
    wg = (np.random.default_rng(6700 + T).standard_normal(H) * 2.0).astype(np.float32)
    x = (synth.activations(6800 + T, T, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    d_x = dev(x.view(np.uint16))
    outs = {}
    for name, gate in (("plain", None), ("gated", wg)):
        layer = MoeLayer(gpu, wr, experts, k, shared=shared, shared_gate=gate)
        out = torch.zeros((T, H), dtype=torch.float32, device=DEV)
        idx = torch.zeros((T, k), dtype=torch.int32, device=DEV)
        layer.forward(gpu, d_x, out, T, idx)
        torch.cuda.synchronize()
        assert ("moe_shared_gate_kernel" in K.moe.last_launch()) == (gate is not None), K.moe.last_launch()
        want, oi, _ = O.moe_layer(x, wr, experts_np, k, I, bits, 2, shared=shared_np, shared_I=shared_I, shared_gate=gate)
        assert np.array_equal(idx.cpu().numpy(), oi)
        outs[name] = out.cpu().numpy()
        assert np.abs(outs[name] - want).max() <= 2e-3 * np.abs(want).max(), name
    scale = O.moe_shared_gate(x, wg)
    assert np.ptp(scale) > 0.05 or T == 1
    assert np.abs(outs["gated"] - outs["plain"]).max() > 1e-3 * np.abs(outs["plain"]).max()   # the gate does something
    with pytest.raises(InputError, match="without a shared expert"):
        MoeLayer(gpu, wr, experts, k, shared_gate=wg)
    with pytest.raises(K.LaunchError, match="gate without a shared expert"):
        K.moe.layer(1, 1, None, 1, None, 1, None, None, 1, 1 << 30, 1, 128, 8, 2, 128, 0, 4, K.Codebook.MUL1, shared_gate=1)


@pytest.mark.parametrize("T,H,E,k", [(64, 2048, 128, 8), (256, 2048, 512, 10), (33, 256, 6, 2), (40, 1024, 258, 5)])
def test_many_token_routing_in_one_launch_equals_the_two_launch_form(T, H, E, k):
    """From 32 tokens on (even expert count, hidden a multiple of 64) the routing is one launch in
    which the segment sums of a token group x a slab of 128 experts meet in LDS;
    BERTH_MOE_ROUTE_SLAB=0 keeps the partial-sum launch and the finish launch.  Same arithmetic in
    the same order: the same logits, experts and weights, bit for bit, and the oracle's."""
    wr = synth.router_weight(5100 + E, H, E)
    bias = synth.zipf_bias(5101, E)
    x = (synth.activations(5102 + T, T, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    d_x, d_wr = dev(x.view(np.uint16)), dev(wr.view(np.uint16))
    d_bias = torch.from_numpy(bias).to(DEV)
    res = {}
    for slab in (1, 0):
        with knobs(BERTH_MOE_ROUTE_SLAB=slab):
            idx = torch.zeros((T, k), dtype=torch.int32, device=DEV)
            w = torch.zeros((T, k), dtype=torch.float32, device=DEV)
            logits = torch.zeros((T, E), dtype=torch.float32, device=DEV)
            parts = torch.zeros(T * (H // 64) * E, dtype=torch.float32, device=DEV)
            K.moe.route(d_x.data_ptr(), d_wr.data_ptr(), d_bias.data_ptr(), idx.data_ptr(), w.data_ptr(),
                        logits.data_ptr(), parts.data_ptr(), T, H, E, k, True)
            torch.cuda.synchronize()
            assert ("moe_route_slab_kernel" in K.moe.last_launch()) == bool(slab), K.moe.last_launch()
            res[slab] = (idx.cpu().numpy(), w.cpu().numpy().view(np.uint32), logits.cpu().numpy().view(np.uint32))
    for a, b in zip(res[1], res[0]):
        assert np.array_equal(a, b)
    oi, ow, ol = O.moe_route(x, wr, k, bias=bias, want_logits=True)
    assert np.array_equal(res[1][0], oi)
    assert np.array_equal(res[1][2], ol.view(np.uint32))


def test_moe_validation_errors():
    with pytest.raises(K.LaunchError, match="null"):
        K.moe.layer(None, None, None, None, None, None, None, None, None, 0, 1, 128, 8, 2, 128, 0, 4, K.Codebook.MUL1)
    with pytest.raises(K.LaunchError, match="top-k"):
        K.moe.route(1, 1, None, 1, 1, None, 1, 1, 128, 4, 5)


def test_moe_one_token_inline_routing_equals_the_routing_kernel():
    """One token, at most 128 experts: by default only the router's 64-row segment sums come
    from a launch of their own and every workgroup of the gate / up launch redoes the ordered
    sum, the top-k and the sort for itself; BERTH_MOE_INLINE_ROUTE=0 keeps the routing kernel.
    Same arithmetic in the same order: the same experts, weights and output bits."""
    import os
    gpu = Gpu(0)
    for H, E, k, I, bits, shared_I in ((2048, 128, 8, 768, 4, 0), (512, 16, 4, 256, 3, 256), (1024, 64, 6, 384, 4, 512)):
        wr, _, experts, _, shared = _make_layer(gpu, 8800 + H + E, H, E, I, bits, shared_I)
        layer = MoeLayer(gpu, wr, experts, k, shared=shared, bias=synth.zipf_bias(3, E))
        x = (synth.activations(8801 + H, 1, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
        d_x = dev(x.view(np.uint16))
        res = {}
        for mode, env in (("1", {}), ("unresolved", {"BERTH_MOE_RESOLVED": "0"}), ("0", {"BERTH_MOE_INLINE_ROUTE": "0"})):
            with knobs(**env):
                out = torch.zeros((1, H), dtype=torch.float32, device=DEV)
                idx = torch.full((1, k), -1, dtype=torch.int32, device=DEV)
                w = torch.zeros((1, k), dtype=torch.float32, device=DEV)
                layer.forward(gpu, d_x, out, 1, idx, w)
                torch.cuda.synchronize()
                res[mode] = (out.cpu().numpy().view(np.uint32), idx.cpu().numpy(), w.cpu().numpy().view(np.uint32),
                             K.moe.last_launch())
        # the down launch takes its linears from the records the gate / up launch left, unless told not to
        assert "moe_route_segments_kernel" in res["1"][3] and "+route" in res["1"][3] and "resolved" in res["1"][3], res["1"][3]
        assert "+route" in res["unresolved"][3] and "resolved" not in res["unresolved"][3], res["unresolved"][3]
        assert "moe_route_one_token_kernel" in res["0"][3] and "+route" not in res["0"][3], res["0"][3]
        for other in ("unresolved", "0"):
            for a, b in zip(res["1"][:3], res[other][:3]):
                assert np.array_equal(a, b), (H, E, other, res["1"][3])


@pytest.mark.parametrize("T,H,E,k,I,bits", [
    (1, 256, 8, 2, 128, 4),          # one row per expert
    (3, 256, 8, 2, 128, 4),          # six rows: still the dot-product kernel, several rows per problem
    (64, 512, 16, 4, 256, 4),        # the MFMA path with rotated rows in a caller buffer
    (33, 256, 4, 2, 128, 3),
])
def test_stage_entry_points_compose_to_the_layer(T, H, E, k, I, bits):
    """route -> permute -> grouped gate/up -> grouped down -> combine, each through its own entry
    point, against the same stages inside berth_moe_layer (same kernels: bit for bit) and the
    oracle."""
    gpu = Gpu(0)
    wr, experts_np, experts, _, _ = _make_layer(gpu, 4100 + T, H, E, I, bits)
    layer = MoeLayer(gpu, wr, experts, k)
    x = (synth.activations(4200 + T, T, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    d_x = dev(x.view(np.uint16))
    want_out = torch.zeros((T, H), dtype=torch.float32, device=DEV)
    layer.forward(gpu, d_x, want_out, T)
    torch.cuda.synchronize()
    offs = K.moe.workspace_offsets(T, H, E, k, I, 0)
    ws = layer._ws.cpu().numpy()
    P = T * k

    def inside(name, dtype, shape):
        n = int(np.prod(shape)) * np.dtype(dtype).itemsize
        return ws[offs[name]:offs[name] + n].view(dtype).reshape(shape).copy()

    idx = torch.zeros((T, k), dtype=torch.int32, device=DEV)
    w = torch.zeros((T, k), dtype=torch.float32, device=DEV)
    parts = torch.zeros(T * ((H + 63) // 64) * E, dtype=torch.float32, device=DEV)
    K.moe.route(d_x.data_ptr(), layer.router.data_ptr(), None, idx.data_ptr(), w.data_ptr(), None, parts.data_ptr(),
                T, H, E, k, True)
    off = torch.zeros(E + 1, dtype=torch.int32, device=DEV)
    perm = torch.zeros(P, dtype=torch.int32, device=DEV)
    inv = torch.zeros(P, dtype=torch.int32, device=DEV)
    scratch = torch.zeros(K.moe.permute_scratch_bytes(T, k, E), dtype=torch.uint8, device=DEV)
    K.moe.permute(idx.data_ptr(), off.data_ptr(), perm.data_ptr(), inv.data_ptr(), scratch.data_ptr(), T, k, E)
    g = torch.zeros((P, I), dtype=torch.float16, device=DEV)
    u = torch.zeros((P, I), dtype=torch.float16, device=DEV)
    slot = torch.zeros((P, H), dtype=torch.float32, device=DEV)
    a_had = torch.zeros(2 * P * max(H, I), dtype=torch.float16, device=DEV)
    K.moe.grouped_exl3(d_x.data_ptr(), None, perm.data_ptr(), k, layer.table.data_ptr(), 3, 0, 2, g.data_ptr(),
                       u.data_ptr(), scratch.data_ptr(), a_had.data_ptr(), T, k, E, H, I, bits, 2, False)
    first = K.moe.last_launch()
    K.moe.grouped_exl3(g.data_ptr(), u.data_ptr(), None, 1, layer.table.data_ptr(), 3, 2, 1, slot.data_ptr(), None,
                       scratch.data_ptr(), a_had.data_ptr(), T, k, E, I, H, bits, 2, True)
    out = torch.zeros((T, H), dtype=torch.float32, device=DEV)
    K.moe.combine(slot.data_ptr(), None, w.data_ptr(), inv.data_ptr(), out.data_ptr(), T, H, k)
    torch.cuda.synchronize()
    assert ("exl3_gemm_" in first) == (P > 8), first
    assert np.array_equal(idx.cpu().numpy(), inside("idx", np.int32, (T, k)))
    assert np.array_equal(perm.cpu().numpy(), inside("perm", np.int32, (P,)))
    assert np.array_equal(inv.cpu().numpy(), inside("inv", np.int32, (P,)))
    assert np.array_equal(g.cpu().numpy().view(np.uint16), inside("gate_out", np.uint16, (P, I)))
    assert np.array_equal(u.cpu().numpy().view(np.uint16), inside("up_out", np.uint16, (P, I)))
    assert np.array_equal(slot.cpu().numpy().view(np.uint32), inside("slot_out", np.uint32, (P, H)))
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want_out.cpu().numpy().view(np.uint32))
    want, oi, _ = O.moe_layer(x, wr, experts_np, k, I, bits, 2)
    assert np.array_equal(idx.cpu().numpy(), oi)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-3 * np.abs(want).max()


def test_stage_entry_points_validate_before_launching():
    P0 = 0x1000
    bad = [
        (dict(num_lins=3), "num_lins must be 1 or 2"),
        (dict(num_lins=2, c1=None), "c1 goes with the second linear"),
        (dict(a_up=P0, num_lins=2), "silu input serves one linear"),
        (dict(lin_base=2, num_lins=2), "exceeds lins_per_expert"),
        (dict(size_k=100), "multiples of 128"),
        (dict(k_bits=9), "1..=8"),
        (dict(T=64, a_had=None), "a_had is required above 8 rows"),
        (dict(k=9, E=8), "top-k exceeds"),
        (dict(gather=P0, gather_div=0), "gather_div must be positive"),
    ]
    for change, message in bad:
        a = dict(a=P0, a_up=None, gather=None, gather_div=1, experts=P0, lins_per_expert=3, lin_base=0, num_lins=2,
                 c0=P0, c1=P0, scratch=P0, a_had=P0, T=1, k=2, E=8, size_k=256, size_n=128, k_bits=4, codebook=2,
                 c_fp32=False)
        a.update(change)
        with pytest.raises(K.LaunchError, match=message):
            K.moe.grouped_exl3(a["a"], a["a_up"], a["gather"], a["gather_div"], a["experts"], a["lins_per_expert"],
                               a["lin_base"], a["num_lins"], a["c0"], a["c1"], a["scratch"], a["a_had"], a["T"], a["k"],
                               a["E"], a["size_k"], a["size_n"], a["k_bits"], a["codebook"], a["c_fp32"])
    with pytest.raises(K.LaunchError, match="null device pointer"):
        K.moe.combine(None, None, P0, P0, P0, 1, 128, 2)
    with pytest.raises(K.LaunchError, match="sizes must be positive"):
        K.moe.combine(P0, None, P0, P0, P0, 0, 128, 2)
