"""From an EXL3 checkpoint directory on disk to outputs on the GPU: the reader
(libberth_exl3_reader.so), the loaders of the Python mirror
(`Exl3Linear.load`, `MlpLayer.load`: crates/berth-engine/src/device.rs:92-125,
mlp.rs:52-112) and of the C++ host layer (through berth_host_check), checked
against the CPU oracle on the same tensors."""
import os
import subprocess

import numpy as np
import pytest
import torch

from berth_amd import exl3, plan as P, synth
from berth_amd.device import Exl3Linear, Gpu, InputError, MlpLayer, RowScratch, WeightsError
from berth_amd.moe import MoeLayer
from berth_amd.kernels import Codebook, OutDtype
from oracle import oracle as O
from tests import ckpt_util as U
from tests.gpu_util import close, host_f16

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "berth_amd", "lib", "berth_host_check")
H, I = 256, 384
MLP0 = "model.language_model.layers.0.mlp"
MLP1 = "model.language_model.layers.1.mlp"


def signs_only(scale):
    """+-1 with the sign of `scale`: what a packed su / sv tensor can hold."""
    return np.where(scale.view(np.uint16) >> 15, np.float16(-1), np.float16(1)).astype(np.float16)


@pytest.fixture(scope="module")
def ckpt_dir(tmp_path_factory):
    d = tmp_path_factory.mktemp("ckpt")
    lins = {
        f"{MLP0}.gate_proj": (synth.linear(8000, H, I, 4), "mul1"),
        f"{MLP0}.up_proj": (synth.linear(8003, H, I, 4), "mul1"),
        f"{MLP0}.down_proj": (synth.linear(8006, I, H, 4), "mul1"),
        "attn.q_proj": (synth.linear(8010, H, 512, 3), "mcg"),
        "attn.k_proj": (synth.linear(8013, H, 128, 5), None),
    }
    tensors = []
    for prefix, (lin, cb) in lins.items():
        tensors += U.linear_tensors(prefix, *lin, codebook=cb)
    # packed signs: the stored scales are pure signs
    tr, suh, svh = synth.linear(8020, H, 256, 2)
    lins["attn.packed"] = ((tr, signs_only(suh), signs_only(svh)), "mul1")
    tensors += U.linear_tensors("attn.packed", tr, suh, svh, packed=True)
    # a half-integer rate (1.5 bpw: 24 words per tile), refused by the loaders, and an MLP whose up
    # projection carries a bias
    tensors += U.linear_tensors("attn.half", np.zeros((H // 16, 128 // 16, 24), np.uint16), *synth.linear(1, H, 128, 1)[1:])
    for part, (k, n) in (("gate_proj", (H, I)), ("up_proj", (H, I)), ("down_proj", (I, H))):
        tensors += U.linear_tensors(f"{MLP1}.{part}", *synth.linear(8030, k, n, 2),
                                    bias=(np.arange(n, dtype=np.float32) / 64 - 2).astype(np.float16)
                                    if part == "up_proj" else None)
    tensors.append(("model.norm.weight", "BF16", (H,), bytes(2 * H)))
    U.write_checkpoint(d, tensors)
    return d, lins


def test_python_loader_runs_every_linear_of_the_checkpoint(ckpt_dir):
    d, lins = ckpt_dir
    ckpt = exl3.Checkpoint.open(d)
    assert len(ckpt.linears()) == len(lins) + 4 and len(ckpt.other_tensors()) == 1
    gpu = Gpu(0)
    for prefix, ((tr, suh, svh), cb) in lins.items():
        lin = Exl3Linear.load(gpu, ckpt, prefix)
        want_cb = {"mul1": Codebook.MUL1, "mcg": Codebook.MCG, None: Codebook.DEFAULT}[cb]
        assert (lin.size_k, lin.size_n, lin.k_bits, lin.codebook) == (suh.size, svh.size, tr.shape[2] // 16, want_cb)
        x = synth.activations(8100, 1, lin.size_k)
        c = torch.zeros(lin.size_n, dtype=torch.float16, device=gpu.device)
        lin.forward(gpu, gpu.upload(x.view(np.uint16)), c, OutDtype.F16)
        gpu.synchronize()
        want, _ = O.linear(x, tr, suh, svh, lin.size_k, lin.size_n, lin.k_bits, int(want_cb))
        assert close(host_f16(c), want.reshape(-1))[0] == 0, prefix


def test_python_mlp_loader_and_refusals(ckpt_dir):
    d, lins = ckpt_dir
    ckpt = exl3.Checkpoint.open(d)
    gpu = Gpu(0)
    mlp = MlpLayer.load(gpu, ckpt, 0)
    assert (mlp.hidden, mlp.intermediate) == (H, I)
    x = (synth.activations(8200, 1, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    y = torch.zeros(H, dtype=torch.float32, device=gpu.device)
    mlp.forward(gpu, gpu.upload(x.view(np.uint16)), y)
    gpu.synchronize()
    assert np.abs(y.cpu().numpy() - _mlp_oracle(lins, x)).max() <= 2e-3 * np.abs(_mlp_oracle(lins, x)).max()
    # crates/berth-engine/src/device.rs:95-97, mlp.rs:67-75, device.rs:167-173
    with pytest.raises(WeightsError, match="attn.half: half-integer rate"):
        Exl3Linear.load(gpu, ckpt, "attn.half")
    with pytest.raises(WeightsError, match="nope is not an EXL3 linear"):
        Exl3Linear.load(gpu, ckpt, "nope")
    with pytest.raises(WeightsError, match="layers.7.mlp.gate_proj is not an EXL3 linear"):
        MlpLayer.load(gpu, ckpt, 7)


def _mlp_oracle(lins, x):
    gate, up, down = (lins[f"{MLP0}.{p}"][0] for p in ("gate_proj", "up_proj", "down_proj"))
    g, _ = O.linear(x, *gate, H, I, 4, 2)
    u, _ = O.linear(x, *up, H, I, 4, 2)
    want, _ = O.linear(O.silu_mul(g, u).reshape(1, I), *down, I, H, 4, 2, out_fp32=True)
    return want.reshape(-1)


def _host_check(*args):
    assert os.path.exists(EXE), "berth_host_check is not built (python -m berth_amd.build)"
    return subprocess.run([EXE, *map(str, args)], capture_output=True, text=True, timeout=300)


@pytest.mark.parametrize("prefix", ["attn.q_proj", "attn.k_proj", "attn.packed"])
def test_cpp_loader_linear(ckpt_dir, tmp_path, prefix):
    d, lins = ckpt_dir
    (tr, suh, svh), cb = lins[prefix]
    x = synth.activations(8300, 1, H)
    x.view(np.uint16).tofile(tmp_path / "x.bin")
    r = _host_check("ckpt-linear", d, prefix, tmp_path)
    assert r.returncode == 0, r.stdout + r.stderr
    cbi = {"mul1": 2, "mcg": 1, None: 0}[cb]
    assert f"ckpt-linear ok {prefix} K={H} N={svh.size} bits={tr.shape[2] // 16} codebook={cbi}" in r.stdout
    y = np.fromfile(tmp_path / "y.bin", dtype=np.float32)
    want, _ = O.linear(x, tr, suh, svh, H, svh.size, tr.shape[2] // 16, cbi, out_fp32=True)
    assert close(y, want.reshape(-1))[0] == 0


def test_cpp_loader_mlp_and_refusals(ckpt_dir, tmp_path):
    d, lins = ckpt_dir
    x = (synth.activations(8200, 1, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    x.view(np.uint16).tofile(tmp_path / "x.bin")
    r = _host_check("ckpt-mlp", d, 0, tmp_path)
    assert r.returncode == 0 and f"ckpt-mlp ok layer=0 hidden={H} intermediate={I}" in r.stdout, r.stdout + r.stderr
    y = np.fromfile(tmp_path / "y.bin", dtype=np.float32)
    want = _mlp_oracle(lins, x)
    assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max()
    r = _host_check("ckpt-linear", d, "attn.half", tmp_path)
    assert r.returncode == 1 and "attn.half: half-integer rate" in r.stderr
    r = _host_check("ckpt-linear", d, "nope", tmp_path)
    assert r.returncode == 1 and "nope is not an EXL3 linear" in r.stderr


# ---------------------------------------------------------------------------------------------
# a MoE layer from a checkpoint directory: config keys -> MoeDims -> Ffn::Moe -> MoeLayer.load

MOE_H, MOE_E, MOE_K, MOE_I = 256, 8, 2, 128
MOE_MLP = "model.language_model.layers.1.mlp"


def _moe_config(shared_i):
    cfg = {k: (dict(v) if isinstance(v, dict) else v) for k, v in U.CONFIG.items()}
    cfg["architectures"] = [P.ARCH_QWEN3_5_MOE]
    cfg["text_config"].update(hidden_size=MOE_H, num_experts=MOE_E, num_experts_per_tok=MOE_K,
                              moe_intermediate_size=MOE_I, shared_expert_intermediate_size=shared_i)
    return cfg


def _bf16_bits(values_f32):
    """fp32 -> bf16 bit patterns, round to nearest even."""
    u = values_f32.astype(np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _moe_parts(seed, shared_i, bits=4):
    experts = []
    for e in range(MOE_E):
        s = seed + 10 * e
        experts.append((synth.linear(s, MOE_H, MOE_I, bits), synth.linear(s + 3, MOE_H, MOE_I, bits),
                        synth.linear(s + 6, MOE_I, MOE_H, bits)))
    s = seed + 7001
    shared = (synth.linear(s, MOE_H, shared_i, bits), synth.linear(s + 3, MOE_H, shared_i, bits),
              synth.linear(s + 6, shared_i, MOE_H, bits))
    # router values that need rounding on the way to fp16
    wf = synth.router_weight(seed + 5, MOE_H, MOE_E).astype(np.float32) * np.float32(1.00037) + np.float32(3e-6)
    return experts, shared, wf


@pytest.fixture(scope="module")
def moe_ckpt_per_expert(tmp_path_factory):
    """`experts.<e>.<proj>` names, a BF16 router, shared expert as wide as a routed one."""
    d = tmp_path_factory.mktemp("moe_ckpt_a")
    experts, shared, wf = _moe_parts(9100, MOE_I)
    bits16 = _bf16_bits(wf)                                              # [H][E] values as stored precision
    stored = (bits16.astype(np.uint32) << 16).view(np.float32)
    tensors = [(f"{MOE_MLP}.gate.weight", "BF16", (MOE_E, MOE_H), np.ascontiguousarray(bits16.T).tobytes())]
    for e, trio in enumerate(experts):
        for name, lin in zip(("gate_proj", "up_proj", "down_proj"), trio):
            tensors += U.linear_tensors(f"{MOE_MLP}.experts.{e}.{name}", *lin)
    for name, lin in zip(("gate_proj", "up_proj", "down_proj"), shared):
        tensors += U.linear_tensors(f"{MOE_MLP}.shared_expert.{name}", *lin)
    tensors.append(("model.language_model.norm.weight", "BF16", (MOE_H,), bytes(2 * MOE_H)))
    tensors.append(("model.visual.pos_embed.weight", "BF16", (64,), bytes(128)))
    U.write_checkpoint(d, tensors, _moe_config(MOE_I))
    return d, experts, shared, stored.astype(np.float16), MOE_I, None


@pytest.fixture(scope="module")
def moe_ckpt_stacked(tmp_path_factory):
    """`experts.gate_up_proj` / `experts.down_proj` stacked along K, an F32 router, a wider shared expert
    with a BF16 `shared_expert_gate.weight` on it."""
    d = tmp_path_factory.mktemp("moe_ckpt_b")
    shared_i = 256
    experts, shared, wf = _moe_parts(9300, shared_i)
    # one stacked tensor has one input scale per expert: gate and up share it
    experts = [(g, (u[0], g[1], u[2]), dn) for g, u, dn in experts]
    tensors = [(f"{MOE_MLP}.gate.weight", "F32", (MOE_E, MOE_H), np.ascontiguousarray(wf.T).tobytes())]
    gate_up = np.concatenate([np.concatenate([g[0], u[0]], axis=1) for g, u, _ in experts], axis=0)
    tensors += U.linear_tensors(f"{MOE_MLP}.experts.gate_up_proj", gate_up,
                                np.concatenate([g[1] for g, _, _ in experts]),
                                np.concatenate([np.concatenate([g[2], u[2]]) for g, u, _ in experts]))
    down = np.concatenate([dn[0] for _, _, dn in experts], axis=0)
    tensors += U.linear_tensors(f"{MOE_MLP}.experts.down_proj", down, np.concatenate([dn[1] for _, _, dn in experts]),
                                np.concatenate([dn[2] for _, _, dn in experts]))
    for name, lin in zip(("gate_proj", "up_proj", "down_proj"), shared):
        tensors += U.linear_tensors(f"{MOE_MLP}.shared_expert.{name}", *lin)
    gate_bits = _bf16_bits((np.random.default_rng(9301).standard_normal(MOE_H) * 1.5).astype(np.float32))
    tensors.append((f"{MOE_MLP}.shared_expert_gate.weight", "BF16", (1, MOE_H), gate_bits.tobytes()))
    U.write_checkpoint(d, tensors, _moe_config(shared_i))
    return d, experts, shared, wf.astype(np.float16), shared_i, (gate_bits.astype(np.uint32) << 16).view(np.float32)


def _moe_tokens(T):
    return (synth.activations(9500 + T, T, MOE_H).astype(np.float32) / np.sqrt(MOE_H)).astype(np.float16)


def _moe_want(case, x):
    _, experts, shared, wr, shared_i, shared_gate = case
    return O.moe_layer(x, wr, experts, MOE_K, MOE_I, 4, 2, shared=shared, shared_I=shared_i, shared_gate=shared_gate)


@pytest.mark.parametrize("which", ["per_expert", "stacked"])
@pytest.mark.parametrize("T", [1, 5])
def test_python_moe_loader_follows_the_plan(request, which, T):
    case = request.getfixturevalue(f"moe_ckpt_{which}")
    ckpt = exl3.Checkpoint.open(case[0])
    plan = P.build_plan(P.model_shape(ckpt))
    ffn = plan.layers[1].ffn
    assert ffn == P.Ffn(P.Router(MOE_E, MOE_K), P.SharedExpert(case[4]), P.RoutedExperts(MOE_E, MOE_K, MOE_I))
    gpu = Gpu(0)
    layer = MoeLayer.load(gpu, ckpt, 1, ffn)
    assert (layer.hidden, layer.num_experts, layer.top_k, layer.intermediate, layer.shared_I) == \
        (MOE_H, MOE_E, MOE_K, MOE_I, case[4])
    assert (layer.shared_gate is not None) == (case[5] is not None)
    if case[5] is not None:
        assert np.array_equal(layer.shared_gate.cpu().numpy(), case[5])
    x = _moe_tokens(T)
    out = torch.zeros((T, MOE_H), dtype=torch.float32, device=gpu.device)
    idx = torch.zeros((T, MOE_K), dtype=torch.int32, device=gpu.device)
    layer.forward(gpu, gpu.upload(x.view(np.uint16)), out, T, idx)
    gpu.synchronize()
    want, oi, _ = _moe_want(case, x)
    assert np.array_equal(idx.cpu().numpy(), oi)
    assert np.abs(out.cpu().numpy() - want).max() <= 2e-3 * np.abs(want).max()
    # the bytes one token reads, from the same checkpoint: backbone + top_k / experts of the pool
    listed = P.tensor_bytes(ckpt)
    pool = sum(b for n, b in listed.tensors if P.is_routed_expert(n))
    placed = P.place(plan, listed)
    assert pool > 0 and placed.bytes_moved == listed.total() - pool + pool * MOE_K // MOE_E
    assert not any(n.startswith("model.visual.") for n, _ in listed.tensors)


def test_python_moe_loader_refusals(moe_ckpt_per_expert, ckpt_dir, tmp_path):
    d = moe_ckpt_per_expert[0]
    ckpt = exl3.Checkpoint.open(d)
    gpu = Gpu(0)
    good = P.Ffn(P.Router(MOE_E, MOE_K), P.SharedExpert(MOE_I), P.RoutedExperts(MOE_E, MOE_K, MOE_I))
    with pytest.raises(InputError, match="layer 1 is planned with a dense MLP"):
        MoeLayer.load(gpu, ckpt, 1, P.DENSE_MLP)
    with pytest.raises(WeightsError, match="layers.0.mlp.gate.weight is missing"):
        MoeLayer.load(gpu, ckpt, 0, good)
    with pytest.raises(WeightsError, match=r"gate.weight: expected \[16\]\[hidden\]"):
        MoeLayer.load(gpu, ckpt, 1, P.Ffn(P.Router(16, MOE_K), P.SharedExpert(MOE_I), P.RoutedExperts(16, MOE_K, MOE_I)))
    with pytest.raises(WeightsError, match="experts.0.gate_proj: 256x128 where the plan has 256x256"):
        MoeLayer.load(gpu, ckpt, 1, P.Ffn(P.Router(MOE_E, MOE_K), P.SharedExpert(MOE_I), P.RoutedExperts(MOE_E, MOE_K, 256)))
    # a gate of the wrong size on the shared expert and a bias on an expert are both refused
    experts, shared, wf = _moe_parts(9700, MOE_I, bits=2)
    tensors = [(f"{MOE_MLP}.gate.weight", "F32", (MOE_E, MOE_H), np.ascontiguousarray(wf.T).tobytes()),
               (f"{MOE_MLP}.shared_expert_gate.weight", "F32", (2, MOE_H), bytes(8 * MOE_H))]
    U.write_checkpoint(tmp_path, tensors, _moe_config(MOE_I))
    with pytest.raises(WeightsError, match=rf"shared_expert_gate.weight: expected \[1\]\[{MOE_H}\]"):
        MoeLayer.load(gpu, exl3.Checkpoint.open(tmp_path), 1, good)


@pytest.mark.parametrize("which", ["per_expert", "stacked"])
def test_cpp_moe_loader_follows_the_plan(request, tmp_path, which):
    case = request.getfixturevalue(f"moe_ckpt_{which}")
    T = 3
    x = _moe_tokens(T)
    x.view(np.uint16).tofile(tmp_path / "x.bin")
    (tmp_path / "meta.txt").write_text(str(T))
    r = _host_check("ckpt-moe", case[0], 1, tmp_path)
    assert r.returncode == 0, r.stdout + r.stderr
    assert (f"ckpt-moe ok layer=1 tokens={T} hidden={MOE_H} experts={MOE_E} top_k={MOE_K} intermediate={MOE_I} "
            f"shared={case[4]}") in r.stdout
    # the stacking order of a pooled expert tensor is this loader's assumption: said once, on stderr
    assert ("convention not fixed by the reference" in r.stderr and "stacked expert tensors" in r.stderr) == \
        (which == "stacked"), r.stderr
    assert ("shared_expert_gate scales the shared expert's row" in r.stderr) == (which == "stacked"), r.stderr
    want, oi, _ = _moe_want(case, x)
    assert np.array_equal(np.fromfile(tmp_path / "idx.bin", dtype=np.int32).reshape(T, MOE_K), oi)
    y = np.fromfile(tmp_path / "y.bin", dtype=np.float32).reshape(T, MOE_H)
    assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max()
    r = _host_check("ckpt-moe", case[0], 0, tmp_path)
    assert r.returncode == 1 and "layers.0.mlp.gate.weight is missing" in r.stderr
    r = _host_check("ckpt-moe", case[0], 9, tmp_path)
    assert r.returncode == 1 and "layer 9 is not in the plan" in r.stderr


def test_biased_linear_and_mlp(ckpt_dir, tmp_path):
    """A linear that carries a bias adds it after the product (y = W x + b), in the Python mirror
    and in the C++ layer; the MLP then takes the four-call path."""
    d, _ = ckpt_dir
    ckpt = exl3.Checkpoint.open(d)
    gpu = Gpu(0)
    tr, suh, svh = synth.linear(8030, H, I, 2)
    bias = (np.arange(I, dtype=np.float32) / 64 - 2).astype(np.float16)
    up = Exl3Linear.load(gpu, ckpt, f"{MLP1}.up_proj")
    assert up.bias is not None
    bare = Exl3Linear(gpu, "bare", tr, suh, svh)
    x = synth.activations(8400, 1, H)
    d_x = gpu.upload(x.view(np.uint16))
    for out, dtype in ((OutDtype.F16, torch.float16), (OutDtype.F32, torch.float32)):
        c = torch.zeros(I, dtype=dtype, device=gpu.device)
        plain = torch.zeros(I, dtype=dtype, device=gpu.device)
        up.forward(gpu, d_x, c, out)
        bare.forward(gpu, d_x, plain, out)
        gpu.synchronize()
        # the bias step itself, bit for bit: one fp32 sum on the linear's output as written, rounded once
        want = plain.cpu().numpy().astype(np.float32) + bias.astype(np.float32)
        assert np.array_equal(c.cpu().numpy(), want.astype(np.float16) if out == OutDtype.F16 else want)
        ref, _ = O.linear(x, tr, suh, svh, H, I, 2, 2, out_fp32=out == OutDtype.F32)
        assert close(c.cpu().numpy(), ref.reshape(-1).astype(np.float32) + bias.astype(np.float32))[0] == 0
    # several rows through the prefill entry
    rows = 5
    xr = synth.activations(8402, rows, H)
    scratch = RowScratch(gpu, rows, H, I)
    c = torch.zeros((rows, I), dtype=torch.float32, device=gpu.device)
    plain = torch.zeros((rows, I), dtype=torch.float32, device=gpu.device)
    up.forward_rows(gpu, scratch, gpu.upload(xr.view(np.uint16)), c, rows, OutDtype.F32)
    bare.forward_rows(gpu, scratch, gpu.upload(xr.view(np.uint16)), plain, rows, OutDtype.F32)
    gpu.synchronize()
    assert np.array_equal(c.cpu().numpy(), plain.cpu().numpy() + bias.astype(np.float32)[None, :])
    mlp = MlpLayer.load(gpu, ckpt, 1)
    assert mlp.has_bias
    xs = (synth.activations(8401, 1, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    y = torch.zeros(H, dtype=torch.float32, device=gpu.device)
    mlp.forward(gpu, gpu.upload(xs.view(np.uint16)), y)
    gpu.synchronize()
    gate, down = synth.linear(8030, H, I, 2), synth.linear(8030, I, H, 2)
    g, _ = O.linear(xs, *gate, H, I, 2, 2)
    u, _ = O.linear(xs, tr, suh, svh, H, I, 2, 2)
    u = (u.reshape(-1).astype(np.float32) + bias.astype(np.float32)).astype(np.float16)
    want, _ = O.linear(O.silu_mul(g, u.reshape(1, I)).reshape(1, I), *down, I, H, 2, 2, out_fp32=True)
    assert np.abs(y.cpu().numpy() - want.reshape(-1)).max() <= 2e-3 * np.abs(want).max()
    # the C++ layer: same layer, same answer
    xs.view(np.uint16).tofile(tmp_path / "x.bin")
    r = _host_check("ckpt-mlp", d, 1, tmp_path)
    assert r.returncode == 0 and "ckpt-mlp ok layer=1" in r.stdout, r.stdout + r.stderr
    yc = np.fromfile(tmp_path / "y.bin", dtype=np.float32)
    assert np.abs(yc - want.reshape(-1)).max() <= 2e-3 * np.abs(want).max()
