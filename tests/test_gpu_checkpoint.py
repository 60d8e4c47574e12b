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

from berth_amd import exl3, synth
from berth_amd.device import Exl3Linear, Gpu, MlpLayer, WeightsError
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
    # a half-integer rate (1.5 bpw: 24 words per tile) and a biased MLP, both refused by the loaders
    tensors += U.linear_tensors("attn.half", np.zeros((H // 16, 128 // 16, 24), np.uint16), *synth.linear(1, H, 128, 1)[1:])
    for part, (k, n) in (("gate_proj", (H, I)), ("up_proj", (H, I)), ("down_proj", (I, H))):
        tensors += U.linear_tensors(f"{MLP1}.{part}", *synth.linear(8030, k, n, 2),
                                    bias=np.zeros(n, np.float16) if part == "up_proj" else None)
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
    with pytest.raises(WeightsError, match="up_proj: bias is present and is not applied"):
        MlpLayer.load(gpu, ckpt, 1)
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
    r = _host_check("ckpt-mlp", d, 1, tmp_path)
    assert r.returncode == 1 and "up_proj: bias is present and is not applied" in r.stderr
    r = _host_check("ckpt-linear", d, "attn.half", tmp_path)
    assert r.returncode == 1 and "attn.half: half-integer rate" in r.stderr
    r = _host_check("ckpt-linear", d, "nope", tmp_path)
    assert r.returncode == 1 and "nope is not an EXL3 linear" in r.stderr
