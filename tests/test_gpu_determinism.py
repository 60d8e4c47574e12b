"""The benchmark-sized launches run many times: every repeat must give the bits of the first run
(split-K and shared-tile sums are added in a fixed order, whatever the arrival order of the
workgroups, and a handoff that let a counter overtake partial sums would show up here as a
differing output).  Weights are generated on the device; nothing is compared with the oracle
here, the parity tests do that at sizes the oracle finishes quickly."""
import numpy as np
import pytest
import torch

from berth_amd import synth
from berth_amd.device import Exl3Linear, Exl3MultiLinear, Gpu, MlpLayer, RowScratch
from berth_amd.kernels import OutDtype
from berth_amd.moe import MoeLayer

pytestmark = pytest.mark.gpu


def _rand_lin(gpu, g, name, Kk, N, bits=4):
    tr = torch.randint(0, 65536, (Kk * N * bits // 16,), generator=g, device=gpu.device, dtype=torch.int32).to(torch.int16)
    sc = [((torch.randint(0, 2, (n,), generator=g, device=gpu.device).float() * 2 - 1)
           * torch.exp(0.1 * torch.randn(n, generator=g, device=gpu.device))).half() for n in (Kk, N)]
    return Exl3Linear.from_device(name, tr, sc[0], sc[1], bits)


def _repeat(fn, outs, reps):
    fn()
    torch.cuda.synchronize()
    first = [o.clone() for o in outs]
    assert any(bool(f.ne(0).any()) for f in first)
    for r in range(reps):
        for o in outs:
            o.zero_()
        fn()
        torch.cuda.synchronize()
        for i, (o, f) in enumerate(zip(outs, first)):
            assert torch.equal(o.view(torch.uint8), f.view(torch.uint8)), (r, i)


@pytest.fixture(scope="module")
def layer_set():
    gpu = Gpu(0)
    g = torch.Generator(device=gpu.device)
    g.manual_seed(5)
    lins = {n: _rand_lin(gpu, g, n, *synth.SHAPES_27B[n]) for n in synth.SHAPES_27B}
    return gpu, g, lins


def test_decode_launches_of_the_27b_set_repeat_bit_exactly(layer_set):
    gpu, g, lins = layer_set
    x = {Kk: torch.randn(1, Kk, generator=g, device=gpu.device).half() for Kk in (5120, 6144, 17408)}
    for n, l in lins.items():
        out = torch.zeros(l.size_n, dtype=torch.float16, device=gpu.device)
        _repeat(lambda: l.forward(gpu, x[l.size_k], out, OutDtype.F16), [out], 40)
    qkv = Exl3MultiLinear(gpu, [lins["q_proj"], lins["k_proj"], lins["v_proj"]])
    outs = [torch.zeros((1, lins[n].size_n), dtype=torch.float16, device=gpu.device) for n in ("q_proj", "k_proj", "v_proj")]
    _repeat(lambda: qkv.forward(gpu, x[5120], outs, OutDtype.F16, 1), outs, 40)
    mlp = MlpLayer(gpu, lins["gate_proj"], lins["up_proj"], lins["down_proj"])
    y = torch.zeros(5120, dtype=torch.float32, device=gpu.device)
    xm = (x[5120].float() / 70).half()
    _repeat(lambda: mlp.forward(gpu, xm, y, rows=1), [y], 40)


@pytest.mark.parametrize("rows,reps", [(3, 20), (8, 20), (24, 20), (100, 20), (512, 8)])
def test_row_launches_of_the_27b_set_repeat_bit_exactly(layer_set, rows, reps):
    gpu, g, lins = layer_set
    scratch = RowScratch(gpu, rows, 17408, 17408)
    for n in (("o_proj", "k_proj", "gate_proj", "down_proj") if rows == 512 else ("o_proj", "down_proj")):
        l = lins[n]
        x = torch.randn(rows, l.size_k, generator=g, device=gpu.device).half()
        out = torch.zeros((rows, l.size_n), dtype=torch.float32, device=gpu.device)
        _repeat(lambda: l.forward_rows(gpu, scratch, x, out, rows, OutDtype.F32), [out], reps)


def test_moe_layer_of_config3_repeats_bit_exactly():
    gpu = Gpu(0)
    g = torch.Generator(device=gpu.device)
    g.manual_seed(6)
    H, E, k, I = 2048, 128, 8, 768
    experts = [tuple(_rand_lin(gpu, g, f"e{e}.{j}", *shape) for j, shape in enumerate(((H, I), (H, I), (I, H))))
               for e in range(E)]
    layer = MoeLayer(gpu, synth.router_weight(77, H, E), experts, k)
    for T in (1, 8, 64, 200):
        xt = gpu.upload(synth.activations(300 + T, T, H).view(np.uint16))
        out = torch.zeros((T, H), dtype=torch.float32, device=gpu.device)
        _repeat(lambda: layer.forward(gpu, xt, out, T), [out], 30)
