"""The decode launches recorded into a HIP graph and replayed: every replay must give the
bits of the eager launch.  The split-K arrival counters reset themselves inside the
kernels and no launch of this library clears memory with a memset node, so nothing in a
recorded launch depends on state a replay does not restore.  Eager work of the same
library runs between the replays (it shares the split-K workspace and the counters)."""
import numpy as np
import pytest
import torch

from berth_amd import synth
from berth_amd.device import Exl3Linear, Gpu, MlpLayer
from berth_amd.kernels import OutDtype
from berth_amd.moe import MoeLayer
from tests.gpu_util import host_f16

pytestmark = pytest.mark.gpu


def _capture(gpu, fn):
    """fn() once eagerly on a side stream (warm-up: the library allocates its workspace on
    first use, which must not happen under capture), then recorded."""
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=gpu.device)
    side.wait_stream(torch.cuda.current_stream(gpu.device))
    with torch.cuda.stream(side):
        fn()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            fn()
    torch.cuda.current_stream(gpu.device).wait_stream(side)
    torch.cuda.synchronize()
    return graph


def test_split_k_gemv_and_mlp_block_replay_bit_exact():
    gpu = Gpu(0)
    H, I, bits = 1024, 2816, 4
    lins = [Exl3Linear(gpu, n, *synth.linear(4100 + 3 * j, *shape, bits))
            for j, (n, shape) in enumerate((("gate", (H, I)), ("up", (H, I)), ("down", (I, H))))]
    mlp = MlpLayer(gpu, *lins, max_rows=1)
    other = Exl3Linear(gpu, "other", *synth.linear(4200, 2048, 768, bits))
    xs = [gpu.upload((synth.activations(4300 + i, 1, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
                     .view(np.uint16)) for i in range(3)]
    x = torch.zeros_like(xs[0])
    y_lin = torch.zeros(I, dtype=torch.float16, device=gpu.device)
    y_mlp = torch.zeros(H, dtype=torch.float32, device=gpu.device)
    x_other = gpu.upload(synth.activations(4400, 1, 2048).view(np.uint16))
    y_other = torch.zeros(768, dtype=torch.float32, device=gpu.device)

    def step():
        lins[0].forward(gpu, x, y_lin, OutDtype.F16)        # split-K GEMV
        mlp.forward(gpu, x, y_mlp, rows=1)                  # pair launch + SiLU-gated down projection

    want = []
    for xi in xs:
        x.copy_(xi)
        step()
        torch.cuda.synchronize()
        want.append((host_f16(y_lin).copy(), y_mlp.cpu().numpy().copy()))
    assert not np.array_equal(want[0][1], want[1][1])

    graph = _capture(gpu, step)
    for rep in range(6):
        x.copy_(xs[rep % 3])
        y_lin.zero_()
        y_mlp.zero_()
        graph.replay()
        torch.cuda.synchronize()
        got_lin, got_mlp = host_f16(y_lin), y_mlp.cpu().numpy()
        assert np.array_equal(got_lin.view(np.uint16), want[rep % 3][0].view(np.uint16)), rep
        assert np.array_equal(got_mlp.view(np.uint32), want[rep % 3][1].view(np.uint32)), rep
        # eager work of the same library between replays
        other.forward(gpu, x_other, y_other, OutDtype.F32)
        torch.cuda.synchronize()


@pytest.mark.parametrize("T", [1, 40])
def test_moe_layer_replays_bit_exact(T):
    """One token (route with the sort, two grouped launches) and forty tokens (two route
    launches, permute, rotated rows, grouped MFMA launches, combine)."""
    gpu = Gpu(0)
    H, E, k, I, bits = 512, 16, 4, 256, 4
    experts = []
    for e in range(E):
        experts.append(tuple(Exl3Linear(gpu, f"e{e}.{n}", *synth.linear(5000 + 10 * e + 3 * j, *shape, bits))
                             for j, (n, shape) in enumerate((("gate", (H, I)), ("up", (H, I)), ("down", (I, H))))))
    layer = MoeLayer(gpu, synth.router_weight(51, H, E), experts, k)
    xs = [gpu.upload(synth.activations(5200 + i, T, H).view(np.uint16)) for i in range(3)]
    x = torch.zeros_like(xs[0])
    out = torch.zeros((T, H), dtype=torch.float32, device=gpu.device)

    def step():
        layer.forward(gpu, x, out, T)

    want = []
    for xi in xs:
        x.copy_(xi)
        step()
        torch.cuda.synchronize()
        want.append(out.cpu().numpy().copy())
    assert not np.array_equal(want[0], want[1])

    graph = _capture(gpu, step)
    for rep in range(6):
        x.copy_(xs[rep % 3])
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want[rep % 3].view(np.uint32)), rep
        x.copy_(xs[(rep + 1) % 3])
        step()                                              # eager call of the same layer in between
        torch.cuda.synchronize()


@pytest.mark.parametrize("rows,Kk,N", [(24, 1024, 768), (200, 512, 8320), (300, 256, 16640)])
def test_row_launches_replay_bit_exact(rows, Kk, N):
    """The input rotation pre-pass and the MFMA kernels (32-row tiles with split-K, evenly dealt
    128-row tiles, 256-row tiles): shared tiles are finished through self-resetting counters."""
    from berth_amd.device import RowScratch
    gpu = Gpu(0)
    lin = Exl3Linear(gpu, "rows", *synth.linear(6100 + rows, Kk, N, 4))
    scratch = RowScratch(gpu, rows, Kk, N)
    xs = [gpu.upload(synth.activations(6200 + i, rows, Kk).view(np.uint16)) for i in range(2)]
    x = torch.zeros_like(xs[0])
    out = torch.zeros((rows, N), dtype=torch.float32, device=gpu.device)

    def step():
        lin.forward_rows(gpu, scratch, x, out, rows, OutDtype.F32)

    want = []
    for xi in xs:
        x.copy_(xi)
        step()
        torch.cuda.synchronize()
        want.append(out.cpu().numpy().copy())
    graph = _capture(gpu, step)
    for rep in range(6):
        x.copy_(xs[rep % 2])
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want[rep % 2].view(np.uint32)), rep
        x.copy_(xs[(rep + 1) % 2])
        step()
        torch.cuda.synchronize()
