"""Seeded sweep of the MoE layer over ragged configurations: token counts on both sides of
the one-token, 8-row and 32-token boundaries, odd and even expert counts, top-k up to the
expert count, intermediate sizes of one to four Hadamard blocks, bit rates 2..5, with and
without a router bias, with no shared expert, one of the routed size (inside the grouped
launches) and one of another size (dense launches).  Bars as in test_gpu_moe: top-k indices
bit-exact, routing weights to 1e-5, every stage within rtol 2e-3 / atol 1e-3 of the oracle on
the inputs that stage consumed, the layer within 2e-3 of the output scale, a second call
bit-identical."""
import os

import numpy as np
import pytest
import torch

from berth_amd import synth
from berth_amd.device import Gpu
from berth_amd.moe import MoeLayer
from oracle import oracle as O
from tests.gpu_util import DEV, dev
from tests.test_gpu_moe import _check_stages, _make_layer

pytestmark = pytest.mark.gpu

TOKENS = [1, 1, 2, 3, 7, 8, 9, 16, 31, 32, 33, 64, 100, 130]


def _cases():
    """BERTH_SWEEP_REPEATS (default 1) passes over the token counts, each with fresh shapes;
    BERTH_SWEEP_SEED shifts the seed."""
    rng = np.random.default_rng(77031 + int(os.environ.get("BERTH_SWEEP_SEED", "0")))
    out = []
    for T in TOKENS * int(os.environ.get("BERTH_SWEEP_REPEATS", "1")):
        H = 128 * int(rng.integers(1, 7))
        E = int(rng.integers(2, 40))
        k = int(rng.integers(1, min(E, 8) + 1))
        I = 128 * int(rng.integers(1, 5))
        bits = int(rng.integers(2, 6))
        shared_I = int(rng.choice([0, 0, I, 128 * int(rng.integers(1, 4))]))
        skew = float(rng.choice([1.0, 1.0, 20.0]))
        out.append((T, H, E, k, I, bits, shared_I, skew))
    return out


@pytest.mark.parametrize("T,H,E,k,I,bits,shared_I,skew", _cases())
def test_moe_layer_ragged_configurations(T, H, E, k, I, bits, shared_I, skew):
    gpu = Gpu(0)
    seed = 13 * T + H + 7 * E + I
    wr, experts_np, experts, shared_np, shared = _make_layer(gpu, seed, H, E, I, bits, shared_I, skew)
    bias = synth.zipf_bias(seed, E) if skew > 1 else None
    layer = MoeLayer(gpu, wr, experts, k, shared=shared, bias=bias)
    x = (synth.activations(seed + 1, T, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    d_x = dev(x.view(np.uint16))
    out = torch.zeros((T, H), dtype=torch.float32, device=DEV)
    idx = torch.zeros((T, k), dtype=torch.int32, device=DEV)
    w = torch.zeros((T, k), dtype=torch.float32, device=DEV)
    layer.forward(gpu, d_x, out, T, idx, w)
    torch.cuda.synchronize()
    want, oi, ow = O.moe_layer(x, wr, experts_np, k, I, bits, 2, bias=bias, shared=shared_np, shared_I=shared_I)
    assert np.array_equal(idx.cpu().numpy(), oi)
    assert np.allclose(w.cpu().numpy(), ow, rtol=1e-5, atol=1e-7)
    _check_stages(layer, x, experts_np, shared_np, oi, w.cpu().numpy(), out.cpu().numpy(), T, H, E, k, I, bits, shared_I)
    err = np.abs(out.cpu().numpy() - want)
    assert err.max() <= 2e-3 * np.abs(want).max(), (err.max(), np.abs(want).max())
    out2 = torch.zeros_like(out)
    layer.forward(gpu, d_x, out2, T)
    torch.cuda.synchronize()
    assert np.array_equal(out2.cpu().numpy().view(np.uint32), out.cpu().numpy().view(np.uint32))


def _route_cases():
    rng = np.random.default_rng(8812 + int(os.environ.get("BERTH_SWEEP_SEED", "0")))
    out = []
    for T in [1, 1, 2, 5, 8, 9, 31, 32, 33, 70, 256, 300] * int(os.environ.get("BERTH_SWEEP_REPEATS", "1")):
        E = int(rng.choice([int(rng.integers(1, 130)), int(rng.integers(130, 1025))]))
        k = int(rng.integers(1, min(E, 32) + 1))
        H = int(rng.choice([64 * int(rng.integers(1, 40)), int(rng.integers(1, 2500))]))
        out.append((T, H, E, k, bool(rng.integers(0, 2)), bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("T,H,E,k,with_bias,renorm", _route_cases())
def test_route_and_permute_ragged(T, H, E, k, with_bias, renorm):
    """Router shapes from one expert to 1024, top-k up to 32, hidden sizes that are not
    multiples of the 64-row segment: logits and top-k bit-exact; then the permutation of the
    selection against the oracle's stable counting sort."""
    from berth_amd import kernels as K
    from tests.test_gpu_moe import _route
    x = synth.activations(T + H + E, T, H)
    wr = synth.router_weight(E + H, H, E)
    bias = synth.zipf_bias(E + 1, E) if with_bias else None
    idx, w, logits = _route(x, wr, k, bias=bias, renorm=renorm)
    oi, ow, ol = O.moe_route(x, wr, k, bias=bias, renorm=renorm, want_logits=True)
    assert np.array_equal(logits.view(np.uint32), ol.view(np.uint32))
    assert np.array_equal(idx, oi)
    assert np.allclose(w, ow, rtol=1e-5, atol=1e-7)
    if T * k <= 65535:
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
