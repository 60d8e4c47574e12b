"""Seeded sweeps of the launches that carry several linears: sliced multi-linear bundles
(`berth_ops_mgemm`, the q/k/v and gate/up bundles of decode) and the MLP block in one call
(`berth_exl3_mlp`), over ragged widths, row counts 1..8 and the MFMA route above 8, bit rates
and output types.  Bars as in the fixed-shape tests of the same entry points."""
import os

import numpy as np
import pytest
import torch

from berth_amd import kernels as K
from berth_amd import synth
from berth_amd.device import Exl3Linear, Exl3MultiLinear, Gpu
from berth_amd.kernels import OutDtype
from oracle import oracle as O
from tests.gpu_util import DEV, close, dev, host_f16, host_u16
from tests.test_gpu_mlp import test_fused_mlp_stage_by_stage as _mlp_case

pytestmark = pytest.mark.gpu

REPEATS = int(os.environ.get("BERTH_SWEEP_REPEATS", "1"))
SEED = int(os.environ.get("BERTH_SWEEP_SEED", "0"))


def _bundle_cases():
    rng = np.random.default_rng(5150 + SEED)
    out = []
    for _ in range(12 * REPEATS):
        rows = int(rng.integers(1, 9))
        Kk = 128 * int(rng.integers(1, 17))
        unit = 128 * int(rng.integers(1, 4))
        widths = tuple(unit * int(rng.integers(1, 7)) for _ in range(int(rng.integers(2, 5))))
        out.append((rows, Kk, widths, int(rng.integers(2, 7)), bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("rows,Kk,widths,bits,fp32", _bundle_cases())
def test_sliced_bundle_ragged(rows, Kk, widths, bits, fp32):
    gpu = Gpu(0)
    seed = 3 * rows + Kk + sum(widths) + bits
    lins_np = [synth.linear(seed + 11 * i, Kk, n, bits) for i, n in enumerate(widths)]
    multi = Exl3MultiLinear(gpu, [Exl3Linear(gpu, f"l{i}", *l) for i, l in enumerate(lins_np)])
    x = synth.activations(seed + 5, rows, Kk)
    outs = [torch.zeros((rows, n), dtype=torch.float32 if fp32 else torch.float16, device=DEV) for n in widths]
    multi.forward(gpu, dev(x.view(np.uint16)), outs, OutDtype.F32 if fp32 else OutDtype.F16, rows)
    torch.cuda.synchronize()
    launch = K.ops.last_launch()
    assert "sliced" in launch, launch
    first = [o.cpu().numpy().copy() for o in outs]
    for i, (tr, suh, svh) in enumerate(lins_np):
        want, want_had = O.linear(x, tr, suh, svh, Kk, widths[i], bits, 2, out_fp32=fp32)
        got = first[i] if fp32 else host_f16(outs[i])
        bad, worst = close(got, want)
        assert bad == 0, (i, bad, worst, launch)
        slab = host_u16(multi.a_had)[i * rows * Kk:(i + 1) * rows * Kk]
        assert np.array_equal(slab, want_had.view(np.uint16).reshape(-1)), (i, launch)
    multi.forward(gpu, dev(x.view(np.uint16)), outs, OutDtype.F32 if fp32 else OutDtype.F16, rows)
    torch.cuda.synchronize()
    for i in range(len(widths)):
        assert np.array_equal(outs[i].cpu().numpy().view(np.uint8), first[i].view(np.uint8)), (i, launch)


def _many_row_cases():
    rng = np.random.default_rng(7370 + SEED)
    out = []
    for rows in [9, 31, 32, 33, 100, 129, 257, 300] * REPEATS:
        Kk = 128 * int(rng.integers(1, 9))
        unit = 128 * int(rng.integers(1, 4))
        widths = tuple(unit * int(rng.integers(1, 7)) for _ in range(int(rng.integers(2, 5))))
        out.append((rows, Kk, widths, int(rng.integers(2, 6)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("rows,Kk,widths,bits,fp32,host_lists", _many_row_cases())
def test_sliced_bundle_many_rows(rows, Kk, widths, bits, fp32, host_lists):
    """More than 8 rows: the bundle is one dense MFMA launch (32-, 128- or 256-row tiles by row
    count and width) behind one launch that rotates the input once per source.  Each source
    against the oracle's single linear, the rotated slabs bit for bit, lists by value and from
    device memory, and a second call for the same bits."""
    gpu = Gpu(0)
    seed = 7 * rows + Kk + sum(widths) + bits
    lins_np = [synth.linear(seed + 11 * i, Kk, n, bits) for i, n in enumerate(widths)]
    multi = Exl3MultiLinear(gpu, [Exl3Linear(gpu, f"l{i}", *l) for i, l in enumerate(lins_np)])
    x = synth.activations(seed + 5, rows, Kk)
    odt = OutDtype.F32 if fp32 else OutDtype.F16
    outs = [torch.zeros((rows, n), dtype=torch.float32 if fp32 else torch.float16, device=DEV) for n in widths]
    d_x = dev(x.view(np.uint16))
    by_value = host_lists and multi.slices <= 16
    multi.forward(gpu, d_x, outs, odt, rows, by_value=by_value)
    want_text = "by value" if by_value else "sliced x"
    torch.cuda.synchronize()
    launch = K.ops.last_launch()
    assert want_text in launch and "had_r_128_slabs_kernel" in launch and "exl3_gemm" in launch, launch
    first = [o.cpu().numpy().copy() for o in outs]
    for i, (tr, suh, svh) in enumerate(lins_np):
        want, want_had = O.linear(x, tr, suh, svh, Kk, widths[i], bits, 2, out_fp32=fp32)
        got = first[i] if fp32 else host_f16(outs[i])
        bad, worst = close(got, want)
        assert bad == 0, (i, bad, worst, launch)
        slab = host_u16(multi.a_had)[i * rows * Kk:(i + 1) * rows * Kk]
        assert np.array_equal(slab, want_had.view(np.uint16).reshape(-1)), (i, launch)
    multi.forward(gpu, d_x, outs, odt, rows, by_value=by_value)
    torch.cuda.synchronize()
    for i in range(len(widths)):
        assert np.array_equal(outs[i].cpu().numpy().view(np.uint8), first[i].view(np.uint8)), (i, launch)


@pytest.mark.parametrize("rows,shared_input", [(12, True), (40, False), (150, True)])
def test_uniform_bundle_many_rows(rows, shared_input):
    """Uniform mode above 8 rows: n linears of one shape, outputs [n][rows][N] behind one
    pointer, one input for all or one per linear; every linear has its own input scales, so
    every slab of the rotated input is its own."""
    from berth_amd.kernels import Codebook
    Kk, N, n_mat = 384, 640, 3
    lins = [synth.linear(900 + i + rows, Kk, N, 4) for i in range(n_mat)]
    x = synth.activations(910 + rows, n_mat * rows, Kk).reshape(n_mat, rows, Kk)
    d = [[dev(t.view(np.uint16)) for t in lin] for lin in lins]
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=DEV)
    b_list, suh_list, svh_list = (i64([dd[j].data_ptr() for dd in d]) for j in range(3))
    d_x = dev(x.view(np.uint16))
    c = torch.zeros((n_mat, rows, N), dtype=torch.float16, device=DEV)
    a_had = torch.zeros((n_mat, rows, Kk), dtype=torch.float16, device=DEV)
    rc = K.ops.exl3_mgemm(d_x.data_ptr(), b_list.data_ptr(), c.data_ptr(), suh_list.data_ptr(), a_had.data_ptr(),
                          svh_list.data_ptr(), rows, Kk, N, 4, Codebook.MUL1, OutDtype.F16, 1 if shared_input else n_mat,
                          n_mat)
    torch.cuda.synchronize()
    assert rc > 0 and "uniform x3" in K.ops.last_launch(), K.ops.last_launch()
    got = host_f16(c).reshape(n_mat, rows, N)
    for i, (tr, suh, svh) in enumerate(lins):
        xi = x[0] if shared_input else x[i]
        want, want_had = O.linear(np.ascontiguousarray(xi), tr, suh, svh, Kk, N, 4, 2, out_fp32=False)
        bad, worst = close(got[i], want)
        assert bad == 0, (i, bad, worst)
        assert np.array_equal(host_u16(a_had).reshape(n_mat, rows * Kk)[i], want_had.view(np.uint16).reshape(-1)), i


def _mlp_cases():
    rng = np.random.default_rng(6260 + SEED)
    rows_list = [1, 1, 2, 5, 8, 9, 20, 33]
    return [(rows, 128 * int(rng.integers(1, 9)), 128 * int(rng.integers(1, 25)), int(rng.integers(2, 6)))
            for rows in rows_list * REPEATS]


@pytest.mark.parametrize("rows,H,I,bits", _mlp_cases())
def test_mlp_block_ragged(rows, H, I, bits):
    _mlp_case(rows, H, I, bits)
