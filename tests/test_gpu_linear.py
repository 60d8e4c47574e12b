"""GPU parity of the EXL3 linear path against the CPU oracle, through the C ABI.

Bars: dequantised weights, rotated activations (a_had), Hadamard rows and the
SiLU gate are bit-exact; linear outputs are within rtol 2e-3 / atol 1e-3 of the
oracle's fp32 matmul over the oracle-decoded weights."""
import os

import numpy as np
import pytest
import torch

from berth_amd import kernels as K
from berth_amd import synth
from berth_amd.device import Exl3Linear, Gpu
from berth_amd.kernels import Codebook, OutDtype
from oracle import oracle as O
from tests.gpu_util import DEV, close, dev, host_f16, host_u16

pytestmark = pytest.mark.gpu


def _reconstruct(tr, Kk, N, bits, cb, n_offset=0, slice_n=None):
    slice_n = slice_n or N
    out = torch.zeros((Kk, slice_n), dtype=torch.float16, device=DEV)
    d_tr = dev(tr)
    K.prefill_lin.reconstruct(out.data_ptr(), d_tr.data_ptr(), Kk, slice_n, N, n_offset, bits, Codebook(cb))
    torch.cuda.synchronize()
    return host_u16(out)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("cb", [0, 1, 2])
def test_dequant_bit_exact(bits, cb):
    Kk, N = 144, 384            # 9 tile rows (not a multiple of the 4 a workgroup takes)
    tr = synth.trellis_words(1000 + 10 * bits + cb, Kk, N, bits)
    got = _reconstruct(tr, Kk, N, bits, cb)
    want = O.dequant(tr, Kk, N, bits, cb).view(np.uint16)
    assert np.array_equal(got, want)


def test_dequant_every_state_of_every_codebook():
    """A 4 bpw trellis built so that all 65536 states occur: a de Bruijn-like
    sweep is not needed, 8 bpw tiles expose two arbitrary bytes per state."""
    Kk, N = 256, 256            # 256 tiles x 256 states = 65536 states at 8 bpw
    words = np.arange(65536, dtype=np.uint32)
    # at 8 bpw state t = bytes (t-1, t) of the stream: lay all 16-bit values out as byte pairs
    stream = np.zeros((256, 256), dtype=np.uint8)
    rng = np.random.default_rng(0)
    stream[:] = rng.integers(0, 256, size=(256, 256), dtype=np.uint8)
    tr = (stream[:, 0::2].astype(np.uint16) << 8 | stream[:, 1::2]).reshape(16, 16, 128)
    for cb in (0, 1, 2):
        got = _reconstruct(tr, Kk, N, 8, cb)
        want = O.dequant(tr, Kk, N, 8, cb).view(np.uint16)
        assert np.array_equal(got, want)
    del words


def test_dequant_column_slice():
    Kk, N, bits = 64, 512, 4
    tr = synth.trellis_words(5, Kk, N, bits)
    want = O.dequant(tr, Kk, N, bits, 2).view(np.uint16)
    got = _reconstruct(tr, Kk, N, bits, 2, n_offset=128, slice_n=256)
    assert np.array_equal(got, want[:, 128:384])


def test_dequant_full_size_config0_is_bit_exact():
    Kk = N = 4096
    tr = synth.trellis_words(0, Kk, N, 4)
    got = _reconstruct(tr, Kk, N, 4, 2)
    want = O.dequant(tr, Kk, N, 4, 2).view(np.uint16)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("Kk,N,bits,cb,n_offset,slice_n", [(256, 384, 4, 2, 0, None), (128, 128, 3, 2, 0, None),
                                                          (384, 512, 4, 2, 128, 256), (256, 256, 5, 0, 0, None),
                                                          (1024, 1280, 4, 2, 256, 1024), (128, 256, 2, 1, 128, 128)])
def test_reconstruct_had_bit_exact(Kk, N, bits, cb, n_offset, slice_n):
    """The effective weight diag(suh) Hh W Hh diag(svh) (the reference's weight for 1024 rows and
    more, crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:96-123), whole and as a column
    slice, against the oracle: same butterfly order, one rounding, so the same bits."""
    tr, suh, svh = synth.linear(77 + Kk + bits, Kk, N, bits)
    slice_n = slice_n or N
    d_tr, d_suh, d_svh = dev(tr), dev(suh.view(np.uint16)), dev(svh.view(np.uint16))
    out = torch.zeros((Kk, slice_n), dtype=torch.float16, device=DEV)
    K.prefill_lin.reconstruct_had(out.data_ptr(), d_tr.data_ptr(), d_suh.data_ptr(), d_svh.data_ptr(), Kk, slice_n, N,
                                  n_offset, bits, Codebook(cb))
    torch.cuda.synchronize()
    assert "exl3_reconstruct_had_kernel" in K.prefill_lin.last_launch()
    want = O.reconstruct_had(tr, suh, svh, Kk, N, bits, cb).view(np.uint16)
    assert np.array_equal(host_u16(out), want[:, n_offset:n_offset + slice_n])


def test_reconstruct_had_then_plain_gemm_is_the_operator():
    """a @ W_eff through berth_prefill_hgemm against the fused linear of the same rows: the two
    routes round in different places (W_eff to fp16 here, the rotated activation there), so the
    bar is a relative one over the whole output."""
    m, Kk, N, bits = 48, 512, 768, 4
    tr, suh, svh = synth.linear(901, Kk, N, bits)
    x = synth.activations(902, m, Kk)
    d_tr, d_suh, d_svh, d_x = dev(tr), dev(suh.view(np.uint16)), dev(svh.view(np.uint16)), dev(x.view(np.uint16))
    w_eff = torch.zeros((Kk, N), dtype=torch.float16, device=DEV)
    K.prefill_lin.reconstruct_had(w_eff.data_ptr(), d_tr.data_ptr(), d_suh.data_ptr(), d_svh.data_ptr(), Kk, N, N, 0,
                                  bits, Codebook.MUL1)
    c = torch.zeros((m, N), dtype=torch.float32, device=DEV)
    K.prefill_lin.hgemm(d_x.data_ptr(), w_eff.data_ptr(), c.data_ptr(), m, Kk, N, N, OutDtype.F32)
    torch.cuda.synchronize()
    want, _ = O.linear(x, tr, suh, svh, Kk, N, bits, 2, out_fp32=True)
    got = c.cpu().numpy().astype(np.float64)
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel < 5e-4, rel


@pytest.mark.parametrize("pre", [True, False])
@pytest.mark.parametrize("fp32", [False, True])
def test_had_r_128_bit_exact(pre, fp32):
    rows, cols = 5, 384
    sc = synth.sign_scale(3, cols)
    x16 = synth.activations(4, rows, cols)
    d_sc = dev(sc.view(np.uint16))
    if fp32:
        x = (x16.astype(np.float32) * 3.7).astype(np.float32)
        d_x = torch.from_numpy(x).to(DEV)
        d_o = torch.zeros_like(d_x)
        K.prefill_lin.had_r_128(d_x.data_ptr(), d_o.data_ptr(), d_sc.data_ptr(), pre, rows, cols, True)
        torch.cuda.synchronize()
        want = O.had_rows_f32(x, sc, pre)
        assert np.array_equal(d_o.cpu().numpy().view(np.uint32), want.view(np.uint32))
    else:
        d_x = dev(x16.view(np.uint16))
        d_o = torch.zeros_like(d_x)
        K.prefill_lin.had_r_128(d_x.data_ptr(), d_o.data_ptr(), d_sc.data_ptr(), pre, rows, cols, False)
        torch.cuda.synchronize()
        want = O.had_rows_f16(x16, sc, pre).view(np.uint16)
        assert np.array_equal(host_u16(d_o), want)


@pytest.mark.parametrize("rows,cols", [(1, 128), (3, 256), (7, 640), (33, 1152), (700, 12032), (513, 17408)])
def test_had_r_128_ragged_sizes_bit_exact(rows, cols):
    """Block counts that are not multiples of the four blocks a wave takes, and tensors with
    more blocks than one pass of the grid covers (the kernel strides over them); in place too."""
    sc = synth.sign_scale(rows + cols, cols)
    x16 = synth.activations(rows * 3 + cols, rows, cols)
    d_sc = dev(sc.view(np.uint16))
    for pre in (True, False):
        d_x = dev(x16.view(np.uint16))
        d_o = torch.zeros_like(d_x)
        K.prefill_lin.had_r_128(d_x.data_ptr(), d_o.data_ptr(), d_sc.data_ptr(), pre, rows, cols, False)
        torch.cuda.synchronize()
        want = O.had_rows_f16(x16, sc, pre).view(np.uint16)
        assert np.array_equal(host_u16(d_o).reshape(rows, cols), want)
        K.prefill_lin.had_r_128(d_x.data_ptr(), d_x.data_ptr(), d_sc.data_ptr(), pre, rows, cols, False)   # in place
        torch.cuda.synchronize()
        assert np.array_equal(host_u16(d_x).reshape(rows, cols), want)
    x32 = (x16.astype(np.float32) * 1.7).astype(np.float32)
    d_x = torch.from_numpy(x32).to(DEV)
    d_o = torch.zeros_like(d_x)
    K.prefill_lin.had_r_128(d_x.data_ptr(), d_o.data_ptr(), d_sc.data_ptr(), False, rows, cols, True)
    torch.cuda.synchronize()
    assert np.array_equal(d_o.cpu().numpy().view(np.uint32), O.had_rows_f32(x32, sc, False).view(np.uint32))


def test_silu_mul_reference_fixture_bit_exact(golden_dir):
    g = np.fromfile(os.path.join(golden_dir, "silu.gate.bin"), dtype=np.uint16)
    u = np.fromfile(os.path.join(golden_dir, "silu.up.bin"), dtype=np.uint16)
    want = np.fromfile(os.path.join(golden_dir, "silu.out.bin"), dtype=np.uint16)
    d_g, d_u = dev(g), dev(u)
    K.ops.silu_mul(d_g.data_ptr(), d_u.data_ptr(), d_u.data_ptr(), g.size, 0.0)   # in place on up
    torch.cuda.synchronize()
    assert "silu_mul_kernel" in K.ops.last_launch()
    assert np.array_equal(host_u16(d_u), want)


def test_silu_mul_random_matches_oracle():
    rng = np.random.default_rng(8)
    g = (rng.normal(size=4096) * 4).astype(np.float16)
    u = (rng.normal(size=4096) * 4).astype(np.float16)
    d_g, d_u, d_o = dev(g.view(np.uint16)), dev(u.view(np.uint16)), torch.zeros(4096, dtype=torch.float16, device=DEV)
    K.ops.silu_mul(d_g.data_ptr(), d_u.data_ptr(), d_o.data_ptr(), 4096, 0.0)
    torch.cuda.synchronize()
    want = O.silu_mul(g, u).view(np.uint16)
    d = np.abs(host_u16(d_o).view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32))
    assert d.max() <= 1 and (d == 0).mean() > 0.999


def _run_linear(m, Kk, N, bits, cb, out_fp32, seed, prefill=False):
    tr, suh, svh = synth.linear(seed, Kk, N, bits)
    x = synth.activations(seed + 7, m, Kk)
    d = {k: dev(v.view(np.uint16)) for k, v in dict(tr=tr, suh=suh, svh=svh, x=x).items()}
    c = torch.zeros((m, N), dtype=torch.float32 if out_fp32 else torch.float16, device=DEV)
    a_had = torch.zeros((m, Kk), dtype=torch.float16, device=DEV)
    out = OutDtype.F32 if out_fp32 else OutDtype.F16
    if prefill:
        w = torch.zeros(Kk * min(N, 32768), dtype=torch.float16, device=DEV) if m > 144 else None
        K.prefill_lin.exl3_linear(d["x"].data_ptr(), d["tr"].data_ptr(), c.data_ptr(), d["suh"].data_ptr(),
                                  a_had.data_ptr(), d["svh"].data_ptr(), w.data_ptr() if w is not None else None,
                                  m, Kk, N, bits, Codebook(cb), out)
        launch = K.prefill_lin.last_launch()
    else:
        K.exl3_linear(d["x"].data_ptr(), d["tr"].data_ptr(), c.data_ptr(), d["suh"].data_ptr(),
                      a_had.data_ptr(), d["svh"].data_ptr(), m, Kk, N, bits, Codebook(cb), out)
        launch = K.last_launch()
    torch.cuda.synchronize()
    want, want_had = O.linear(x, tr, suh, svh, Kk, N, bits, cb, out_fp32=out_fp32)
    got = c.cpu().numpy() if out_fp32 else host_f16(c)
    return got, want, host_u16(a_had), want_had.view(np.uint16), launch


@pytest.mark.parametrize("bits,cb", [(4, 2), (2, 2), (3, 2), (5, 2), (6, 2), (8, 2), (1, 2), (4, 0), (4, 1), (3, 1)])
@pytest.mark.parametrize("out_fp32", [False, True])
def test_gemv_m1(bits, cb, out_fp32):
    got, want, ah, want_ah, launch = _run_linear(1, 512, 384, bits, cb, out_fp32, 50 + bits)
    assert "exl3_gemv_kernel" in launch
    assert np.array_equal(ah, want_ah)
    bad, worst = close(got, want)
    assert bad == 0, (bad, worst)


@pytest.mark.parametrize("Kk,N", [(128, 128), (4096, 4096), (5120, 1024), (1024, 5120), (2048, 768), (768, 2048)])
def test_gemv_m1_shapes_split_k(Kk, N):
    got, want, ah, want_ah, launch = _run_linear(1, Kk, N, 4, 2, True, Kk + N)
    assert np.array_equal(ah, want_ah)
    bad, worst = close(got, want)
    assert bad == 0, (bad, worst, launch)


@pytest.mark.parametrize("Kk,N,bits,half", [(2048, 768, 4, True), (768, 2048, 3, True), (128, 128, 5, True),
                                             (384, 256, 2, True), (4096, 4096, 4, True), (5120, 8192, 4, False), (2048, 768, 4, None)])
def test_gemv_m1_half_k_block_units(Kk, N, bits, half):
    """One-row launches with few column blocks and k-blocks walk half k-blocks (two waves
    share a k-block: both rotate it, each decodes 4 of its 8 tile rows, the first writes the
    rotated activation); wide ones keep whole k-blocks.  half=None: the same shape with
    half units switched off, in a fresh process (the switch is read once)."""
    if half is None:
        import subprocess, sys
        code = ("import numpy as np\nfrom tests.test_gpu_linear import _run_linear\nfrom tests.gpu_util import close\n"
                f"got, want, ah, want_ah, launch = _run_linear(1, {Kk}, {N}, {bits}, 2, True, 7)\n"
                "assert '/half' not in launch, launch\nassert np.array_equal(ah, want_ah)\n"
                "assert close(got, want)[0] == 0\nprint('ok')\n")
        env = dict(os.environ, BERTH_GEMV_HALF_UNITS="0")
        r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=240,
                           cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
        assert r.returncode == 0 and "ok" in r.stdout, r.stdout + r.stderr
        return
    got, want, ah, want_ah, launch = _run_linear(1, Kk, N, bits, 2, True, 7)
    assert ("/half" in launch) == half, launch
    assert np.array_equal(ah, want_ah), launch
    bad, worst = close(got, want)
    assert bad == 0, (bad, worst, launch)


def test_gemv_m1_is_deterministic_and_counters_reset():
    outs = []
    for _ in range(3):
        got, _, _, _, launch = _run_linear(1, 4096, 512, 4, 2, True, 99)
        outs.append(got.view(np.uint32).copy())
    assert "split_k=" in launch and "split_k=1 " not in launch
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


@pytest.mark.parametrize("m", [2, 3, 4, 5, 8])
def test_gemv_small_rows(m):
    got, want, ah, want_ah, launch = _run_linear(m, 512, 256, 4, 2, m % 2 == 0, 70 + m, prefill=True)
    assert "exl3_gemv_kernel" in launch
    assert np.array_equal(ah, want_ah)
    bad, worst = close(got, want)
    assert bad == 0, (bad, worst)


@pytest.mark.parametrize("m", [9, 32, 47, 144, 145, 200])
@pytest.mark.parametrize("out_fp32", [False, True])
def test_gemm_rows(m, out_fp32):
    got, want, ah, want_ah, launch = _run_linear(m, 512, 384, 4, 2, out_fp32, 80 + m, prefill=True)
    assert "exl3_gemm_kernel" in launch
    assert np.array_equal(ah, want_ah)
    bad, worst = close(got, want)
    assert bad == 0, (bad, worst)


@pytest.mark.parametrize("bits,cb", [(2, 2), (3, 2), (5, 2), (6, 2), (4, 0), (4, 1)])
def test_gemm_other_rates(bits, cb):
    got, want, ah, want_ah, _ = _run_linear(64, 256, 256, bits, cb, True, 90 + bits, prefill=True)
    assert np.array_equal(ah, want_ah)
    bad, worst = close(got, want)
    assert bad == 0, (bad, worst)


@pytest.mark.parametrize("m,Kk,N", [(16, 4096, 256), (24, 5120, 1024), (32, 2048, 768), (33, 2048, 512), (100, 4096, 256)])
def test_gemm_split_k(m, Kk, N):
    got, want, ah, want_ah, launch = _run_linear(m, Kk, N, 4, 2, True, 300 + m, prefill=True)
    assert "split_k=" in launch and "split_k=1 " not in launch, launch
    assert np.array_equal(ah, want_ah)
    bad, worst = close(got, want)
    assert bad == 0, (bad, worst, launch)
    got2, _, _, _, _ = _run_linear(m, Kk, N, 4, 2, True, 300 + m, prefill=True)
    assert np.array_equal(got.view(np.uint32), got2.view(np.uint32))


def _check_balanced(m, Kk, N, fp32, tile, bits=4, cb=2):
    got, want, ah, want_ah, launch = _run_linear(m, Kk, N, bits, cb, fp32, 700 + m, prefill=True)
    name = "exl3_gemm_wide_kernel" if tile == 256 else "exl3_gemm_balanced_kernel"
    assert f"{name}<{bits},{cb},{tile}x256>" in launch, launch
    assert np.array_equal(ah, want_ah)
    bad, worst = close(got, want)
    assert bad == 0, (bad, worst, launch)
    got2, _, _, _, _ = _run_linear(m, Kk, N, bits, cb, fp32, 700 + m, prefill=True)
    assert np.array_equal(got.view(np.uint16), got2.view(np.uint16))


@pytest.mark.parametrize("m,Kk,N,fp32", [(128, 1024, 16384, True), (100, 640, 16640, False), (65, 256, 17408, True)])
def test_gemm_128_row_tiles_dealt_out_evenly(m, Kk, N, fp32):
    """Enough 128 x 256 tiles to use them: the (tile, k-block) units are cut into one equal
    range per compute unit, tiles shared by several workgroups are summed in k order."""
    _check_balanced(m, Kk, N, fp32, 128)


@pytest.mark.parametrize("m,Kk,N,fp32,bits", [(512, 512, 16384, True, 4), (300, 256, 16640, False, 4),
                                              (640, 256, 11008, True, 3)])
def test_gemm_256_row_tiles_dealt_out_evenly(m, Kk, N, fp32, bits):
    """More than 128 rows and at least half as many 256 x 256 tiles as compute units: tiles
    of eight waves; every weight is decoded once per tile and reaches the MFMA waves through
    LDS.  Dealt out the same way.  The last row tile may be short (44 or 128 rows)."""
    _check_balanced(m, Kk, N, fp32, 256, bits)


@pytest.mark.parametrize("m,Kk,N,tile,bits,cb", [(128, 512, 16384, 128, 2, 2), (96, 384, 16640, 128, 3, 2),
                                                 (128, 256, 16384, 128, 5, 2), (70, 256, 16384, 128, 6, 2),
                                                 (128, 384, 16384, 128, 4, 0), (100, 256, 16640, 128, 4, 1),
                                                 (128, 256, 16384, 128, 8, 2), (512, 384, 16384, 256, 2, 2),
                                                 (300, 256, 16640, 256, 5, 2), (512, 256, 16384, 256, 4, 1),
                                                 (260, 256, 16384, 256, 6, 0)])
def test_gemm_pipelined_tiles_other_rates_and_codebooks(m, Kk, N, tile, bits, cb):
    """The 128- and 256-row loops issue the decode of the next half-step (128 rows) or macro-step
    (256 rows) behind the MFMAs of the current one; the scheduling groups that hold that order
    are sized for 4 bpw with the mul1 codebook.  Every other bit rate and both other codebooks
    through the same loops: same results as the oracle, same bits on a second run."""
    _check_balanced(m, Kk, N, bool(bits & 1), tile, bits, cb)


@pytest.mark.parametrize("m,Kk,N,tile", [(1280, 384, 16640, 256), (1024, 256, 16384, 256), (2048, 128, 16384, 256)])
def test_gemm_ranges_that_run_through_whole_tiles(m, Kk, N, tile):
    """More (tile, k-block) units per workgroup than a tile has k-blocks: a workgroup's range
    covers the end of one tile, whole tiles (finished without any hand-over) and the start of
    another; with exactly one tile per workgroup nothing is shared at all."""
    _check_balanced(m, Kk, N, False, tile)


def test_gemm_256_row_tiles_on_narrow_outputs():
    """BERTH_GEMM_ROWS256=2 (read once per process) takes 256-row tiles wherever they are
    possible: short last tiles (second row half with 72, 2 or no rows at all), a single tile
    row, 8320 and 4352 columns (half of the last column tile empty), 3 and 5 bpw."""
    import os
    import subprocess
    import sys
    code = (
        "import tests.test_gpu_linear as T\n"
        "for m, K, N, f, b in ((512, 1024, 4096, True, 4), (384, 640, 5632, False, 4), (200, 768, 8320, True, 4),\n"
        "                      (130, 256, 16384, False, 4), (300, 1024, 5632, True, 3), (640, 512, 4352, False, 5)):\n"
        "    T._check_balanced(m, K, N, f, 256, b)\n"
        "print('ok')\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=600, cwd=root,
                       env=dict(os.environ, BERTH_GEMM_ROWS256="2"))
    assert r.returncode == 0 and "ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_gemm_128_row_tiles_for_more_than_128_rows():
    """BERTH_GEMM_ROWS256=0 (read once per process) keeps 128-row tiles at any row count."""
    import os
    import subprocess
    import sys
    code = (
        "import tests.test_gpu_linear as T\n"
        "for m, K, N, f in ((512, 1024, 4096, True), (200, 768, 8320, False)):\n"
        "    T._check_balanced(m, K, N, f, 128)\n"
        "print('ok')\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=600, cwd=root,
                       env=dict(os.environ, BERTH_GEMM_ROWS256="0"))
    assert r.returncode == 0 and "ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_gemm_128_row_tiles_one_workgroup_per_tile_and_split():
    """The same tiles without the even deal (BERTH_GEMM_BALANCED=0, read once per process)."""
    import os
    import subprocess
    import sys
    code = (
        "import numpy as np, tests.test_gpu_linear as T\n"
        "for m, K, N in ((512, 1024, 4096), (200, 768, 8320)):\n"
        "    got, want, ah, want_ah, launch = T._run_linear(m, K, N, 4, 2, True, 700 + m, prefill=True)\n"
        "    assert 'exl3_gemm_kernel<4,2,128x256>' in launch, launch\n"
        "    assert np.array_equal(ah, want_ah) and T.close(got, want)[0] == 0, launch\n"
        "print('ok')\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=600, cwd=root,
                       env=dict(os.environ, BERTH_GEMM_BALANCED="0"))
    assert r.returncode == 0 and "ok" in r.stdout, r.stdout + r.stderr


def test_linear_through_decode_entry_with_many_rows():
    """forward_n passes rows 2..144 of a K = 6 linear to the m = 1 entry
    (crates/berth-engine/src/device.rs:338-352)."""
    got, want, ah, want_ah, launch = _run_linear(20, 256, 256, 6, 2, False, 123)
    assert "exl3_gemm_kernel" in launch
    assert np.array_equal(ah, want_ah)
    assert close(got, want)[0] == 0


def test_hgemm_matches_oracle():
    rng = np.random.default_rng(12)
    m, k, n = 70, 200, 136
    a = rng.normal(size=(m, k)).astype(np.float16)
    b = rng.normal(size=(k, n)).astype(np.float16)
    d_a, d_b = dev(a.view(np.uint16)), dev(b.view(np.uint16))
    for fp32 in (True, False):
        c = torch.zeros((m, n + 8), dtype=torch.float32 if fp32 else torch.float16, device=DEV)
        K.prefill_lin.hgemm(d_a.data_ptr(), d_b.data_ptr(), c.data_ptr(), m, k, n, n + 8,
                            OutDtype.F32 if fp32 else OutDtype.F16)
        torch.cuda.synchronize()
        want = O.hgemm(a, b, True)
        got = c.cpu().numpy()[:, :n] if fp32 else host_f16(c)[:, :n]
        assert np.allclose(got, want, rtol=2e-3, atol=2e-3)
        assert not c.cpu().numpy()[:, n:].any() if fp32 else True


def test_full_size_gemv_round_trip_property():
    """At the 27B gate shape the oracle is too slow to run in a test; check the
    size-independent property that the kernel is linear in the activation:
    y(x1 + x2) == y(x1) + y(x2) within tolerance, and y(0) == 0 exactly."""
    Kk, N = 5120, 17408
    tr, suh, svh = synth.linear(7, Kk, N, 4)
    d_tr, d_suh, d_svh = dev(tr), dev(suh.view(np.uint16)), dev(svh.view(np.uint16))
    a_had = torch.zeros(Kk, dtype=torch.float16, device=DEV)

    def run(xv):
        c = torch.zeros(N, dtype=torch.float32, device=DEV)
        dx = dev(xv.view(np.uint16))
        K.exl3_linear(dx.data_ptr(), d_tr.data_ptr(), c.data_ptr(), d_suh.data_ptr(), a_had.data_ptr(),
                      d_svh.data_ptr(), 1, Kk, N, 4, Codebook.MUL1, OutDtype.F32)
        torch.cuda.synchronize()
        return c.cpu().numpy()

    x1 = (synth.activations(1, 1, Kk) * np.float16(0.5)).astype(np.float16)
    x2 = (synth.activations(2, 1, Kk) * np.float16(0.5)).astype(np.float16)
    y0 = run(np.zeros((1, Kk), dtype=np.float16))
    assert not y0.any()
    y1, y2 = run(x1), run(x2)
    xs = (x1.astype(np.float32) + x2.astype(np.float32)).astype(np.float16)
    ys = run(xs)
    scale = np.abs(ys).max()
    assert np.abs(ys - (y1 + y2)).max() < 4e-3 * scale
    # spot-check 256 output columns against the oracle on the matching trellis slice
    sub = tr[:, 16:32, :]                       # columns 256..511
    want, _ = O.linear(x1, sub, suh, svh[256:512], Kk, 256, 4, 2, out_fp32=True)
    assert close(y1[256:512], want.reshape(-1))[0] == 0


def test_lm_head_shape_6bpw_slices_match_oracle():
    """The 27B lm_head (K 5120, N 248320, 6 bpw, mul1, fp16 logits: trellis
    [320, 15520, 96], crates/berth-exl3/tests/qwen38_27b.rs:66-76) at full size;
    three 256-column windows (first, middle, last) are checked against the oracle."""
    Kk, N, bits = 5120, 248320, 6
    tr, suh, svh = synth.linear(66, Kk, N, bits)
    assert tr.shape == (320, 15520, 96) and tr.nbytes == 953_548_800
    x = synth.activations(67, 1, Kk)
    d_tr, d_suh, d_svh, d_x = dev(tr), dev(suh.view(np.uint16)), dev(svh.view(np.uint16)), dev(x.view(np.uint16))
    a_had = torch.zeros(Kk, dtype=torch.float16, device=DEV)
    c = torch.zeros(N, dtype=torch.float16, device=DEV)
    K.exl3_linear(d_x.data_ptr(), d_tr.data_ptr(), c.data_ptr(), d_suh.data_ptr(), a_had.data_ptr(),
                  d_svh.data_ptr(), 1, Kk, N, bits, Codebook.MUL1, OutDtype.F16)
    torch.cuda.synchronize()
    assert "exl3_gemv_stream_kernel<6,2" in K.last_launch()      # a weight this large takes the streaming kernel
    got = host_f16(c)
    for c0 in (0, 124160, N - 256):
        sub = np.ascontiguousarray(tr[:, c0 // 16:c0 // 16 + 16, :])
        want, _ = O.linear(x, sub, suh, svh[c0:c0 + 256], Kk, 256, bits, 2, out_fp32=False)
        assert close(got[c0:c0 + 256], want.reshape(-1))[0] == 0, c0


@pytest.mark.parametrize("rows", [1, 3])
def test_very_wide_output_uses_closer_counters(rows):
    """More column blocks than the arrival-counter table holds at one counter per 128 bytes
    (K 256, N 128 x 5000, 2 bpw): the launch packs its counters closer together.  Windows at both
    ends and in the middle against the oracle, and the same call again gives the same bits (the
    counters were left at zero)."""
    Kk, N, bits = 256, 128 * 5000, 2
    tr, suh, svh = synth.linear(4242, Kk, N, bits)
    x = synth.activations(4243, rows, Kk)
    d_tr, d_suh, d_svh, d_x = dev(tr), dev(suh.view(np.uint16)), dev(svh.view(np.uint16)), dev(x.view(np.uint16))
    a_had = torch.zeros(rows * Kk, dtype=torch.float16, device=DEV)
    outs = []
    for _ in range(2):
        c = torch.zeros(rows * N, dtype=torch.float16, device=DEV)
        K.exl3_linear(d_x.data_ptr(), d_tr.data_ptr(), c.data_ptr(), d_suh.data_ptr(), a_had.data_ptr(),
                      d_svh.data_ptr(), rows, Kk, N, bits, Codebook.MUL1, OutDtype.F16)
        torch.cuda.synchronize()
        outs.append(host_f16(c).reshape(rows, N))
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))
    for c0 in (0, 128 * 2500, N - 256):
        sub = np.ascontiguousarray(tr[:, c0 // 16:c0 // 16 + 16, :])
        want, _ = O.linear(x, sub, suh, svh[c0:c0 + 256], Kk, 256, bits, 2, out_fp32=False)
        assert close(outs[0][:, c0:c0 + 256], want.reshape(rows, 256))[0] == 0, c0


@pytest.mark.parametrize("name,kernel", [("gate_proj", "exl3_gemm_wide_kernel<4,2,256x256>"),
                                         ("down_proj", "exl3_gemm_balanced_kernel<4,2,128x256>"),
                                         ("q_proj", "exl3_gemm_balanced_kernel<4,2,128x256>"),
                                         ("o_proj", "exl3_gemm_balanced_kernel<4,2,128x256>"),
                                         ("k_proj", "exl3_gemm_kernel<4,2,32x256>")])
def test_prefill_27b_shapes_at_512_rows_slices_match_oracle(name, kernel):
    """BASELINE configs[2] at full size (512 rows, 4 bpw, the 27B shapes): each of the four
    launch forms the dispatcher picks there, with 256-column windows (first, an odd middle
    one, last) of all 512 rows checked against the oracle on the matching trellis slice."""
    Kk, N = synth.SHAPES_27B[name]
    rows, bits = 512, 4
    tr, suh, svh = synth.linear(880 + len(name), Kk, N, bits)
    x = synth.activations(881, rows, Kk)
    d = {k: dev(v.view(np.uint16)) for k, v in dict(tr=tr, suh=suh, svh=svh, x=x).items()}
    c = torch.zeros((rows, N), dtype=torch.float16, device=DEV)
    a_had = torch.zeros((rows, Kk), dtype=torch.float16, device=DEV)
    w = torch.zeros(Kk * min(N, 32768), dtype=torch.float16, device=DEV)
    K.prefill_lin.exl3_linear(d["x"].data_ptr(), d["tr"].data_ptr(), c.data_ptr(), d["suh"].data_ptr(),
                              a_had.data_ptr(), d["svh"].data_ptr(), w.data_ptr(), rows, Kk, N, bits, Codebook.MUL1,
                              OutDtype.F16)
    torch.cuda.synchronize()
    assert kernel in K.prefill_lin.last_launch(), K.prefill_lin.last_launch()
    got = host_f16(c).reshape(rows, N)
    mid = (N // 512) * 256 + 256 if N > 1024 else 256
    for c0 in (0, mid, N - 256):
        sub = np.ascontiguousarray(tr[:, c0 // 16:c0 // 16 + 16, :])
        want, want_had = O.linear(x, sub, suh, svh[c0:c0 + 256], Kk, 256, bits, 2, out_fp32=False)
        bad, worst = close(got[:, c0:c0 + 256], want)
        assert bad == 0, (name, c0, bad, worst)
    assert np.array_equal(host_u16(a_had).reshape(rows, Kk), want_had.view(np.uint16))


# ---- multi-linear (exl3_mgemm)
@pytest.mark.parametrize("rows,fp32", [(1, False), (1, True), (3, False)])
def test_mgemm_sliced_qkv_bundle(rows, fp32):
    from berth_amd.device import Exl3Linear, Exl3MultiLinear, Gpu
    gpu = Gpu(0)
    Kk, Ns = 512, (768, 256, 256)
    lins_np = [synth.linear(700 + i, Kk, n, 4) for i, n in enumerate(Ns)]
    lins = [Exl3Linear(gpu, f"l{i}", *l) for i, l in enumerate(lins_np)]
    multi = Exl3MultiLinear(gpu, lins)
    assert multi.width == 256 and multi.slices == 5
    x = synth.activations(710, rows, Kk)
    d_x = dev(x.view(np.uint16))
    outs = [torch.zeros((rows, n), dtype=torch.float32 if fp32 else torch.float16, device=DEV) for n in Ns]
    multi.forward(gpu, d_x, outs, OutDtype.F32 if fp32 else OutDtype.F16, rows)
    torch.cuda.synchronize()
    assert "sliced x5" in K.ops.last_launch()
    for i, (tr, suh, svh) in enumerate(lins_np):
        want, want_had = O.linear(x, tr, suh, svh, Kk, Ns[i], 4, 2, out_fp32=fp32)
        got = outs[i].cpu().numpy() if fp32 else host_f16(outs[i])
        assert close(got, want)[0] == 0, i
        slab = host_u16(multi.a_had)[i * rows * Kk:(i + 1) * rows * Kk]
        assert np.array_equal(slab, want_had.view(np.uint16).reshape(-1))


def test_mgemm_uniform_mode():
    Kk, N, n_mat = 256, 256, 3
    lins = [synth.linear(800 + i, Kk, N, 4) for i in range(n_mat)]
    x = synth.activations(810, n_mat, Kk)            # one row per matrix
    d = [[dev(t.view(np.uint16)) for t in lin] for lin in lins]
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=DEV)
    b_list, suh_list, svh_list = (i64([dd[j].data_ptr() for dd in d]) for j in range(3))
    d_x = dev(x.view(np.uint16))
    for bszm_in in (n_mat, 1):
        c = torch.zeros((n_mat, 1, N), dtype=torch.float32, device=DEV)
        a_had = torch.zeros((n_mat, Kk), dtype=torch.float16, device=DEV)
        rc = K.ops.exl3_mgemm(d_x.data_ptr(), b_list.data_ptr(), c.data_ptr(), suh_list.data_ptr(), a_had.data_ptr(),
                              svh_list.data_ptr(), 1, Kk, N, 4, Codebook.MUL1, OutDtype.F32, bszm_in, n_mat)
        torch.cuda.synchronize()
        assert rc > 0
        for i, (tr, suh, svh) in enumerate(lins):
            xi = x[i:i + 1] if bszm_in > 1 else x[0:1]
            want, _ = O.linear(xi, tr, suh, svh, Kk, N, 4, 2, out_fp32=True)
            assert close(c[i].cpu().numpy(), want)[0] == 0


def test_unpack_signs_known_answers():
    """The five known-answer cases of crates/berth-exl3/src/signs.rs:48-92 and a
    random tensor against the oracle, on the device."""
    ONE, NEG = 0x3C00, 0xBC00

    def run(words):
        raw = np.asarray(words, dtype="<u2").view(np.uint8)
        d_in = torch.from_numpy(raw.copy()).to(DEV)
        d_out = torch.zeros(raw.size * 8, dtype=torch.int16, device=DEV)
        K.unpack_signs(d_in.data_ptr(), d_out.data_ptr(), raw.size)
        torch.cuda.synchronize()
        return d_out.cpu().numpy().view(np.uint16)

    s = run([1])
    assert len(s) == 16 and s[0] == NEG and (s[1:] == ONE).all()
    s = run([0x8000])
    assert (s[:15] == ONE).all() and s[15] == NEG
    assert (run([0]) == ONE).all() and (run([0xFFFF]) == NEG).all()
    s = run([5, 1])
    assert len(s) == 32 and (s[0], s[1], s[2], s[16], s[17]) == (NEG, ONE, NEG, NEG, ONE)
    words = np.random.default_rng(8).integers(0, 65536, size=1088, dtype=np.uint16)
    assert np.array_equal(run(words), np.asarray(O.unpack_signs(words.astype("<u2").tobytes()), dtype=np.uint16))


def test_linear_from_packed_signs():
    """A linear whose su / sv are packed sign words gives the same output as the
    one built from the expanded fp16 signs."""
    gpu = Gpu(0)
    Kk, N, bits = 256, 384, 4
    tr = synth.trellis_words(70, Kk, N, bits)
    rng = np.random.default_rng(71)
    su = rng.integers(0, 65536, size=Kk // 16, dtype=np.uint16)
    sv = rng.integers(0, 65536, size=N // 16, dtype=np.uint16)
    suh = np.asarray(O.unpack_signs(su.astype("<u2").tobytes()), dtype=np.uint16).view(np.float16)
    svh = np.asarray(O.unpack_signs(sv.astype("<u2").tobytes()), dtype=np.uint16).view(np.float16)
    x = synth.activations(72, 1, Kk)
    lin = Exl3Linear.from_packed_signs(gpu, "packed", tr, su, sv)
    c = torch.zeros(N, dtype=torch.float32, device=DEV)
    lin.forward(gpu, dev(x.view(np.uint16)), c, OutDtype.F32)
    torch.cuda.synchronize()
    want, _ = O.linear(x, tr, suh, svh, Kk, N, bits, 2, out_fp32=True)
    assert close(c.cpu().numpy(), want.ravel())[0] == 0


def _window_check(name, Kk, N, bits, out_fp32, seed):
    """One row through berth_exl3_linear at a 27B shape; three 256-column windows (first,
    middle, last) against the oracle on the matching trellis slices, a_had bit-exact."""
    tr, suh, svh = synth.linear(seed, Kk, N, bits)
    x = synth.activations(seed + 1, 1, Kk)
    d_tr, d_suh, d_svh, d_x = dev(tr), dev(suh.view(np.uint16)), dev(svh.view(np.uint16)), dev(x.view(np.uint16))
    a_had = torch.zeros(Kk, dtype=torch.float16, device=DEV)
    c = torch.zeros(N, dtype=torch.float32 if out_fp32 else torch.float16, device=DEV)
    K.exl3_linear(d_x.data_ptr(), d_tr.data_ptr(), c.data_ptr(), d_suh.data_ptr(), a_had.data_ptr(),
                  d_svh.data_ptr(), 1, Kk, N, bits, Codebook.MUL1, OutDtype.F32 if out_fp32 else OutDtype.F16)
    launch = K.last_launch()
    torch.cuda.synchronize()
    got = c.cpu().numpy() if out_fp32 else host_f16(c)
    want_had = None
    for c0 in (0, (N // 512) * 256, N - 256):
        sub = np.ascontiguousarray(tr[:, c0 // 16:c0 // 16 + 16, :])
        want, want_had = O.linear(x, sub, suh, svh[c0:c0 + 256], Kk, 256, bits, 2, out_fp32=out_fp32)
        bad, worst = close(got[c0:c0 + 256], want.reshape(-1))
        assert bad == 0, (name, bits, c0, bad, worst, launch)
    assert np.array_equal(host_u16(a_had), want_had.view(np.uint16).reshape(-1)), (name, launch)


@pytest.mark.parametrize("name", ["q_proj", "o_proj", "down_proj"])
def test_27b_shapes_batch1_4bpw_windows_match_oracle(name):
    """BASELINE configs[1] at 4 bpw, the shapes the other full-size tests leave out."""
    Kk, N = synth.SHAPES_27B[name]
    _window_check(name, Kk, N, 4, name != "q_proj", 7100 + Kk % 97)


@pytest.mark.parametrize("bits", [2, 3, 5])
@pytest.mark.parametrize("name", ["gate_proj", "down_proj", "q_proj", "o_proj", "k_proj"])
def test_27b_shapes_batch1_other_rates_windows_match_oracle(name, bits):
    """BASELINE configs[1] at 2, 3 and 5 bpw on every shape of the set (v_proj has k_proj's)."""
    Kk, N = synth.SHAPES_27B[name]
    _window_check(name, Kk, N, bits, name in ("down_proj", "o_proj"), 7200 + 10 * bits + Kk % 97 + len(name))
