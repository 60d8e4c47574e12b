"""GPU parity of the one-row streaming GEMV kernel (one resident workgroup of sixteen waves
per compute unit, static split of the tile rows, hybrid table / arithmetic decode) against
the CPU oracle, through the C ABI.

The library takes this kernel by itself for large weights only; here the knobs that are
read at every call (BERTH_GEMV_STREAM_*) force it onto small shapes with few workgroups, so
that every way a workgroup's units can lie is covered at sizes the oracle finishes in
seconds: one column block, the end of one and the start of the next (two activation
regions), several whole column blocks, column blocks shared by two and by many workgroups.

Bars: rotated activation (a_had) bit-exact; outputs within rtol 2e-3 / atol 1e-3 of the
oracle's fp32 matmul over the oracle-decoded weights."""
import contextlib
import os

import numpy as np
import pytest
import torch

from berth_amd import kernels as K
from berth_amd import synth
from berth_amd.kernels import Codebook, OutDtype
from oracle import oracle as O
from tests.gpu_util import DEV, close, dev, host_f16, host_u16, knobs

pytestmark = pytest.mark.gpu


def forced(wgs=0, lut="0xA", min_units=2):
    return knobs(BERTH_GEMV_STREAM=1, BERTH_GEMV_STREAM_SHRINK=1, BERTH_GEMV_STREAM_MIN_UNITS=min_units,
                 BERTH_GEMV_STREAM_WGS=wgs, BERTH_GEMV_STREAM_LUT=lut)


def run_linear(Kk, N, bits, cb, out_fp32, seed):
    tr, suh, svh = synth.linear(seed, Kk, N, bits)
    x = synth.activations(seed + 7, 1, Kk)
    d = {k: dev(v.view(np.uint16)) for k, v in dict(tr=tr, suh=suh, svh=svh, x=x).items()}
    c = torch.zeros((1, N), dtype=torch.float32 if out_fp32 else torch.float16, device=DEV)
    a_had = torch.zeros((1, Kk), dtype=torch.float16, device=DEV)
    K.exl3_linear(d["x"].data_ptr(), d["tr"].data_ptr(), c.data_ptr(), d["suh"].data_ptr(), a_had.data_ptr(),
                  d["svh"].data_ptr(), 1, Kk, N, bits, Codebook(cb), OutDtype.F32 if out_fp32 else OutDtype.F16)
    launch = K.last_launch()
    torch.cuda.synchronize()
    want, want_had = O.linear(x, tr, suh, svh, Kk, N, bits, cb, out_fp32=out_fp32)
    got = c.cpu().numpy() if out_fp32 else host_f16(c)
    return got, want, host_u16(a_had), want_had.view(np.uint16), launch


def check(Kk, N, bits, cb, out_fp32, seed):
    got, want, ah, want_ah, launch = run_linear(Kk, N, bits, cb, out_fp32, seed)
    assert "exl3_gemv_stream_kernel" in launch, launch
    assert np.array_equal(ah, want_ah), launch
    bad, worst = close(got, want)
    assert bad == 0, (bad, worst, launch)
    return launch


# (K, N, workgroup cap): how the units of a workgroup lie
LAYOUTS = [
    (1024, 256, 0),      # 2 column blocks x 64 tile rows, 4 workgroups: each inside one column block
    (1024, 384, 4),      # 3 x 64 over 4 workgroups: end of one column block + start of the next
    (512, 1024, 2),      # 8 x 32 over 2 workgroups: four whole column blocks each
    (512, 1280, 3),      # 10 x 32 over 3: whole column blocks and a shared one in the middle
    (2048, 128, 0),      # one column block shared by every workgroup
    (4096, 256, 5),      # K 4096: two regions of the rotated activation in the straddling workgroup
    (256, 1536, 1),      # a single workgroup, twelve column blocks
    (640, 640, 7),       # odd everything
]


@pytest.mark.parametrize("Kk,N,wgs", LAYOUTS)
@pytest.mark.parametrize("lut", ["0", "0xA"])
def test_stream_layouts_4bpw(Kk, N, wgs, lut):
    with forced(wgs=wgs, lut=lut):
        launch = check(Kk, N, 4, 2, True, 3000 + Kk + N)
    assert f"table={lut.lower()}" in launch.lower(), launch


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("cb", [0, 1, 2])
@pytest.mark.parametrize("lut", ["0", "0xA"])
def test_stream_every_rate_and_codebook(bits, cb, lut):
    with forced(wgs=3, lut=lut):
        check(1024, 384, bits, cb, bits % 2 == 0, 4000 + 10 * bits + cb)


def test_stream_large_k_two_regions():
    """K = 17408 (136 k-blocks, more than a workgroup's LDS region holds): the kernel applies
    only while every workgroup's units need at most 64 k-blocks."""
    with forced(wgs=0, lut="0xA", min_units=4):
        launch = check(17408, 256, 4, 2, True, 5001)
    assert "grid=" in launch


def test_stream_is_deterministic_and_counters_reset():
    outs = []
    with forced(wgs=5):
        for _ in range(3):
            got, _, _, _, launch = run_linear(2048, 256, 4, 2, True, 99)
            outs.append(got.view(np.uint32).copy())
    assert "exl3_gemv_stream_kernel" in launch
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


def test_stream_agrees_with_the_many_workgroup_kernel():
    """Same operator, two kernels with different summation orders: both within the bar of the
    oracle and within twice the bar of each other."""
    with forced(wgs=6):
        a, want, _, _, la = run_linear(3072, 512, 4, 2, True, 123)
    with knobs(BERTH_GEMV_STREAM=0):
        b, _, _, _, lb = run_linear(3072, 512, 4, 2, True, 123)
    assert "stream" in la and "stream" not in lb
    assert close(a, want)[0] == 0 and close(b, want)[0] == 0
    assert close(a, b, rtol=4e-3, atol=2e-3)[0] == 0


@pytest.mark.parametrize("lut", ["0", "0xA"])
def test_stream_mlp_block_pair_and_silu_input(lut):
    """berth_exl3_mlp at one row: gate and up as a pair launch on one rotated input, the down
    projection with the SiLU gate evaluated while its input is rotated."""
    from tests.test_gpu_mlp import run_mlp_block
    with forced(wgs=4, lut=lut):
        launch = run_mlp_block(1, 512, 1024, 4)
    assert launch.count("exl3_gemv_stream_kernel") == 2 and "pair" in launch and "silu" in launch, launch


@pytest.mark.parametrize("fp32", [False, True])
def test_stream_mgemm_sliced_bundle(fp32):
    from berth_amd.device import Exl3Linear, Exl3MultiLinear, Gpu
    gpu = Gpu(0)
    Kk, Ns = 1024, (768, 256, 256)
    lins_np = [synth.linear(700 + i, Kk, n, 4) for i, n in enumerate(Ns)]
    lins = [Exl3Linear(gpu, f"l{i}", *l) for i, l in enumerate(lins_np)]
    multi = Exl3MultiLinear(gpu, lins)
    x = synth.activations(710, 1, Kk)
    d_x = dev(x.view(np.uint16))
    outs = [torch.zeros((1, n), dtype=torch.float32 if fp32 else torch.float16, device=DEV) for n in Ns]
    with forced(wgs=2):
        multi.forward(gpu, d_x, outs, OutDtype.F32 if fp32 else OutDtype.F16, 1)
        launch = K.ops.last_launch()
    torch.cuda.synchronize()
    assert "sliced x5" in launch and "exl3_gemv_stream_kernel" in launch, launch
    for i, (tr, suh, svh) in enumerate(lins_np):
        want, want_had = O.linear(x, tr, suh, svh, Kk, Ns[i], 4, 2, out_fp32=fp32)
        got = outs[i].cpu().numpy() if fp32 else host_f16(outs[i])
        assert close(got, want)[0] == 0, i
        slab = host_u16(multi.a_had)[i * Kk:(i + 1) * Kk]
        assert np.array_equal(slab, want_had.view(np.uint16).reshape(-1))


def test_stream_mgemm_sliced_with_a_narrow_slice():
    """Slices narrower than the bundle's width end early: their units stop at their last column
    block and the waves behind it idle."""
    Kk, width = 1024, 384
    widths = (384, 128, 256)
    lins = [synth.linear(900 + i, Kk, n, 4) for i, n in enumerate(widths)]
    x = synth.activations(910, 1, Kk)
    d = [[dev(t.view(np.uint16)) for t in lin] for lin in lins]
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    outs = [torch.zeros((1, n), dtype=torch.float32, device=DEV) for n in widths]
    a_had = torch.zeros((3, Kk), dtype=torch.float16, device=DEV)
    b_list, svh_list = i64([dd[0].data_ptr() for dd in d]), i64([dd[2].data_ptr() for dd in d])
    suh_list = i64([dd[1].data_ptr() for dd in d])
    c_ptrs = i64([o.data_ptr() for o in outs])
    d_x, size_n, n_stride, had_src = dev(x.view(np.uint16)), i32(list(widths)), i32(list(widths)), i32([0, 1, 2])
    with forced(wgs=2):
        rc = K.ops.exl3_mgemm(d_x.data_ptr(), b_list.data_ptr(), outs[0].data_ptr(),
                              suh_list.data_ptr(), a_had.data_ptr(), svh_list.data_ptr(), 1, Kk, width, 4,
                              Codebook.MUL1, OutDtype.F32, 1, 3, size_n.data_ptr(), c_ptrs.data_ptr(),
                              n_stride.data_ptr(), had_src.data_ptr(), 3)
        launch = K.ops.last_launch()
    torch.cuda.synchronize()
    assert rc > 0 and "exl3_gemv_stream_kernel" in launch, launch
    for i, (tr, suh, svh) in enumerate(lins):
        want, want_had = O.linear(x, tr, suh, svh, Kk, widths[i], 4, 2, out_fp32=True)
        assert close(outs[i].cpu().numpy(), want)[0] == 0, i
        assert np.array_equal(host_u16(a_had).reshape(-1)[i * Kk:(i + 1) * Kk], want_had.view(np.uint16).reshape(-1))


def test_stream_mgemm_uniform_mode():
    Kk, N, n_mat = 1024, 256, 3
    lins = [synth.linear(800 + i, Kk, N, 4) for i in range(n_mat)]
    x = synth.activations(810, n_mat, Kk)
    d = [[dev(t.view(np.uint16)) for t in lin] for lin in lins]
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device=DEV)
    b_list, suh_list, svh_list = (i64([dd[j].data_ptr() for dd in d]) for j in range(3))
    d_x = dev(x.view(np.uint16))
    for bszm_in in (n_mat, 1):
        c = torch.zeros((n_mat, 1, N), dtype=torch.float32, device=DEV)
        a_had = torch.zeros((n_mat, Kk), dtype=torch.float16, device=DEV)
        with forced(wgs=2):
            rc = K.ops.exl3_mgemm(d_x.data_ptr(), b_list.data_ptr(), c.data_ptr(), suh_list.data_ptr(),
                                  a_had.data_ptr(), svh_list.data_ptr(), 1, Kk, N, 4, Codebook.MUL1, OutDtype.F32,
                                  bszm_in, n_mat)
            launch = K.ops.last_launch()
        torch.cuda.synchronize()
        assert rc > 0 and "exl3_gemv_stream_kernel" in launch, launch
        for i, (tr, suh, svh) in enumerate(lins):
            xi = x[i:i + 1] if bszm_in > 1 else x[0:1]
            want, want_had = O.linear(xi, tr, suh, svh, Kk, N, 4, 2, out_fp32=True)
            assert close(c[i].cpu().numpy(), want)[0] == 0, (bszm_in, i)
            assert np.array_equal(host_u16(a_had).reshape(-1)[i * Kk:(i + 1) * Kk], want_had.view(np.uint16).reshape(-1))


def test_state_tables_hold_every_decoded_state():
    """The table the hybrid decode reads is the dequantisation of every state: an 8 bpw trellis
    whose tiles hold arbitrary byte pairs exercises a wide range of states through both paths."""
    Kk, N = 1024, 256
    for cb in (0, 1, 2):
        with forced(wgs=2, lut="0xA"):
            check(Kk, N, 8, cb, True, 6000 + cb)


def test_mgemm_host_lists_give_the_bits_of_device_lists():
    """berth_ops_mgemm_hostlists (the problems by value in the kernel arguments) against
    berth_ops_mgemm (device lists) on one sliced bundle with a narrow slice and on a uniform
    bundle with one shared and with per-problem inputs: outputs and rotated inputs bit for bit."""
    Kk = 1024
    widths = (384, 128, 256)
    lins = [synth.linear(930 + i, Kk, n, 4) for i, n in enumerate(widths)]
    d = [[dev(t.view(np.uint16)) for t in lin] for lin in lins]
    x = synth.activations(940, 3, Kk)
    d_x = dev(x.view(np.uint16))
    host = dict(b=np.array([dd[0].data_ptr() for dd in d], dtype=np.uint64),
                suh=np.array([dd[1].data_ptr() for dd in d], dtype=np.uint64),
                svh=np.array([dd[2].data_ptr() for dd in d], dtype=np.uint64),
                size_n=np.array(widths, dtype=np.int32), stride=np.array(widths, dtype=np.int32),
                src=np.array([0, 1, 2], dtype=np.int32))
    devl = {k: torch.from_numpy(v.view(np.int64) if v.dtype == np.uint64 else v).to(DEV) for k, v in host.items()}

    def sliced(fn, lists, addr):
        outs = [torch.zeros((1, n), dtype=torch.float32, device=DEV) for n in widths]
        a_had = torch.zeros((3, Kk), dtype=torch.float16, device=DEV)
        c_host = np.array([o.data_ptr() for o in outs], dtype=np.uint64)
        c_list = c_host if lists is host else torch.from_numpy(c_host.view(np.int64)).to(DEV)
        with forced(wgs=2, lut="0"):
            fn(d_x.data_ptr(), addr(lists["b"]), outs[0].data_ptr(), addr(lists["suh"]), a_had.data_ptr(),
               addr(lists["svh"]), 1, Kk, 384, 4, Codebook.MUL1, OutDtype.F32, 1, 3, addr(lists["size_n"]), addr(c_list),
               addr(lists["stride"]), addr(lists["src"]), 3)
            launch = K.ops.last_launch()
        torch.cuda.synchronize()
        return [o.cpu().numpy().view(np.uint32) for o in outs], host_u16(a_had), launch

    ref, ref_had, ref_launch = sliced(K.ops.exl3_mgemm, devl, lambda t: t.data_ptr())
    got, got_had, got_launch = sliced(K.ops.exl3_mgemm_hostlists, host, lambda a: a.ctypes.data)
    assert "by value" in got_launch and "by value" not in ref_launch and "exl3_gemv_stream_kernel" in ref_launch
    assert all(np.array_equal(a, b) for a, b in zip(got, ref)) and np.array_equal(got_had, ref_had)

    # uniform: three linears of one shape
    N = 256
    ulins = [synth.linear(950 + i, Kk, N, 4) for i in range(3)]
    ud = [[dev(t.view(np.uint16)) for t in lin] for lin in ulins]
    uh = [np.array([dd[j].data_ptr() for dd in ud], dtype=np.uint64) for j in range(3)]
    udv = [torch.from_numpy(a.view(np.int64)).to(DEV) for a in uh]
    for bszm_in in (3, 1):
        res = []
        for fn, lists, addr in ((K.ops.exl3_mgemm, udv, lambda t: t.data_ptr()),
                                (K.ops.exl3_mgemm_hostlists, uh, lambda a: a.ctypes.data)):
            c = torch.zeros((3, 1, N), dtype=torch.float16, device=DEV)
            a_had = torch.zeros((3, Kk), dtype=torch.float16, device=DEV)
            with forced(wgs=2, lut="0"):
                fn(d_x.data_ptr(), addr(lists[0]), c.data_ptr(), addr(lists[1]), a_had.data_ptr(), addr(lists[2]), 1, Kk, N,
                   4, Codebook.MUL1, OutDtype.F16, bszm_in, 3)
            torch.cuda.synchronize()
            res.append((host_u16(c), host_u16(a_had)))
        assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1]), bszm_in


def test_mgemm_host_lists_refuse_what_the_streaming_kernel_does_not_serve():
    bad = 0xdead000
    one = np.array([bad], dtype=np.uint64)
    with pytest.raises(K.LaunchError, match="host lists"):      # three rows
        K.ops.exl3_mgemm_hostlists(bad, one.ctypes.data, bad, one.ctypes.data, bad, one.ctypes.data, 3, 1024, 256, 4,
                                   Codebook.MUL1, OutDtype.F16, 1, 1)
    with pytest.raises(K.LaunchError, match="host lists"):      # a weight too small for the streaming kernel
        K.ops.exl3_mgemm_hostlists(bad, one.ctypes.data, bad, one.ctypes.data, bad, one.ctypes.data, 1, 128, 128, 4,
                                   Codebook.MUL1, OutDtype.F16, 1, 1)
    many = np.full(17, bad, dtype=np.uint64)
    with pytest.raises(K.LaunchError, match="host lists"):      # seventeen problems
        K.ops.exl3_mgemm_hostlists(bad, many.ctypes.data, bad, many.ctypes.data, bad, many.ctypes.data, 1, 5120, 17408, 4,
                                   Codebook.MUL1, OutDtype.F16, 1, 17)
    assert K.ops.last_launch() == ""


def test_stale_accumulator_is_reported_and_cleared():
    """Forced from the host: an accumulator word of the streaming kernel is given a contribution
    count no launch leaves behind.  The launch that meets it leaves that column block unwritten
    and raises the device's fault word; the next launch reports it (and launches nothing), the
    query reads clean afterwards, and the launch after that is back to normal.  Every kernel
    exits by itself."""
    import ctypes as C
    from tests.test_gpu_runtime import Runtime
    Kk, N, bits = 4096, 8192, 4
    tr, suh, svh = synth.linear(960, Kk, N, bits)
    x = synth.activations(961, 1, Kk)
    d = {k: dev(v.view(np.uint16)) for k, v in dict(tr=tr, suh=suh, svh=svh, x=x).items()}
    a_had = torch.zeros(Kk, dtype=torch.float16, device=DEV)

    def launch(c):
        K.exl3_linear(d["x"].data_ptr(), d["tr"].data_ptr(), c.data_ptr(), d["suh"].data_ptr(), a_had.data_ptr(),
                      d["svh"].data_ptr(), 1, Kk, N, bits, Codebook.MUL1, OutDtype.F32)
        text = K.last_launch()
        torch.cuda.synchronize()
        return text

    good = torch.zeros(N, dtype=torch.float32, device=DEV)
    assert "exl3_gemv_stream_kernel" in launch(good)
    accum, slots = C.c_void_p(), C.c_int()
    assert K.load().berth_kernels_accumulators(C.byref(accum), C.byref(slots)) == 0 and slots.value >= N // 128
    rt = Runtime()
    block = 5
    stale = np.array([200], dtype=np.uint64)                       # 200 contributions already "there"
    rt.ok(rt.copy_from_host(None, accum.value + block * 1024, stale.ctypes.data, 8))
    assert K.pending_fault(0) == 0
    c = torch.full((N,), 555.0, dtype=torch.float32, device=DEV)
    launch(c)                                                       # accepted; every kernel exits
    got = c.cpu().numpy()
    assert (got[block * 128:(block + 1) * 128] == 555.0).all()      # nobody could finish the block: left unwritten
    keep = np.ones(N, dtype=bool)
    keep[block * 128:(block + 1) * 128] = False
    assert np.array_equal(got[keep].view(np.uint32), good.cpu().numpy()[keep].view(np.uint32))
    with pytest.raises(K.LaunchError, match=f"accumulator of column block {block} inconsistent"):
        launch(c)
    assert K.last_launch() == "" and K.pending_fault(0) == 0       # reported once, accumulators cleared
    launch(c)
    assert np.array_equal(c.cpu().numpy().view(np.uint32), good.cpu().numpy().view(np.uint32))
    # the query alone also reads and clears a report
    rt.ok(rt.copy_from_host(None, accum.value + block * 1024, stale.ctypes.data, 8))
    launch(c)
    assert K.pending_fault(0) == 0x40000001 + block and K.pending_fault(0) == 0
    zero = np.zeros(128, dtype=np.uint64)
    rt.ok(rt.copy_from_host(None, accum.value + block * 1024, zero.ctypes.data, 1024))
    launch(c)
    assert np.array_equal(c.cpu().numpy().view(np.uint32), good.cpu().numpy().view(np.uint32))
    rt.context_free(rt.ctx)
