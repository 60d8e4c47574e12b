"""GPU parity of the glue ops around the MLP (RMS norm, fused-residual RMS norm,
fp32 add) through the C ABI: bit-exact against the CPU oracle and against the
reference's fixtures (tests/golden/norm*.bin, add.*.bin)."""
import numpy as np
import pytest
import torch

from berth_amd import kernels as K
from oracle import oracle as O
from tests.gpu_util import DEV, dev, host_u16
from tests.test_oracle_glue import EPS, load, recover_weight, to_bf16_bits

pytestmark = pytest.mark.gpu


def _dev32(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(DEV)


def _dev16(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(DEV)


def _rms(x, wbits, eps, bias, scale, bf16, residual=None):
    rows, dim = x.shape
    d_x, d_w = _dev32(x), _dev16(wbits)
    y = torch.zeros((rows, dim), dtype=torch.float16, device=DEV)
    if residual is None:
        K.ops.rms_norm(d_x.data_ptr(), d_w.data_ptr(), y.data_ptr(), rows, dim, eps, bias, scale, bf16)
        torch.cuda.synchronize()
        return y.cpu().numpy(), None
    d_r = _dev32(residual)
    K.ops.rms_norm_res_in(d_x.data_ptr(), d_w.data_ptr(), y.data_ptr(), d_r.data_ptr(), rows, dim, eps, bias, scale, bf16)
    torch.cuda.synchronize()
    return y.cpu().numpy(), d_r.cpu().numpy()


@pytest.mark.parametrize("yfile", ["norm_input.y.bin", "norm_final.y.bin"])
def test_rms_norm_fixture(yfile):
    x, y = load("norm.x.bin", np.float32), load(yfile, np.float16)
    got, _ = _rms(x.reshape(1, -1), recover_weight(x, y), EPS, 1.0, 1.0, True)
    assert np.array_equal(got.view(np.uint16).ravel(), y.view(np.uint16))
    assert "rms_norm_kernel<0,float,half,bfloat16,float>" in K.ops.last_launch()


def test_rms_norm_res_in_fixture():
    x, r = load("norm_res.x.bin", np.float32), load("norm_res.r.bin", np.float32)
    r_out, y = load("norm_res.r_out.bin", np.float32), load("norm_res.y.bin", np.float16)
    got, res = _rms(x.reshape(1, -1), recover_weight(r_out, y), EPS, 1.0, 1.0, True, residual=r.reshape(1, -1))
    assert np.array_equal(res.view(np.uint32).ravel(), r_out.view(np.uint32))
    assert np.array_equal(got.view(np.uint16).ravel(), y.view(np.uint16))


@pytest.mark.parametrize("rows,dim,bf16", [(1, 5120, True), (7, 2048, True), (3, 132, False), (64, 4096, False)])
def test_rms_norm_matches_oracle(rows, dim, bf16):
    rng = np.random.default_rng(rows * 1000 + dim)
    x = rng.normal(0, 2.5, size=(rows, dim)).astype(np.float32)
    r = rng.normal(0, 1.0, size=(rows, dim)).astype(np.float32)
    wf = rng.normal(0, 0.4, size=dim).astype(np.float32)
    bits = to_bf16_bits(wf) if bf16 else wf.astype(np.float16).view(np.uint16)
    got, _ = _rms(x, bits, 1e-6, 1.0, 1.0, bf16)
    want = O.rms_norm(x, bits, 1e-6, 1.0, 1.0, weight_bf16=bf16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    got, res = _rms(x, bits, 1e-5, 0.0, 0.5, bf16, residual=r)
    want, wres = O.rms_norm(x, bits, 1e-5, 0.0, 0.5, weight_bf16=bf16, residual=r)
    assert np.array_equal(res.view(np.uint32), wres.view(np.uint32))
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_add_f32_fixture_and_alias():
    a, b, c = load("add.a.bin", np.float32), load("add.b.bin", np.float32), load("add.c.bin", np.float32)
    d_a, d_b = _dev32(a), _dev32(b)
    d_c = torch.zeros_like(d_a)
    K.ops.add_f32(d_a.data_ptr(), d_b.data_ptr(), d_c.data_ptr(), a.size)
    torch.cuda.synchronize()
    assert np.array_equal(d_c.cpu().numpy().view(np.uint32), c.view(np.uint32))
    assert K.ops.last_launch() == "add_f32 block=256 grid=20"
    K.ops.add_f32(d_a.data_ptr(), d_b.data_ptr(), d_a.data_ptr(), a.size)      # c may alias a
    torch.cuda.synchronize()
    assert np.array_equal(d_a.cpu().numpy().view(np.uint32), c.view(np.uint32))


def test_rms_norm_f16_matches_the_fp32_input_norm_on_widened_rows():
    """berth_ops_rms_norm_f16 (fp16 rows, bf16 weight, no residual): the fp16 input widens
    exactly, so the result is bit for bit that of the oracle's norm on the widened rows.  The
    reference holds no fixture for this variant (parity unpinned beyond that identity)."""
    rng = np.random.default_rng(5)
    rows, dim = 3, 5120
    x = (rng.normal(size=(rows, dim)) * 3).astype(np.float16)
    w = (rng.normal(size=dim) * 0.3).astype(np.float32)
    w_bf16 = (w.view(np.uint32) >> 16).astype(np.uint16)
    d_x, d_w = dev(x.view(np.uint16)), dev(w_bf16)
    y = torch.zeros((rows, dim), dtype=torch.float16, device=DEV)
    K.ops.rms_norm_f16(d_x.data_ptr(), d_w.data_ptr(), y.data_ptr(), rows, dim, 1e-6)
    torch.cuda.synchronize()
    assert "rms_norm_kernel<0,half,half,bfloat16,half>" in K.ops.last_launch()
    want = O.rms_norm(x.astype(np.float32), w_bf16, 1e-6, 1.0, 1.0, weight_bf16=True)
    assert np.array_equal(host_u16(y).reshape(rows, dim), want.view(np.uint16).reshape(rows, dim))


def test_embed_copy_and_concat_are_exact():
    """berth_ops_embed_tokens / _f16, berth_ops_memcpy_d2d, berth_ops_cat_f16_last: gathers and
    copies, checked against numpy (bf16 -> fp32 is an exact widen; bf16 -> fp16 one rounding)."""
    rng = np.random.default_rng(6)
    vocab, hidden = 97, 256
    w32 = (rng.normal(size=(vocab, hidden)) * 2).astype(np.float32)
    w_bf16 = (w32.view(np.uint32) >> 16).astype(np.uint16)
    exact = (w_bf16.astype(np.uint32) << 16).view(np.float32)
    ids = np.array([0, 1, 42, 96, 7, 7], dtype=np.int32)
    d_w, d_ids = dev(w_bf16), torch.from_numpy(ids).to(DEV)
    out32 = torch.zeros((ids.size, hidden), dtype=torch.float32, device=DEV)
    out16 = torch.zeros((ids.size, hidden), dtype=torch.float16, device=DEV)
    K.ops.embed_tokens(d_w.data_ptr(), d_ids.data_ptr(), out32.data_ptr(), hidden, ids.size)
    assert "embed_bf16_f32" in K.ops.last_launch()
    K.ops.embed_tokens(d_w.data_ptr(), d_ids.data_ptr(), out16.data_ptr(), hidden, ids.size, f16=True)
    assert "embed_bf16_f16" in K.ops.last_launch()
    torch.cuda.synchronize()
    assert np.array_equal(out32.cpu().numpy().view(np.uint32), exact[ids].view(np.uint32))
    assert np.array_equal(host_u16(out16), exact[ids].astype(np.float16).view(np.uint16))
    cat = torch.zeros((ids.size, 2 * hidden), dtype=torch.float16, device=DEV)
    other = dev(rng.integers(0, 65536, size=(ids.size, hidden), dtype=np.uint16))
    K.ops.cat_f16_last(out16.data_ptr(), other.data_ptr(), cat.data_ptr(), ids.size, hidden)
    copy = torch.zeros_like(cat)
    K.ops.memcpy_d2d(copy.data_ptr(), cat.data_ptr(), cat.numel() * 2)
    assert "DeviceToDevice bytes=" in K.ops.last_launch()
    torch.cuda.synchronize()
    got = host_u16(copy).reshape(ids.size, 2 * hidden)
    assert np.array_equal(got[:, :hidden], host_u16(out16)) and np.array_equal(got[:, hidden:], host_u16(other))


def test_reference_smoke_entries_run():
    lib = K.load()
    assert lib.berth_exl3_smoke_int8(0) == 0 and lib.berth_exl3_smoke_int8(1) == 0 and lib.berth_exl3_smoke_gemm() == 0
