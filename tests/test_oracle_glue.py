"""Pins the oracle's glue ops around the MLP (RMS norm with and without the fused
residual, fp32 add) against the reference's own fixtures
(testdata/kernels/ops/norm*.bin, add.*.bin, copied as data to tests/golden).

The norm fixtures were produced with checkpoint weights that are not in the tree.
The weight of every channel is recovered from the fixture itself as the bf16 value
nearest to y / (x * rms) - 1; the check is that with those bf16 weights EVERY
output is reproduced bit for bit.  For channels whose weight is large (the final
norm has weights up to 1.7, where neighbouring bf16 values are 3e-3 apart while an
fp16 output pins the product to 2.4e-4) a wrong mean, epsilon, bias or operation
order cannot be absorbed by the choice of weight, so the formula is pinned."""
import os

import numpy as np
import pytest

from oracle import oracle as O

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
EPS = float(np.array([897988541], dtype=np.uint32).view(np.float32)[0])    # meta.json epsilon_f32_bits


def load(name, dtype):
    return np.fromfile(os.path.join(G, name), dtype=dtype)


def to_bf16_bits(v):
    u = np.asarray(v, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def recover_weight(v, y):
    """bf16 bit patterns w with y = fp16(v * rms * (w + 1))."""
    rms = 1.0 / np.sqrt(np.mean(v.astype(np.float64) ** 2) + EPS)
    q = y.astype(np.float64) / (v.astype(np.float64) * rms)
    return to_bf16_bits(q - 1.0)


def test_eps_is_1e_minus_6():
    assert abs(EPS - 1e-6) < 1e-12


@pytest.mark.parametrize("yfile", ["norm_input.y.bin", "norm_final.y.bin"])
def test_rms_norm_reproduces_the_fixture(yfile):
    x, y = load("norm.x.bin", np.float32), load(yfile, np.float16)
    assert x.size == 5120 and y.size == 5120
    w = recover_weight(x, y)
    got = O.rms_norm(x, w, EPS, 1.0, 1.0, weight_bf16=True)
    assert np.array_equal(got.view(np.uint16).ravel(), y.view(np.uint16))
    if "final" in yfile:
        wf = (w.astype(np.uint32) << 16).view(np.float32)
        assert (np.abs(wf) >= 1.0).sum() > 100, "no coarse-grid weights: the fixture would pin nothing"


def test_rms_norm_res_in_reproduces_the_fixture():
    x, r = load("norm_res.x.bin", np.float32), load("norm_res.r.bin", np.float32)
    r_out, y = load("norm_res.r_out.bin", np.float32), load("norm_res.y.bin", np.float16)
    w = recover_weight(r_out, y)
    got, res = O.rms_norm(x, w, EPS, 1.0, 1.0, weight_bf16=True, residual=r)
    assert np.array_equal(res.view(np.uint32).ravel(), r_out.view(np.uint32))     # residual += x, exact in fp32
    assert np.array_equal(got.view(np.uint16).ravel(), y.view(np.uint16))


def test_a_wrong_epsilon_or_bias_breaks_the_fixture():
    """Power of the check: the same recovery with a wrong formula does not close."""
    x, y = load("norm.x.bin", np.float32), load("norm_final.y.bin", np.float16)
    w = recover_weight(x, y)
    for eps, bias in ((1e-2, 1.0), (EPS, 0.0)):
        got = O.rms_norm(x, w, eps, bias, 1.0, weight_bf16=True)
        assert (got.view(np.uint16).ravel() != y.view(np.uint16)).mean() > 0.2
    # and a mean over the wrong count cannot be absorbed by re-fitting the weights
    rms_bad = 1.0 / np.sqrt(np.sum(x.astype(np.float64) ** 2) / (x.size - 64) + EPS)
    q = y.astype(np.float64) / (x.astype(np.float64) * rms_bad)
    w_bad = (to_bf16_bits(q - 1.0).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    refit = (x.astype(np.float64) * rms_bad * (w_bad + 1.0)).astype(np.float16)
    assert (refit.view(np.uint16) != y.view(np.uint16)).mean() > 0.02


def test_rms_norm_matches_float64_on_random_rows():
    rng = np.random.default_rng(5)
    x = rng.normal(0, 3, size=(4, 512)).astype(np.float32)
    for bf16 in (True, False):
        wf = rng.normal(0, 0.5, size=512).astype(np.float32)
        bits = to_bf16_bits(wf) if bf16 else wf.astype(np.float16).view(np.uint16)
        wv = (bits.astype(np.uint32) << 16).view(np.float32) if bf16 else bits.view(np.float16).astype(np.float32)
        got = O.rms_norm(x, bits, 1e-5, 0.5, 2.0, weight_bf16=bf16).astype(np.float64)
        rms = 1.0 / np.sqrt(np.mean(x.astype(np.float64) ** 2, axis=1, keepdims=True) + 1e-5)
        want = x * rms * (wv.astype(np.float64) + 0.5) * 2.0
        assert np.allclose(got, want, rtol=2 ** -10, atol=1e-6)


def test_rms_norm_rejects_bad_sizes():
    with pytest.raises(ValueError):
        O.rms_norm(np.zeros(6, np.float32), np.zeros(6, np.uint16), 1e-6)
