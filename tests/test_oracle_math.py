"""Pins the oracle's arithmetic (Hadamard, linear, SiLU gate, MoE) against
library routines, closed forms, the reference's fixtures and brute force."""
import os

import numpy as np
import pytest
import scipy.linalg

from berth_amd import synth
from oracle import oracle as O

RS = np.float32(0.088388347648)   # crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:44


# ---- Hadamard
def test_had128_is_sylvester_hadamard():
    H = scipy.linalg.hadamard(128).astype(np.float64)
    rng = np.random.default_rng(0)
    for _ in range(4):
        v = rng.normal(size=128).astype(np.float32)
        assert np.allclose(O.had128(v), H @ v.astype(np.float64), rtol=1e-5, atol=1e-4)
    e0 = np.zeros(128, dtype=np.float32)
    e0[5] = 1.0
    assert np.array_equal(O.had128(e0), H[:, 5].astype(np.float32))   # exact on +-1


def test_had128_involution_symmetry_parseval():
    rng = np.random.default_rng(1)
    v = rng.integers(-8, 9, size=128).astype(np.float32)    # exact in fp32
    hv = O.had128(v)
    assert np.array_equal(O.had128(hv), v * 128)             # H*H = 128 I
    assert float((hv.astype(np.float64) ** 2).sum()) == 128 * float((v.astype(np.float64) ** 2).sum())
    cols = np.stack([O.had128(np.eye(128, dtype=np.float32)[i]) for i in range(128)])
    assert np.array_equal(cols, cols.T) and (cols[0] == 1).all()


def test_had_rows_pre_and_post_scale():
    rng = np.random.default_rng(2)
    x = rng.normal(size=(3, 256)).astype(np.float16)
    sc = synth.sign_scale(9, 256)
    H = scipy.linalg.hadamard(128).astype(np.float64) / np.sqrt(128.0)
    pre = O.had_rows_f16(x, sc, True).astype(np.float64)
    post = O.had_rows_f16(x, sc, False).astype(np.float64)
    xs = x.astype(np.float64) * sc.astype(np.float64)
    for b in range(2):
        s = slice(128 * b, 128 * b + 128)
        assert np.allclose(pre[:, s], xs[:, s] @ H, rtol=2e-3, atol=2e-3)
        assert np.allclose(post[:, s], (x.astype(np.float64)[:, s] @ H) * sc.astype(np.float64)[s],
                           rtol=2e-3, atol=2e-3)
    z = rng.normal(size=(2, 128)).astype(np.float32)
    p32 = O.had_rows_f32(z, sc[:128], False)
    assert np.allclose(p32, (z.astype(np.float64) @ H) * sc[:128].astype(np.float64), rtol=1e-5, atol=1e-5)


# ---- linear: y = x @ diag(suh) Hh W Hh diag(svh)
@pytest.mark.parametrize("bits,cb,out_fp32", [(4, 2, False), (4, 2, True), (2, 2, True), (3, 0, True), (5, 1, False)])
def test_linear_equals_effective_weight_matmul(bits, cb, out_fp32):
    K, N, m = 256, 384, 3
    tr, suh, svh = synth.linear(40 + bits, K, N, bits)
    x = synth.activations(77, m, K)
    W = O.dequant(tr, K, N, bits, cb).astype(np.float64)
    Hh = scipy.linalg.hadamard(128).astype(np.float64) / np.sqrt(128.0)
    Hk = np.kron(np.eye(K // 128), Hh)
    Hn = np.kron(np.eye(N // 128), Hh)
    W_eff = np.diag(suh.astype(np.float64)) @ Hk @ W @ Hn @ np.diag(svh.astype(np.float64))
    want = x.astype(np.float64) @ W_eff
    got, a_had = O.linear(x, tr, suh, svh, K, N, bits, cb, out_fp32=out_fp32, acc64=True)
    # a_had is rounded to fp16 before the matmul; that rounding bounds the error
    scale = np.abs(want).max()
    assert np.abs(got.astype(np.float64) - want).max() < 4e-3 * scale
    assert np.allclose(a_had.astype(np.float64),
                       (x.astype(np.float64) * suh.astype(np.float64)) @ Hk, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("bits,cb", [(4, 2), (3, 2), (4, 0)])
def test_reconstruct_had_is_the_effective_weight(bits, cb):
    """bo_reconstruct_had against the closed form diag(suh) (H/sqrt(128)) W (H/sqrt(128)) diag(svh)
    evaluated per 128 x 128 block in float64 with scipy's Hadamard matrix: the fp16 results agree
    bit for bit on more than 99 % of the elements and to half a unit in the last place everywhere
    (the fp32 butterflies sit between the two roundings), and
    a @ W_eff reproduces bo_linear.  A transposed block, a missing scale or a swapped sign vector
    fails either check."""
    Kk, N = 256, 384
    tr, suh, svh = synth.linear(40 + bits, Kk, N, bits)
    W = O.dequant(tr, Kk, N, bits, cb).astype(np.float64)
    Hh = scipy.linalg.hadamard(128).astype(np.float64) / np.sqrt(128.0)
    exact = np.empty_like(W)
    for kb in range(Kk // 128):
        for nb in range(N // 128):
            blk = W[kb * 128:(kb + 1) * 128, nb * 128:(nb + 1) * 128]
            exact[kb * 128:(kb + 1) * 128, nb * 128:(nb + 1) * 128] = Hh @ blk @ Hh
    exact = suh.astype(np.float64)[:, None] * exact * svh.astype(np.float64)[None, :]
    got = O.reconstruct_had(tr, suh, svh, Kk, N, bits, cb)
    same = got.view(np.uint16) == exact.astype(np.float16).view(np.uint16)
    err = np.abs(got.astype(np.float64) - exact)
    # half a unit in the last place of fp16 plus the fp32 butterflies' own error
    assert same.mean() > 0.99 and (err <= 2.0 ** -11 * np.abs(exact) * 1.01 + 4e-6).all(), (same.mean(), err.max())
    x = synth.activations(41, 5, Kk)
    want, _ = O.linear(x, tr, suh, svh, Kk, N, bits, cb, out_fp32=True, acc64=True)
    y = x.astype(np.float64) @ got.astype(np.float64)
    assert np.linalg.norm(y - want) / np.linalg.norm(want) < 5e-4
    # the wrong way round does not pass
    swapped = O.reconstruct_had(tr, suh[::-1].copy(), svh, Kk, N, bits, cb)
    assert np.linalg.norm(x.astype(np.float64) @ swapped.astype(np.float64) - want) / np.linalg.norm(want) > 0.1


def test_linear_fp32_and_fp64_accumulation_agree_within_tolerance():
    K, N = 512, 256
    tr, suh, svh = synth.linear(3, K, N, 4)
    x = synth.activations(4, 2, K)
    y32, _ = O.linear(x, tr, suh, svh, K, N, 4, 2, out_fp32=True, acc64=False)
    y64, _ = O.linear(x, tr, suh, svh, K, N, 4, 2, out_fp32=True, acc64=True)
    assert np.allclose(y32, y64, rtol=2e-4, atol=1e-4)


def test_linear_is_linear_in_the_activation_after_rotation():
    """zero input -> zero output; unit a_had picks one row of W (through Hh, svh)."""
    K, N = 128, 128
    tr, _, svh = synth.linear(8, K, N, 4)
    suh = np.ones(K, dtype=np.float16)
    zero = np.zeros((1, K), dtype=np.float16)
    y, a_had = O.linear(zero, tr, suh, svh, K, N, 4, 2, out_fp32=True)
    assert not y.any() and not a_had.view(np.uint16).any()
    # x = sqrt(128) * H[:,j] / 128 ... use x = H row j scaled so a_had = e_j exactly:
    H = scipy.linalg.hadamard(128).astype(np.float64)
    j = 17
    x = (H[j] / np.sqrt(128.0) * (1 / RS / np.sqrt(128.0))).astype(np.float16).reshape(1, K)
    y, a_had = O.linear(x, tr, suh, svh, K, N, 4, 2, out_fp32=True, acc64=True)
    W = O.dequant(tr, K, N, 4, 2).astype(np.float64)
    ah = a_had.astype(np.float64)
    want = ((ah @ W) @ (H / np.sqrt(128.0))) * svh.astype(np.float64)
    assert np.allclose(y, want, rtol=1e-5, atol=1e-5)
    assert np.argmax(np.abs(ah)) == j


def test_gemv_fused_equals_materialised_linear():
    K, N = 256, 256
    for bits, cb in [(4, 2), (2, 2), (3, 2), (5, 2), (6, 2), (4, 0)]:
        tr, suh, svh = synth.linear(20 + bits, K, N, bits)
        x = synth.activations(21, 1, K)
        y0, ah0 = O.linear(x, tr, suh, svh, K, N, bits, cb, out_fp32=True)
        y1, ah1 = O.gemv_fused(x, tr, suh, svh, K, N, bits, cb, out_fp32=True)
        assert np.array_equal(ah0.view(np.uint16).reshape(-1), ah1.view(np.uint16))
        assert np.allclose(y0.reshape(-1), y1, rtol=2e-4, atol=2e-4)


def test_hgemm_matches_numpy():
    rng = np.random.default_rng(5)
    a = rng.normal(size=(5, 64)).astype(np.float16)
    b = rng.normal(size=(64, 24)).astype(np.float16)
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert np.allclose(O.hgemm(a, b, True), want, rtol=1e-5, atol=1e-5)
    assert np.allclose(O.hgemm(a, b, False).astype(np.float64), want, rtol=2e-3, atol=2e-3)


# ---- fixtures from the reference's test data
def test_silu_mul_fixture(golden_dir):
    g = np.fromfile(os.path.join(golden_dir, "silu.gate.bin"), dtype=np.float16)
    u = np.fromfile(os.path.join(golden_dir, "silu.up.bin"), dtype=np.float16)
    want = np.fromfile(os.path.join(golden_dir, "silu.out.bin"), dtype=np.float16)
    assert g.size == 17408
    got = O.silu_mul(g, u, 0.0)
    # the fixture is reproduced bit for bit by stepwise fp16 arithmetic
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_add_fixture(golden_dir):
    a = np.fromfile(os.path.join(golden_dir, "add.a.bin"), dtype=np.float32)
    b = np.fromfile(os.path.join(golden_dir, "add.b.bin"), dtype=np.float32)
    c = np.fromfile(os.path.join(golden_dir, "add.c.bin"), dtype=np.float32)
    assert np.array_equal(O.add_f32(a, b).view(np.uint32), c.view(np.uint32))


def test_silu_mul_rejects_odd_numel():
    with pytest.raises(ValueError):
        O.silu_mul(np.zeros(3, np.float16), np.zeros(3, np.float16))


# ---- MoE routing
def _route_bruteforce(x, wr, k, bias=None, renorm=True):
    logits = x.astype(np.float64) @ wr.astype(np.float64)
    if bias is not None:
        logits = logits + bias
    idx = np.argsort(-logits, axis=1, kind="stable")[:, :k]
    p = np.exp(logits - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    w = np.take_along_axis(p, idx, axis=1)
    if renorm:
        w = w / w.sum(axis=1, keepdims=True)
    return idx, w, logits


@pytest.mark.parametrize("T,H,E,k", [(4, 64, 8, 2), (3, 200, 16, 4), (1, 2048, 128, 8), (5, 130, 7, 7)])
def test_route_matches_bruteforce(T, H, E, k):
    x = synth.activations(1, T, H)
    wr = synth.router_weight(2, H, E)
    idx, w, logits = O.moe_route(x, wr, k, want_logits=True)
    bi, bw, bl = _route_bruteforce(x, wr, k)
    assert np.allclose(logits, bl, rtol=1e-4, atol=1e-5)
    # selections agree wherever the k-th and (k+1)-th logits are not within rounding
    srt = np.sort(bl, axis=1)[:, ::-1]
    gap_ok = (np.abs(np.diff(srt, axis=1)).min(axis=1) > 1e-5)
    assert np.array_equal(idx[gap_ok], bi[gap_ok])
    assert np.allclose(w[gap_ok], bw[gap_ok], rtol=1e-4, atol=1e-6)
    assert np.allclose(w.sum(axis=1), 1.0, atol=1e-6)


def test_route_without_renorm_and_with_bias():
    x = synth.activations(3, 6, 96)
    wr = synth.router_weight(4, 96, 12)
    bias = synth.zipf_bias(5, 12)
    idx, w = O.moe_route(x, wr, 3, bias=bias, renorm=False)
    bi, bw, _ = _route_bruteforce(x, wr, 3, bias=bias.astype(np.float64), renorm=False)
    assert np.array_equal(idx, bi)
    assert np.allclose(w, bw, rtol=1e-4, atol=1e-6)


def test_route_ties_go_to_lowest_index_and_one_hot():
    H, E = 64, 8
    x = np.ones((1, H), dtype=np.float16)
    wr = np.zeros((H, E), dtype=np.float16)          # all logits equal
    idx, w = O.moe_route(x, wr, 3)
    assert idx.tolist() == [[0, 1, 2]] and np.allclose(w, 1 / 3)
    wr[:, 5] = 1.0                                    # one dominant expert
    idx, w = O.moe_route(x, wr, 2)
    assert idx[0, 0] == 5 and idx[0, 1] == 0 and w[0, 0] > 0.999999


def test_route_k_equals_E_is_full_softmax():
    x = synth.activations(8, 2, 64)
    wr = synth.router_weight(9, 64, 6)
    idx, w = O.moe_route(x, wr, 6)
    _, _, bl = _route_bruteforce(x, wr, 6)
    p = np.exp(bl - bl.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    assert np.allclose(np.take_along_axis(p, idx.astype(np.int64), axis=1), w, rtol=1e-4)
    assert sorted(idx[0].tolist()) == list(range(6))


def test_permute_is_a_stable_counting_sort():
    rng = np.random.default_rng(6)
    idx = rng.integers(0, 5, size=(7, 3)).astype(np.int32)
    off, perm = O.moe_permute(idx, 5)
    flat = idx.reshape(-1)
    assert np.array_equal(perm, np.argsort(flat, kind="stable").astype(np.int32))
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(np.bincount(flat, minlength=5))]))


# ---- MoE layer
def _experts(seed, E, H, I, bits):
    out = []
    for e in range(E):
        s = seed + 10 * e
        out.append((synth.linear(s, H, I, bits), synth.linear(s + 3, H, I, bits),
                    synth.linear(s + 6, I, H, bits)))
    return out


def test_expert_ffn_composition():
    H, I, bits = 128, 256, 4
    ex = _experts(50, 1, H, I, bits)[0]
    x = synth.activations(51, 2, H)
    got = O.expert_ffn(x, *ex, I=I, bits=bits, cb=2)
    g, _ = O.linear(x, *ex[0], H, I, bits, 2)
    u, _ = O.linear(x, *ex[1], H, I, bits, 2)
    a = O.silu_mul(g, u).reshape(2, I)
    o, _ = O.linear(a, *ex[2], I, H, bits, 2, out_fp32=True)
    assert np.array_equal(got, o)


def test_moe_layer_is_weighted_sum_of_expert_ffns():
    T, H, E, k, I, bits = 3, 128, 4, 2, 128, 4
    x = synth.activations(60, T, H)
    wr = (synth.router_weight(61, H, E).astype(np.float32) * 20).astype(np.float16)
    experts = _experts(62, E, H, I, bits)
    shared = _experts(63, 1, H, I, bits)[0]
    out, idx, w = O.moe_layer(x, wr, experts, k, I, bits, 2, shared=shared, shared_I=I)
    ridx, rw = O.moe_route(x, wr, k)
    assert np.array_equal(idx, ridx) and np.array_equal(w, rw)
    want = O.expert_ffn(x, *shared, I=I, bits=bits, cb=2).astype(np.float64)
    for t in range(T):
        for j in range(k):
            o = O.expert_ffn(x[t:t + 1], *experts[idx[t, j]], I=I, bits=bits, cb=2)
            want[t] += float(w[t, j]) * o[0].astype(np.float64)
    assert np.allclose(out, want, rtol=1e-5, atol=1e-4)


def test_shared_gate_is_a_sigmoid_of_the_dot_product_and_scales_only_the_shared_row():
    T, H, E, k, I, bits = 4, 384, 4, 2, 128, 4
    x = (synth.activations(64, T, H).astype(np.float32) / 8).astype(np.float16)
    wg = (np.random.default_rng(65).standard_normal(H) * 0.7).astype(np.float32)
    scale = O.moe_shared_gate(x, wg)
    z = x.astype(np.float64) @ wg.astype(np.float64)
    assert np.allclose(scale, 1.0 / (1.0 + np.exp(-z)), rtol=2e-6, atol=1e-7)
    assert 0.02 < scale.min() and scale.max() < 0.98 and np.ptp(scale) > 0.1       # the case is not saturated
    # a dropped sign or a missing 1 + would show: sigmoid(-z) = 1 - sigmoid(z), sigmoid(0) = 1/2
    assert np.allclose(O.moe_shared_gate(x, -wg), 1.0 - scale, atol=1e-6)
    assert np.array_equal(O.moe_shared_gate(x, np.zeros(H, np.float32)), np.full(T, 0.5, np.float32))
    wr = (synth.router_weight(66, H, E).astype(np.float32) * 20).astype(np.float16)
    experts = _experts(67, E, H, I, bits)
    shared = _experts(68, 1, H, I, bits)[0]
    routed, idx, w = O.moe_layer(x, wr, experts, k, I, bits, 2)
    plain, _, _ = O.moe_layer(x, wr, experts, k, I, bits, 2, shared=shared, shared_I=I)
    gated, gi, gw = O.moe_layer(x, wr, experts, k, I, bits, 2, shared=shared, shared_I=I, shared_gate=wg)
    assert np.array_equal(gi, idx) and np.array_equal(gw, w)
    sh = O.expert_ffn(x, *shared, I=I, bits=bits, cb=2).astype(np.float64)
    assert np.allclose(plain - routed, sh, rtol=1e-4, atol=1e-4 * np.abs(sh).max())
    assert np.allclose(gated - routed, scale[:, None] * sh, rtol=1e-4, atol=1e-4 * np.abs(sh).max())
    with pytest.raises(ValueError):
        O.moe_shared_gate(x, wg[:-1])


def test_moe_layer_k_equals_E_dense_mixture_identical_tokens():
    T, H, E, I, bits = 2, 128, 2, 128, 3
    x1 = synth.activations(70, 1, H)
    x = np.repeat(x1, T, axis=0)
    wr = synth.router_weight(71, H, E)
    experts = _experts(72, E, H, I, bits)
    out, idx, w = O.moe_layer(x, wr, experts, E, I, bits, 2)
    assert np.array_equal(out[0], out[1])
    assert np.allclose(w.sum(axis=1), 1.0, atol=1e-6)
