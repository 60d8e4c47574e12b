"""Pins the oracle's format functions (trellis windows, tile order, codebooks,
sign unpack) against independent restatements: big-integer bit strings, exact
rational arithmetic, the constants the reference's PTX probes hold, and the
reference's own known-answer tests."""
from fractions import Fraction

import numpy as np
import pytest

from oracle import oracle as O


# ---- sign unpack: the five known-answer tests of crates/berth-exl3/src/signs.rs:48-92
ONE, NEG = 0x3C00, 0xBC00


def test_signs_bit0_is_negative_one():
    s = O.unpack_signs((1).to_bytes(2, "little"))
    assert len(s) == 16 and s[0] == NEG and all(v == ONE for v in s[1:])


def test_signs_bit15_is_last():
    s = O.unpack_signs((0x8000).to_bytes(2, "little"))
    assert all(v == ONE for v in s[:15]) and s[15] == NEG


def test_signs_all_clear_all_set():
    assert all(v == ONE for v in O.unpack_signs((0).to_bytes(2, "little")))
    assert all(v == NEG for v in O.unpack_signs((0xFFFF).to_bytes(2, "little")))


def test_signs_two_words_contiguous():
    s = O.unpack_signs((5).to_bytes(2, "little") + (1).to_bytes(2, "little"))
    assert len(s) == 32
    assert (s[0], s[1], s[2], s[16], s[17]) == (NEG, ONE, NEG, NEG, ONE)


def test_signs_odd_length_is_error():
    with pytest.raises(ValueError, match="su"):
        O.unpack_signs(b"\x01")


# ---- trellis windows: brute force over a Python big integer
def _bigint_states(words, bits):
    total = 256 * bits
    big = 0
    for w in words:                       # words in order, msb first
        big = (big << 16) | int(w)
    doubled = (big << total) | big        # tail-biting: the stream repeats
    out = []
    for t in range(256):
        end = (t + 1) * bits              # state = the 16 bits ending here
        start = end - 16 + total          # in the second copy, never negative
        shift = 2 * total - (start + 16)
        out.append((doubled >> shift) & 0xFFFF)
    return out


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_trellis_state_matches_bigint(bits):
    rng = np.random.default_rng(100 + bits)
    words = rng.integers(0, 65536, size=16 * bits, dtype=np.uint16)
    want = _bigint_states(words, bits)
    got = [O.trellis_state(words, bits, t) for t in range(256)]
    assert got == want


@pytest.mark.parametrize("bits", [2, 4, 5])
def test_trellis_is_a_shift_register(bits):
    """Successive states overlap: s[t+1] = ((s[t] << bits) | new) mod 2^16,
    and the register wraps from position 255 back to 0."""
    rng = np.random.default_rng(7)
    words = rng.integers(0, 65536, size=16 * bits, dtype=np.uint16)
    s = [O.trellis_state(words, bits, t) for t in range(256)]
    for t in range(256):
        nxt = s[(t + 1) % 256]
        assert nxt >> bits == s[t] & ((1 << (16 - bits)) - 1)


def test_trellis_state_single_bit_probe():
    """One set bit in the stream shows up in exactly ceil(16/bits) windows."""
    bits = 4
    words = np.zeros(64, dtype=np.uint16)
    words[0] = 0x8000                      # stream bit 0
    s = [O.trellis_state(words, bits, t) for t in range(256)]
    # bit 0 belongs to the new bits of position 0 (its top new bit)
    assert s[0] == 0b1000 and s[1] == 0b1000 << 4 and s[3] == 0b1000 << 12
    assert all(v == 0 for v in s[4:])


# ---- tile order: the m16n8k16 B-fragment ownership rule
def test_tile_perm_is_mma_fragment_order():
    perm = O.tile_perm()
    assert sorted(perm.tolist()) == list(range(256))
    for lane in range(32):
        group, tid = lane // 4, lane % 4   # PTX: groupID, threadID_in_group
        for frag in range(2):              # two 16x8 B fragments side by side
            for i in range(4):             # registers b0..b3 hold rows
                row = tid * 2 + (i & 1) + 8 * (i >> 1)
                col = group + 8 * frag
                assert perm[lane * 8 + frag * 4 + i] == row * 16 + col


# ---- codebooks
def _f16(bits):
    return float(np.array([bits], dtype=np.uint16).view(np.float16)[0])


def _round_f16_exact(q: Fraction) -> int:
    """Nearest-even fp16 bit pattern of an exact rational (finite range)."""
    cands = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    vals = cands.view(np.float16).astype(np.float64)
    ok = np.isfinite(vals)
    target = float(q)
    order = np.argsort(np.abs(vals[ok] - target), kind="stable")[:4]
    best = None
    for j in order:
        b = int(cands[ok][j])
        err = abs(Fraction(float(vals[ok][j])) - q)
        key = (err, b & 1, b)              # ties -> even mantissa
        if best is None or key < best[0]:
            best = (key, b)
    return best[1]


def test_mul1_constants_and_fma_rounding():
    """multiplier from ptx/sm86_probes.cu:248; byte sum :143; value =
    round_once((1024 + sum) * k_inv + k_bias) in exact arithmetic."""
    kinv, kbias = Fraction(_f16(0x1EEE)), Fraction(_f16(0xC931))
    by_sum = {}
    rng = np.random.default_rng(3)
    for s in list(range(0, 65536, 257)) + rng.integers(0, 65536, 600).tolist():
        x = (s * 0x83DCD12D) & 0xFFFFFFFF
        t = sum((x >> (8 * i)) & 0xFF for i in range(4))
        if t not in by_sum:
            by_sum[t] = _round_f16_exact((1024 + t) * kinv + kbias)
        assert O.decode_state(s, 2) == by_sum[t], hex(s)
    assert len(by_sum) > 300


def test_mul1_is_unit_gaussian_like():
    """(sum of 4 uniform bytes - 510) / 147.8: mean 0, variance 1 over all states."""
    tab = O.decode_table(2).view(np.float16).astype(np.float64)
    assert abs(tab.mean()) < 0.02
    assert abs(tab.std() - 1.0) < 0.02
    assert len(np.unique(tab)) <= 1021


@pytest.mark.parametrize("cb,mul,add", [(0, 89226354, 64248484), (1, 0xCBAC1FED, 0)])
def test_3inst_family(cb, mul, add):
    """mask / xor from ptx/sm86_probes.cu:157; one fp16 add of the halves."""
    rng = np.random.default_rng(5)
    for s in rng.integers(0, 65536, 500).tolist() + [0, 1, 0xFFFF]:
        x = (s * mul + add) & 0xFFFFFFFF
        x = (x & 0x8FFF8FFF) ^ 0x3B603B60
        want = _round_f16_exact(Fraction(_f16(x & 0xFFFF)) + Fraction(_f16(x >> 16)))
        assert O.decode_state(s, cb) == want


@pytest.mark.parametrize("cb", [0, 1])
def test_3inst_family_is_unit_gaussian_like(cb):
    tab = O.decode_table(cb).view(np.float16).astype(np.float64)
    assert np.isfinite(tab).all()
    assert abs(tab.mean()) < 0.05 and 0.8 < tab.std() < 1.25


# ---- whole-matrix dequant = states -> codebook -> tile placement
@pytest.mark.parametrize("bits,cb", [(2, 2), (3, 2), (4, 2), (5, 2), (4, 0), (4, 1), (8, 2), (1, 2)])
def test_dequant_matches_python_placement(bits, cb):
    K, N = 32, 48
    rng = np.random.default_rng(bits * 10 + cb)
    tr = rng.integers(0, 65536, size=(K // 16, N // 16, 16 * bits), dtype=np.uint16)
    got = O.dequant(tr, K, N, bits, cb).view(np.uint16)
    table = O.decode_table(cb)
    perm = O.tile_perm()
    want = np.zeros((K, N), dtype=np.uint16)
    for kt in range(K // 16):
        for nt in range(N // 16):
            states = _bigint_states(tr[kt, nt], bits)
            for t in range(256):
                r, c = divmod(int(perm[t]), 16)
                want[kt * 16 + r, nt * 16 + c] = table[states[t]]
    assert np.array_equal(got, want)


def test_fp16_conversions_roundtrip_all_bit_patterns():
    bits = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    f = bits.view(np.float16).astype(np.float32)
    L = O.lib()
    for b in list(range(0, 0x10000, 97)) + [0, 1, 0x3FF, 0x400, 0x7BFF, 0x7C00, 0x8000, 0xFBFF]:
        v = L.bo_f16_to_f32(b)
        if np.isnan(f[b]):
            assert np.isnan(v)
            continue
        assert v == f[b]
        assert L.bo_f32_to_f16(v) == b


def test_f32_to_f16_matches_numpy_rounding():
    rng = np.random.default_rng(11)
    vals = np.concatenate([rng.normal(0, 1, 4000), rng.normal(0, 1e-5, 2000),
                           rng.normal(0, 3e4, 2000), [65504.0, 65519.9, 65520.0, 6e-8, 2.98e-8]])
    L = O.lib()
    with np.errstate(over="ignore"):
        for v in vals.astype(np.float32):
            assert L.bo_f32_to_f16(float(v)) == int(np.float32(v).astype(np.float16).view(np.uint16)), v
