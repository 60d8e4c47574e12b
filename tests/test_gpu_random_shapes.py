"""Seeded sweep of the linear entry points over ragged shapes: row counts on both sides
of every dispatch boundary (1, 8 | 9, 32 | 33, 128 | 129, 256 | 257), K and N that are
not multiples of the tile sizes above 128, every bit rate and codebook, both output
types.  Bars as everywhere: the rotated activation bit-exact, the output within
rtol 2e-3 / atol 1e-3 of the oracle, and a second run of the same call bit-identical."""
import os

import numpy as np
import pytest

from tests.gpu_util import close
from tests.test_gpu_linear import _run_linear

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 7, 8, 9, 31, 32, 33, 64, 100, 127, 128, 129, 144, 145, 255, 256, 257, 300, 513]


def _cases():
    """BERTH_SWEEP_REPEATS (default 2) passes over the row counts, each with fresh shapes;
    BERTH_SWEEP_SEED shifts the seed."""
    rng = np.random.default_rng(20251 + int(os.environ.get("BERTH_SWEEP_SEED", "0")))
    out = []
    for i, m in enumerate(ROWS * int(os.environ.get("BERTH_SWEEP_REPEATS", "2"))):
        Kk = 128 * int(rng.integers(1, 13))
        # mostly narrow outputs, some wide enough for the evenly dealt 128- and 256-row tiles
        N = 128 * int(rng.integers(1, 25)) if i % 4 else 128 * int(rng.integers(100, 140))
        if N > 128 * 25:
            Kk = 128 * int(rng.integers(1, 5))
        bits = int(rng.integers(1, 9))
        cb = int(rng.choice([2, 2, 2, 0, 1]))
        out.append((m, Kk, N, bits, cb, bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("m,Kk,N,bits,cb,fp32", _cases())
def test_linear_ragged_shapes(m, Kk, N, bits, cb, fp32):
    seed = 31 * m + Kk + N + bits
    for prefill in ([False, True] if m > 1 else [False]):
        got, want, ah, want_ah, launch = _run_linear(m, Kk, N, bits, cb, fp32, seed, prefill=prefill)
        assert np.array_equal(ah, want_ah), launch
        bad, worst = close(got, want)
        assert bad == 0, (bad, worst, launch)
        got2, _, _, _, _ = _run_linear(m, Kk, N, bits, cb, fp32, seed, prefill=prefill)
        assert np.array_equal(got.view(np.uint8), got2.view(np.uint8)), launch
