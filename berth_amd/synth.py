"""Seeded synthetic tensors in the shapes the benchmark configurations name.

Everything is numpy (PCG64 via ``default_rng``), so the same seed gives the same
bytes on every host.  fp16 tensors are returned as ``float16`` arrays, trellis
words as ``uint16``.
"""
from __future__ import annotations

import numpy as np

# the 27B-shaped decode linear set: name -> (in-features K, out-features N)
SHAPES_27B = {
    "q_proj": (5120, 6144),
    "k_proj": (5120, 1024),
    "v_proj": (5120, 1024),
    "o_proj": (6144, 5120),
    "gate_proj": (5120, 17408),
    "up_proj": (5120, 17408),
    "down_proj": (17408, 5120),
}


def trellis_words(seed: int, size_k: int, size_n: int, bits: int) -> np.ndarray:
    """Uniform uint16 words, shape (K/16, N/16, 16*bits)."""
    rng = np.random.default_rng(seed)
    shape = (size_k // 16, size_n // 16, 16 * bits)
    return rng.integers(0, 65536, size=shape, dtype=np.uint16)


def sign_scale(seed: int, n: int) -> np.ndarray:
    """fp16 random +-1 signs times lognormal(0, 0.1) magnitudes (suh / svh)."""
    rng = np.random.default_rng(seed)
    sign = rng.integers(0, 2, size=n).astype(np.float64) * 2.0 - 1.0
    mag = np.exp(rng.normal(0.0, 0.1, size=n))
    return (sign * mag).astype(np.float16)


def activations(seed: int, rows: int, cols: int) -> np.ndarray:
    """fp16 N(0, 1)."""
    rng = np.random.default_rng(seed)
    return rng.normal(0.0, 1.0, size=(rows, cols)).astype(np.float16)


def router_weight(seed: int, hidden: int, experts: int) -> np.ndarray:
    """fp16 N(0, 0.02), shape (hidden, experts)."""
    rng = np.random.default_rng(seed)
    return rng.normal(0.0, 0.02, size=(hidden, experts)).astype(np.float16)


def zipf_bias(seed: int, experts: int, s: float = 1.1) -> np.ndarray:
    """fp32 per-expert logit bias -s*ln(rank), rank a seeded permutation of
    1..E, so that expert popularity follows Zipf(s)."""
    rng = np.random.default_rng(seed)
    rank = rng.permutation(experts) + 1
    return (-s * np.log(rank.astype(np.float64))).astype(np.float32)


def linear(seed: int, size_k: int, size_n: int, bits: int):
    """(trellis, suh, svh) of one EXL3 linear."""
    return (trellis_words(seed, size_k, size_n, bits),
            sign_scale(seed + 1, size_k),
            sign_scale(seed + 2, size_n))
