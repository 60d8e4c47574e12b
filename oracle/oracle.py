"""ctypes binding of the CPU oracle (oracle/libberth_oracle.so).

TEST INFRASTRUCTURE ONLY: importable from tests/, the smoke check and the
CPU-baseline leg of the benchmark.  The product never imports this module.
All arrays are numpy; fp16 data travels as uint16 bit patterns or float16.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libberth_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return _LIB_PATH


class _LinT(C.Structure):
    _fields_ = [("trellis", C.c_void_p), ("suh", C.c_void_p), ("svh", C.c_void_p)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        L.bo_trellis_state.restype = C.c_uint32
        L.bo_decode_state.restype = C.c_uint16
        L.bo_f32_to_f16.restype = C.c_uint16
        L.bo_f32_to_f16.argtypes = [C.c_float]
        L.bo_f64_to_f16.restype = C.c_uint16
        L.bo_f64_to_f16.argtypes = [C.c_double]
        L.bo_f16_to_f32.restype = C.c_float
        L.bo_f16_to_f32.argtypes = [C.c_uint16]
        L.bo_unpack_signs.restype = C.c_long
        L.bo_silu_mul_f16.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_float]
        L.bo_rms_norm.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_float,
                                  C.c_float, C.c_float, C.c_int]
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _u16(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype in (np.uint16, np.int16), a.dtype
    return a.view(np.uint16)


def tile_perm() -> np.ndarray:
    out = np.zeros(256, dtype=np.int32)
    lib().bo_tile_perm(_p(out))
    return out


def trellis_state(tile_words, bits: int, t: int) -> int:
    w = _u16(tile_words)
    return int(lib().bo_trellis_state(_p(w), int(bits), int(t)))


def decode_state(state: int, cb: int) -> int:
    return int(lib().bo_decode_state(C.c_uint32(state), int(cb)))


def decode_table(cb: int) -> np.ndarray:
    """fp16 bit pattern of every 16-bit state."""
    return np.array([decode_state(s, cb) for s in range(65536)], dtype=np.uint16)


def dequant(trellis, size_k: int, size_n: int, bits: int, cb: int) -> np.ndarray:
    tr = _u16(trellis)
    assert tr.size == (size_k // 16) * (size_n // 16) * 16 * bits
    out = np.empty((size_k, size_n), dtype=np.uint16)
    rc = lib().bo_dequant(_p(tr), size_k, size_n, bits, cb, _p(out))
    if rc:
        raise ValueError("bo_dequant: bad shape")
    return out.view(np.float16)


def reconstruct_had(trellis, suh, svh, size_k: int, size_n: int, bits: int, cb: int) -> np.ndarray:
    """fp16 [size_k][size_n] effective weight diag(suh) Hh W Hh diag(svh)."""
    tr = _u16(trellis)
    assert tr.size == (size_k // 16) * (size_n // 16) * 16 * bits
    out = np.empty((size_k, size_n), dtype=np.uint16)
    rc = lib().bo_reconstruct_had(_p(tr), _p(_u16(suh)), _p(_u16(svh)), size_k, size_n, bits, cb, _p(out))
    if rc:
        raise ValueError("bo_reconstruct_had: bad shape")
    return out.view(np.float16)


def unpack_signs(packed: bytes) -> np.ndarray:
    buf = np.frombuffer(packed, dtype=np.uint8).copy()
    out = np.empty(max(1, len(packed) // 2 * 16), dtype=np.uint16)
    n = lib().bo_unpack_signs(_p(buf), C.c_size_t(len(packed)), _p(out))
    if n < 0:
        raise ValueError("su: packed sign bytes are not a multiple of 2")
    return out[:n]


def had128(v) -> np.ndarray:
    v = np.array(v, dtype=np.float32).copy()
    assert v.size == 128
    lib().bo_had128(_p(v))
    return v


def had_rows_f16(x, scale, pre: bool) -> np.ndarray:
    x16 = _u16(x)
    rows, cols = x16.shape
    out = np.empty_like(x16)
    sc = None if scale is None else _u16(scale)
    rc = lib().bo_had_rows_f16(_p(x16), _p(out), _p(sc), int(pre), rows, cols)
    if rc:
        raise ValueError("bo_had_rows_f16: bad shape")
    return out.view(np.float16)


def had_rows_f32(x, scale, pre: bool) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, cols = x.shape
    out = np.empty_like(x)
    sc = None if scale is None else _u16(scale)
    rc = lib().bo_had_rows_f32(_p(x), _p(out), _p(sc), int(pre), rows, cols)
    if rc:
        raise ValueError("bo_had_rows_f32: bad shape")
    return out


def linear(a, trellis, suh, svh, size_k, size_n, bits, cb, out_fp32=False, acc64=False):
    """Returns (c, a_had)."""
    a16 = _u16(a).reshape(-1, size_k)
    m = a16.shape[0]
    c = np.empty((m, size_n), dtype=np.float32 if out_fp32 else np.uint16)
    a_had = np.empty((m, size_k), dtype=np.uint16)
    rc = lib().bo_linear(_p(a16), _p(_u16(trellis)), _p(c), _p(_u16(suh)), _p(a_had),
                         _p(_u16(svh)), m, size_k, size_n, bits, cb, int(out_fp32), int(acc64))
    if rc:
        raise ValueError("bo_linear: bad shape")
    return (c if out_fp32 else c.view(np.float16)), a_had.view(np.float16)


def linear_w(a, w, suh, svh, out_fp32=False, acc64=False):
    w16 = _u16(w)
    size_k, size_n = w16.shape
    a16 = _u16(a).reshape(-1, size_k)
    m = a16.shape[0]
    c = np.empty((m, size_n), dtype=np.float32 if out_fp32 else np.uint16)
    a_had = np.empty((m, size_k), dtype=np.uint16)
    rc = lib().bo_linear_w(_p(a16), _p(w16), _p(c), _p(_u16(suh)), _p(a_had), _p(_u16(svh)),
                           m, size_k, size_n, int(out_fp32), int(acc64))
    if rc:
        raise ValueError("bo_linear_w: bad shape")
    return (c if out_fp32 else c.view(np.float16)), a_had.view(np.float16)


def gemv_fused(a, trellis, suh, svh, size_k, size_n, bits, cb, out_fp32=False):
    a16 = _u16(a).reshape(size_k)
    c = np.empty(size_n, dtype=np.float32 if out_fp32 else np.uint16)
    a_had = np.empty(size_k, dtype=np.uint16)
    rc = lib().bo_gemv_fused(_p(a16), _p(_u16(trellis)), _p(c), _p(_u16(suh)), _p(a_had),
                             _p(_u16(svh)), size_k, size_n, bits, cb, int(out_fp32))
    if rc:
        raise ValueError("bo_gemv_fused: bad shape")
    return (c if out_fp32 else c.view(np.float16)), a_had.view(np.float16)


def hgemm(a, b, c_fp32=False):
    a16, b16 = _u16(a), _u16(b)
    m, k = a16.shape
    k2, n = b16.shape
    assert k == k2
    c = np.empty((m, n), dtype=np.float32 if c_fp32 else np.uint16)
    rc = lib().bo_hgemm(_p(a16), _p(b16), _p(c), m, k, n, n, int(c_fp32))
    if rc:
        raise ValueError("bo_hgemm: bad shape")
    return c if c_fp32 else c.view(np.float16)


def silu_mul(gate, up, act_limit: float = 0.0) -> np.ndarray:
    g, u = _u16(gate).reshape(-1), _u16(up).reshape(-1)
    out = np.empty_like(g)
    rc = lib().bo_silu_mul_f16(_p(g), _p(u), _p(out), g.size, float(act_limit))
    if rc:
        raise ValueError("silu_mul: numel must be positive and even")
    return out.view(np.float16)


def add_f32(a, b) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    c = np.empty_like(a)
    lib().bo_add_f32(_p(a), _p(b), _p(c), a.size)
    return c


def moe_route(x, wr, k: int, bias=None, renorm: bool = True, want_logits: bool = False):
    x16, w16 = _u16(x), _u16(wr)
    T, H = x16.shape
    H2, E = w16.shape
    assert H == H2
    idx = np.empty((T, k), dtype=np.int32)
    w = np.empty((T, k), dtype=np.float32)
    logits = np.empty((T, E), dtype=np.float32) if want_logits else None
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    rc = lib().bo_moe_route(_p(x16), _p(w16), _p(b), T, H, E, k, int(renorm), _p(idx), _p(w),
                            _p(logits))
    if rc:
        raise ValueError("bo_moe_route: bad shape")
    return (idx, w, logits) if want_logits else (idx, w)


def moe_permute(idx, E: int):
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    T, k = idx.shape
    offsets = np.empty(E + 1, dtype=np.int32)
    perm = np.empty(T * k, dtype=np.int32)
    rc = lib().bo_moe_permute(_p(idx), T, k, E, _p(offsets), _p(perm))
    if rc:
        raise ValueError("bo_moe_permute: bad input")
    return offsets, perm


def _lin_array(lins):
    arr = (_LinT * len(lins))()
    keep = []
    for i, (tr, suh, svh) in enumerate(lins):
        tr, suh, svh = _u16(tr), _u16(suh), _u16(svh)
        keep += [tr, suh, svh]
        arr[i].trellis = tr.ctypes.data
        arr[i].suh = suh.ctypes.data
        arr[i].svh = svh.ctypes.data
    return arr, keep


def expert_ffn(x, gate, up, down, I: int, bits: int, cb: int) -> np.ndarray:
    """gate/up/down are (trellis, suh, svh) triples; returns fp32 [m][H]."""
    x16 = _u16(x)
    m, H = x16.shape
    arr, keep = _lin_array([gate, up, down])
    out = np.empty((m, H), dtype=np.float32)
    rc = lib().bo_expert_ffn(_p(x16), m, H, I, bits, cb, C.byref(arr[0]), C.byref(arr[1]),
                             C.byref(arr[2]), _p(out))
    del keep
    if rc:
        raise ValueError("bo_expert_ffn failed")
    return out


def moe_shared_gate(x, wg):
    """scale[t] = sigmoid(x[t] . wg), the dot product in the routing's arithmetic."""
    x16 = _u16(x)
    T, H = x16.shape
    g = np.ascontiguousarray(wg, dtype=np.float32).ravel()
    out = np.empty(T, dtype=np.float32)
    if g.size != H or lib().bo_moe_shared_gate(_p(x16), _p(g), T, H, _p(out)):
        raise ValueError("bo_moe_shared_gate: bad shape")
    return out


def moe_layer(x, wr, experts, k: int, I: int, bits: int, cb: int, bias=None, renorm=True,
              shared=None, shared_I: int = 0, shared_gate=None):
    """experts: list of E (gate, up, down) with each a (trellis, suh, svh) triple; shared_gate:
    optional fp32 [H] weights of the per-token scale on the shared expert's row.
    Returns (out fp32 [T][H], idx, w)."""
    x16, w16 = _u16(x), _u16(wr)
    T, H = x16.shape
    E = w16.shape[1]
    flat = [lin for ex in experts for lin in ex]
    arr, keep = _lin_array(flat)
    sh_arr, sh_keep = (None, None)
    if shared is not None:
        sh_arr, sh_keep = _lin_array(list(shared))
    out = np.empty((T, H), dtype=np.float32)
    idx = np.empty((T, k), dtype=np.int32)
    w = np.empty((T, k), dtype=np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    sg = None if shared_gate is None else np.ascontiguousarray(shared_gate, dtype=np.float32).ravel()
    rc = lib().bo_moe_layer_gated(_p(x16), T, H, E, k, I, bits, cb, _p(w16), _p(b), int(renorm),
                                  arr, sh_arr, int(shared_I), _p(sg), _p(out), _p(idx), _p(w))
    del keep, sh_keep
    if rc:
        raise ValueError("bo_moe_layer failed")
    return out, idx, w


def rms_norm(x, weight, epsilon, constant_bias=1.0, constant_scale=1.0, weight_bf16=True, residual=None):
    """x fp32 [rows][dim]; weight: uint16 bit patterns (bf16 or fp16) [dim].  Returns
    y fp16 [rows][dim] (and the updated residual when one is given)."""
    x32 = np.ascontiguousarray(x, dtype=np.float32)
    rows, dim = (1, x32.size) if x32.ndim == 1 else x32.shape
    w16 = np.ascontiguousarray(weight).view(np.uint16)
    y = np.empty((rows, dim), dtype=np.uint16)
    res = None if residual is None else np.array(residual, dtype=np.float32).reshape(rows, dim).copy()
    rc = lib().bo_rms_norm(_p(x32), _p(w16), _p(y), _p(res), rows, dim, C.c_float(epsilon), C.c_float(constant_bias),
                           C.c_float(constant_scale), int(weight_bf16))
    if rc:
        raise ValueError("bo_rms_norm failed")
    return (y.view(np.float16), res) if residual is not None else y.view(np.float16)


def num_threads() -> int:
    return int(lib().bo_num_threads())


def set_num_threads(n: int) -> None:
    lib().bo_set_num_threads(int(n))
