"""ctypes binding of libberth_kernels_hip.so, shaped like the reference's
`berth_kernels` crate (crates/berth-kernels/src/{lib,prefill_lin,ops}.rs): raw
device addresses in, a launch error raised with the shim's message, and
`last_launch()` naming the kernel that ran.

There is no fallback: if the HIP library is missing every call raises.
"""
from __future__ import annotations

import ctypes as C
import enum
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libberth_kernels_hip.so")


class LaunchError(RuntimeError):
    """crates/berth-kernels/src/error.rs `Error::Launch`."""


class Codebook(enum.IntEnum):
    """crates/berth-kernels/src/lib.rs:54-63."""
    DEFAULT = 0
    MCG = 1
    MUL1 = 2


class OutDtype(enum.IntEnum):
    """crates/berth-kernels/src/lib.rs:69-85 (`as_c`)."""
    F16 = 0
    F32 = 1


_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LaunchError(
                f"{LIB_PATH} is missing: build it with `python -m berth_amd.build` "
                "(there is no CPU fallback)")
        L = C.CDLL(LIB_PATH)
        vp, ci = C.c_void_p, C.c_int
        L.berth_exl3_linear.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, vp]
        L.berth_exl3_linear_noalloc.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, vp]
        L.berth_prefill_exl3_linear.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, vp]
        L.berth_prefill_hgemm.argtypes = [vp, vp, vp, ci, ci, ci, ci, ci, vp]
        L.berth_prefill_reconstruct.argtypes = [vp, vp, ci, ci, ci, ci, ci, ci, vp]
        L.berth_prefill_reconstruct_had.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, vp]
        L.berth_prefill_had_r_128.argtypes = [vp, vp, vp, ci, ci, ci, ci, vp]
        L.berth_ops_silu_mul.argtypes = [vp, vp, vp, C.c_int64, C.c_float, vp]
        L.berth_ops_rms_norm.argtypes = [vp, vp, vp, ci, ci, C.c_float, C.c_float, C.c_float, ci, vp]
        L.berth_ops_rms_norm_res_in.argtypes = [vp, vp, vp, vp, ci, ci, C.c_float, C.c_float, C.c_float, ci, vp]
        L.berth_ops_add_f32.argtypes = [vp, vp, vp, ci, vp]
        L.berth_ops_add_bias.argtypes = [vp, vp, ci, ci, ci, vp]
        L.berth_ops_rms_norm_f16.argtypes = [vp, vp, vp, ci, ci, C.c_float, C.c_float, C.c_float, vp]
        L.berth_ops_embed_tokens.argtypes = [vp, vp, vp, ci, ci, vp]
        L.berth_ops_embed_tokens_f16.argtypes = [vp, vp, vp, ci, ci, vp]
        L.berth_ops_memcpy_d2d.argtypes = [vp, vp, C.c_uint64, vp]
        L.berth_ops_cat_f16_last.argtypes = [vp, vp, vp, ci, ci, vp]
        L.berth_exl3_gemm_tune_key.argtypes = [ci] * 9
        L.berth_exl3_gemm_tune_key.restype = C.c_uint64
        L.berth_exl3_salt_hash.argtypes = [C.c_uint64]
        L.berth_exl3_salt_hash.restype = C.c_uint64
        L.berth_ops_mgemm_tune_key.argtypes = [ci] * 12
        L.berth_ops_mgemm_tune_key.restype = C.c_uint64
        L.berth_exl3_gemv_cfg.argtypes = [ci] * 8
        L.berth_exl3_smoke_int8.argtypes = [ci]
        L.berth_exl3_unpack_signs.argtypes = [vp, vp, C.c_int64, vp]
        L.berth_exl3_mlp.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
        L.berth_exl3_unpack_signs.restype = C.c_int
        L.berth_ops_mgemm.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci, ci, vp, vp, vp, vp, ci, vp]
        L.berth_ops_mgemm_hostlists.argtypes = L.berth_ops_mgemm.argtypes
        for name in ("berth_exl3_last_error", "berth_exl3_last_launch", "berth_prefill_last_error",
                     "berth_prefill_last_launch", "berth_ops_last_error", "berth_ops_last_launch"):
            getattr(L, name).restype = C.c_char_p
        L.berth_moe_route.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
        L.berth_moe_permute.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, vp]
        L.berth_moe_permute_scratch_bytes.argtypes = [ci, ci, ci]
        L.berth_moe_grouped_exl3.argtypes = [vp, vp, vp, ci, vp, ci, ci, ci, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, ci,
                                             ci, vp]
        L.berth_moe_combine.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, vp]
        L.berth_moe_permute_scratch_bytes.restype = C.c_size_t
        L.berth_moe_layer.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, C.c_size_t,
                                      ci, ci, ci, ci, ci, ci, ci, ci, ci, vp]
        L.berth_moe_layer_gated.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, C.c_size_t,
                                            ci, ci, ci, ci, ci, ci, ci, ci, ci, vp]
        L.berth_moe_workspace_bytes.argtypes = [ci] * 6
        L.berth_moe_workspace_bytes.restype = C.c_size_t
        L.berth_moe_workspace_offsets.argtypes = [ci] * 6 + [C.POINTER(C.c_size_t)]
        L.berth_moe_workspace_shared_offsets.argtypes = [ci] * 6 + [C.POINTER(C.c_size_t)]
        L.berth_moe_last_error.restype = C.c_char_p
        L.berth_moe_last_launch.restype = C.c_char_p
        L.berth_kernels_workspace.argtypes = [C.POINTER(vp), C.POINTER(C.c_size_t), C.POINTER(vp), C.POINTER(ci)]
        L.berth_kernels_accumulators.argtypes = [C.POINTER(vp), C.POINTER(ci)]
        L.berth_exl3_mlp_block.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, vp]
        L.berth_kernels_pending_fault.restype = C.c_longlong
        L.berth_kernels_pending_fault.argtypes = [ci]
        L.berth_kernels_reload_env.restype = None
        L.berth_kernels_reload_env.argtypes = []
        L.berth_device_cc.argtypes = [ci]
        L.berth_device_sms.argtypes = [ci]
        _lib = L
    return _lib


def _s(b) -> str:
    return (b or b"").decode("utf-8", "replace")


# ---- crates/berth-kernels/src/lib.rs:135-192
def exl3_linear(a, trellis, c, suh, a_had, svh, size_m, size_k, size_n, k_bits,
                codebook: Codebook, out: OutDtype, stream=None) -> None:
    L = load()
    rc = L.berth_exl3_linear(a, trellis, c, suh, a_had, svh, size_m, size_k, size_n, k_bits,
                             int(codebook), int(out), stream)
    if rc != 0:
        raise LaunchError(last_error() or f"exl3 linear launch failed ({rc})")


def exl3_linear_noalloc(a, trellis, c, suh, a_had, svh, size_m, size_k, size_n, k_bits,
                        codebook: Codebook, out: OutDtype, stream=None) -> None:
    """The same operator for callers that cannot allocate device memory (HIP graph capture,
    tight serving loops): up to 8 rows, split-K scratch in a fixed array inside the library."""
    rc = load().berth_exl3_linear_noalloc(a, trellis, c, suh, a_had, svh, size_m, size_k, size_n, k_bits,
                                          int(codebook), int(out), stream)
    if rc != 0:
        raise LaunchError(last_error() or f"exl3 linear (no allocation) launch failed ({rc})")


class Exl3Lin(C.Structure):
    """`berth_exl3_lin`: device addresses of one linear's trellis, suh and svh."""
    _fields_ = [("trellis", C.c_void_p), ("suh", C.c_void_p), ("svh", C.c_void_p)]


def exl3_mlp(x, lins, gate_out, up_out, a_had, act_had, y, size_m, hidden, intermediate, k_bits,
             codebook: Codebook, stream=None) -> None:
    """y = down(silu(gate(x)) * up(x)): the four calls of crates/berth-engine/src/mlp.rs:118-150
    in one entry (two launches up to 8 rows).  lins: three (trellis, suh, svh) address triples."""
    table = (Exl3Lin * 3)(*[Exl3Lin(*t) for t in lins])
    rc = load().berth_exl3_mlp(x, table, gate_out, up_out, a_had, act_had, y, size_m, hidden, intermediate, k_bits,
                               int(codebook), stream)
    if rc != 0:
        raise LaunchError(last_error() or f"exl3 mlp launch failed ({rc})")


class RmsNorm(C.Structure):
    """`berth_rms_norm`: the norm ahead of an MLP (weight fp16 or bf16 [hidden])."""
    _fields_ = [("weight", C.c_void_p), ("epsilon", C.c_float), ("constant_bias", C.c_float),
                ("constant_scale", C.c_float), ("weight_bf16", C.c_int)]


def exl3_mlp_block(x, residual, residual_out, norm: RmsNorm, lins, h_norm, gate_out, up_out, a_had, act_had, y,
                   size_m, hidden, intermediate, k_bits, codebook: Codebook, stream=None) -> None:
    """berth_exl3_mlp_block: residual add + RMS norm, the MLP, and the residual add behind it
    (two launches for one row of streaming-kernel sizes)."""
    arr = (Exl3Lin * 3)(*[Exl3Lin(*l) for l in lins])
    rc = load().berth_exl3_mlp_block(x, residual, residual_out, C.byref(norm), arr, h_norm, gate_out, up_out, a_had,
                                     act_had, y, size_m, hidden, intermediate, k_bits, int(codebook), stream)
    if rc != 0:
        raise LaunchError(last_error() or f"exl3 mlp block launch failed ({rc})")


def unpack_signs(packed, out, packed_bytes: int, stream=None) -> None:
    """crates/berth-exl3/src/signs.rs:25-46 on device memory: packed su / sv words
    -> fp16 signs (16 per u16 word)."""
    rc = load().berth_exl3_unpack_signs(packed, out, packed_bytes, stream)
    if rc != 0:
        raise LaunchError(last_error() or f"unpack_signs launch failed ({rc})")


def last_launch() -> str:
    return _s(load().berth_exl3_last_launch())


def last_error() -> str:
    return _s(load().berth_exl3_last_error())


def reload_env() -> None:
    """Makes the library read the BERTH_* environment knobs again (it reads them once per
    process): call after changing os.environ inside a running process."""
    load().berth_kernels_reload_env()


def pending_fault(device: int = 0) -> int:
    """0, or the code of a fault a kernel on `device` reported since the last report (cleared
    by this call): berth_kernels_pending_fault."""
    return int(load().berth_kernels_pending_fault(device))


def device_cc(device: int = 0) -> int:
    return load().berth_device_cc(device)


def device_sms(device: int = 0) -> int:
    return load().berth_device_sms(device)


class prefill_lin:
    """crates/berth-kernels/src/prefill_lin.rs."""

    @staticmethod
    def exl3_linear(a, trellis, c, suh, a_had, svh, w_scratch, size_m, size_k, size_n, k_bits,
                    codebook: Codebook, out: OutDtype, stream=None) -> None:
        L = load()
        rc = L.berth_prefill_exl3_linear(a, trellis, c, suh, a_had, svh, w_scratch, size_m, size_k,
                                         size_n, k_bits, int(codebook), int(out), stream)
        if rc != 0:
            raise LaunchError(prefill_lin.last_error() or f"prefill exl3 linear launch failed ({rc})")

    @staticmethod
    def hgemm(a, b, c, size_m, size_k, size_n, ldc, out: OutDtype, stream=None) -> None:
        rc = load().berth_prefill_hgemm(a, b, c, size_m, size_k, size_n, ldc, int(out), stream)
        if rc != 0:
            raise LaunchError(prefill_lin.last_error() or f"prefill hgemm launch failed ({rc})")

    @staticmethod
    def reconstruct(unpacked, packed, size_k, slice_n, full_n, n_offset, k_bits,
                    codebook: Codebook, stream=None) -> None:
        rc = load().berth_prefill_reconstruct(unpacked, packed, size_k, slice_n, full_n, n_offset,
                                              k_bits, int(codebook), stream)
        if rc != 0:
            raise LaunchError(prefill_lin.last_error() or f"prefill reconstruct launch failed ({rc})")

    @staticmethod
    def reconstruct_had(unpacked, packed, suh, svh, size_k, slice_n, full_n, n_offset, k_bits,
                        codebook: Codebook, stream=None) -> None:
        """Columns n_offset.. of the effective weight diag(suh) Hh W Hh diag(svh) as fp16
        [size_k][slice_n] (crates/berth-kernels/csrc/prefill_lin/reconstruct.cu:96-123)."""
        rc = load().berth_prefill_reconstruct_had(unpacked, packed, suh, svh, size_k, slice_n, full_n, n_offset,
                                                  k_bits, int(codebook), stream)
        if rc != 0:
            raise LaunchError(prefill_lin.last_error() or f"prefill reconstruct_had launch failed ({rc})")

    @staticmethod
    def had_r_128(inp, out, scale, pre_scale: bool, rows, cols, fp32: bool, stream=None) -> None:
        rc = load().berth_prefill_had_r_128(inp, out, scale, int(pre_scale), rows, cols, int(fp32), stream)
        if rc != 0:
            raise LaunchError(prefill_lin.last_error() or f"prefill had_r_128 launch failed ({rc})")

    @staticmethod
    def last_launch() -> str:
        return _s(load().berth_prefill_last_launch())

    @staticmethod
    def last_error() -> str:
        return _s(load().berth_prefill_last_error())


class ops:
    """crates/berth-kernels/src/ops.rs (the EXL3-path subset)."""

    @staticmethod
    def exl3_mgemm(a, b_list, c, suh_list, a_had, svh_list, size_m, size_k, size_n, k_bits,
                   codebook: Codebook, out: OutDtype, bszm_in, bszm_out, size_n_list=None, c_ptrs=None,
                   n_stride_list=None, had_src_list=None, num_had_src=0, stream=None) -> int:
        """crates/berth-kernels/src/ops.rs:317-367; returns the positive tag."""
        rc = load().berth_ops_mgemm(a, b_list, c, suh_list, a_had, svh_list, size_m, size_k, size_n, k_bits,
                                    int(codebook), int(out), bszm_in, bszm_out, size_n_list, c_ptrs,
                                    n_stride_list, had_src_list, num_had_src, stream)
        if rc > 0:
            return rc
        raise LaunchError(ops.last_error() or f"exl3_mgemm launch failed ({rc})")

    @staticmethod
    def exl3_mgemm_hostlists(a, b_list, c, suh_list, a_had, svh_list, size_m, size_k, size_n, k_bits,
                             codebook: Codebook, out: OutDtype, bszm_in, bszm_out, size_n_list=None, c_ptrs=None,
                             n_stride_list=None, had_src_list=None, num_had_src=0, stream=None) -> int:
        """berth_ops_mgemm_hostlists: exl3_mgemm with the seven lists as host arrays (addresses of
        ctypes / numpy buffers); one row, at most 16 slices, streaming-kernel sizes."""
        rc = load().berth_ops_mgemm_hostlists(a, b_list, c, suh_list, a_had, svh_list, size_m, size_k, size_n, k_bits,
                                              int(codebook), int(out), bszm_in, bszm_out, size_n_list, c_ptrs,
                                              n_stride_list, had_src_list, num_had_src, stream)
        if rc > 0:
            return rc
        raise LaunchError(ops.last_error() or f"exl3_mgemm (host lists) launch failed ({rc})")

    @staticmethod
    def rms_norm(x, weight, y, rows: int, dim: int, epsilon: float, constant_bias: float = 1.0,
                 constant_scale: float = 1.0, weight_bf16: bool = True, stream=None) -> None:
        """crates/berth-kernels/src/ops.rs:398-425."""
        rc = load().berth_ops_rms_norm(x, weight, y, rows, dim, epsilon, constant_bias, constant_scale,
                                       int(weight_bf16), stream)
        if rc != 0:
            raise LaunchError(ops.last_error() or f"rms_norm launch failed ({rc})")

    @staticmethod
    def rms_norm_res_in(x, weight, y, residual, rows: int, dim: int, epsilon: float, constant_bias: float = 1.0,
                        constant_scale: float = 1.0, weight_bf16: bool = True, stream=None) -> None:
        """crates/berth-kernels/src/ops.rs:452-486."""
        rc = load().berth_ops_rms_norm_res_in(x, weight, y, residual, rows, dim, epsilon, constant_bias,
                                              constant_scale, int(weight_bf16), stream)
        if rc != 0:
            raise LaunchError(ops.last_error() or f"rms_norm_res_in launch failed ({rc})")

    @staticmethod
    def rms_norm_f16(x, weight, y, rows: int, dim: int, epsilon: float, constant_bias: float = 1.0,
                     constant_scale: float = 1.0, stream=None) -> None:
        """crates/berth-kernels/src/ops.rs:600-640."""
        rc = load().berth_ops_rms_norm_f16(x, weight, y, rows, dim, epsilon, constant_bias, constant_scale, stream)
        if rc != 0:
            raise LaunchError(ops.last_error() or f"rms_norm_f16 launch failed ({rc})")

    @staticmethod
    def embed_tokens(weight, ids, out, hidden: int, n: int, f16: bool = False, stream=None) -> None:
        """crates/berth-kernels/src/ops.rs:554-598 (bf16 rows to fp32, or to fp16)."""
        fn = load().berth_ops_embed_tokens_f16 if f16 else load().berth_ops_embed_tokens
        rc = fn(weight, ids, out, hidden, n, stream)
        if rc != 0:
            raise LaunchError(ops.last_error() or f"embed_tokens launch failed ({rc})")

    @staticmethod
    def memcpy_d2d(dst, src, nbytes: int, stream=None) -> None:
        rc = load().berth_ops_memcpy_d2d(dst, src, nbytes, stream)
        if rc != 0:
            raise LaunchError(ops.last_error() or f"memcpy_d2d failed ({rc})")

    @staticmethod
    def cat_f16_last(embedding, hidden, out, rows: int, hidden_size: int, stream=None) -> None:
        rc = load().berth_ops_cat_f16_last(embedding, hidden, out, rows, hidden_size, stream)
        if rc != 0:
            raise LaunchError(ops.last_error() or f"cat_f16_last launch failed ({rc})")

    @staticmethod
    def add_f32(a, b, c, n: int, stream=None) -> None:
        """crates/berth-kernels/src/ops.rs:540-552."""
        rc = load().berth_ops_add_f32(a, b, c, n, stream)
        if rc != 0:
            raise LaunchError(ops.last_error() or f"add_f32 launch failed ({rc})")

    @staticmethod
    def add_bias(c, bias, rows: int, n: int, c_fp32: bool, stream=None) -> None:
        """c[rows][n] += bias[n] (fp32 bias) on a linear's output as written."""
        rc = load().berth_ops_add_bias(c, bias, rows, n, int(c_fp32), stream)
        if rc != 0:
            raise LaunchError(ops.last_error() or f"add_bias launch failed ({rc})")

    @staticmethod
    def silu_mul(gate, up, out, numel: int, act_limit: float = 0.0, stream=None) -> None:
        rc = load().berth_ops_silu_mul(gate, up, out, numel, act_limit, stream)
        if rc != 0:
            raise LaunchError(ops.last_error() or f"silu_mul launch failed ({rc})")

    @staticmethod
    def last_launch() -> str:
        return _s(load().berth_ops_last_launch())

    @staticmethod
    def last_error() -> str:
        return _s(load().berth_ops_last_error())


class ExpertLinStruct(C.Structure):
    """`berth_exl3_lin`: device pointers of one EXL3 linear."""
    _fields_ = [("trellis", C.c_void_p), ("suh", C.c_void_p), ("svh", C.c_void_p)]


class moe:
    """The MoE entry points (no counterpart in the reference's crate)."""

    @staticmethod
    def route(x, wr, bias, idx, w, logits, parts_scratch, T, H, E, k, renorm=True, stream=None) -> None:
        rc = load().berth_moe_route(x, wr, bias, idx, w, logits, parts_scratch, T, H, E, k, int(renorm), stream)
        if rc != 0:
            raise LaunchError(moe.last_error() or f"moe route launch failed ({rc})")

    @staticmethod
    def permute(idx, offsets, perm, inv, scratch, T, k, E, stream=None) -> None:
        rc = load().berth_moe_permute(idx, offsets, perm, inv, scratch, T, k, E, stream)
        if rc != 0:
            raise LaunchError(moe.last_error() or f"moe permute launch failed ({rc})")

    @staticmethod
    def grouped_exl3(a, a_up, gather, gather_div, experts_dev, lins_per_expert, lin_base, num_lins, c0, c1,
                     permute_scratch, a_had, T, k, E, size_k, size_n, k_bits, codebook, c_fp32, stream=None) -> None:
        """One grouped EXL3 linear (or the gate / up pair) over the rows `permute` sorted by expert."""
        rc = load().berth_moe_grouped_exl3(a, a_up, gather, gather_div, experts_dev, lins_per_expert, lin_base,
                                           num_lins, c0, c1, permute_scratch, a_had, T, k, E, size_k, size_n, k_bits,
                                           int(codebook), int(c_fp32), stream)
        if rc != 0:
            raise LaunchError(moe.last_error() or f"moe grouped linear failed ({rc})")

    @staticmethod
    def combine(slot_out, shared_out, w, inv, out, T, H, k, stream=None) -> None:
        rc = load().berth_moe_combine(slot_out, shared_out, w, inv, out, T, H, k, stream)
        if rc != 0:
            raise LaunchError(moe.last_error() or f"moe combine failed ({rc})")

    @staticmethod
    def permute_scratch_bytes(T, k, E) -> int:
        return int(load().berth_moe_permute_scratch_bytes(T, k, E))

    @staticmethod
    def workspace_bytes(T, H, E, k, I, shared_I=0) -> int:
        return int(load().berth_moe_workspace_bytes(T, H, E, k, I, shared_I))

    @staticmethod
    def workspace_offsets(T, H, E, k, I, shared_I=0) -> dict:
        out = (C.c_size_t * 9)()
        if load().berth_moe_workspace_offsets(T, H, E, k, I, shared_I, out) != 0:
            raise LaunchError("moe: sizes must be positive")
        names = ("idx", "w", "offsets", "perm", "inv", "gate_out", "up_out", "slot_out", "shared_out")
        return dict(zip(names, (int(v) for v in out)))

    @staticmethod
    def workspace_shared_offsets(T, H, E, k, I, shared_I) -> dict:
        """The always-on expert's own gate / up outputs when shared_I != I."""
        out = (C.c_size_t * 2)()
        if load().berth_moe_workspace_shared_offsets(T, H, E, k, I, shared_I, out) != 0:
            raise LaunchError("moe: no separate buffers for the shared expert at these sizes")
        return {"shared_gate_out": int(out[0]), "shared_up_out": int(out[1])}

    @staticmethod
    def layer(x, wr, bias, experts_dev, shared_host, out, idx_out, w_out, workspace, workspace_bytes,
              T, H, E, k, I, shared_I, k_bits, codebook: Codebook, renorm=True, stream=None, shared_gate=None) -> None:
        """berth_moe_layer; with `shared_gate` (device fp32 [H]) berth_moe_layer_gated."""
        rc = load().berth_moe_layer_gated(x, wr, bias, experts_dev, shared_host, shared_gate, out, idx_out, w_out,
                                          workspace, workspace_bytes, T, H, E, k, I, shared_I, k_bits, int(codebook),
                                          int(renorm), stream)
        if rc != 0:
            raise LaunchError(moe.last_error() or f"moe layer launch failed ({rc})")

    @staticmethod
    def last_launch() -> str:
        return _s(load().berth_moe_last_launch())

    @staticmethod
    def last_error() -> str:
        return _s(load().berth_moe_last_error())
