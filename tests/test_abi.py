"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and validates arguments before any device call (the
host-only tests of crates/berth-kernels/src/lib.rs:235-319 and
crates/berth-kernels/src/prefill_lin.rs:338-383, with dangling pointers)."""
import ctypes as C
import os
import re

import pytest

from berth_amd import kernels as K
from berth_amd.kernels import Codebook, LaunchError, OutDtype

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
P = 0x1000   # non-null, never dereferenced: the checks return first


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(berth_[a-z0-9_]+)\s*\(", text)))


def test_kernel_library_exports_every_declared_symbol():
    lib = K.load()
    names = _declared("berth_kernels_hip.h")
    assert "berth_exl3_linear" in names and "berth_ops_silu_mul" in names
    for name in names:
        assert getattr(lib, name) is not None, name


def test_runtime_library_exports_every_declared_symbol():
    path = os.path.join(ROOT, "berth_amd", "lib", "libberth_hip.so")
    lib = C.CDLL(path)
    names = _declared("berth_hip.h")
    assert len(names) > 20
    for name in names:
        assert getattr(lib, name) is not None, name


def test_reader_library_exports_every_declared_symbol():
    lib = C.CDLL(os.path.join(ROOT, "berth_amd", "lib", "libberth_exl3_reader.so"))
    names = _declared("berth_exl3_reader.h")
    assert "berth_ckpt_open" in names and len(names) >= 20
    for name in names:
        assert getattr(lib, name) is not None, name


def test_reader_library_exports_every_declared_planner_symbol():
    lib = C.CDLL(os.path.join(ROOT, "berth_amd", "lib", "libberth_exl3_reader.so"))
    names = [n for n in _declared("berth_plan.h") if n.startswith("berth_plan_")]
    assert "berth_plan_build" in names and "berth_plan_place" in names and len(names) >= 17
    for name in names:
        assert getattr(lib, name) is not None, name
    # null arguments are refused with a message, not dereferenced
    lib.berth_plan_last_error.restype = C.c_char_p
    assert lib.berth_plan_build(None, None) == -1 and b"null argument" in lib.berth_plan_last_error()
    assert lib.berth_plan_last_error_kind() == 90
    assert lib.berth_plan_place(None, None, None, C.c_size_t(0), None, None, None, None) == -1
    assert lib.berth_plan_is_routed_expert(None) == 0


def test_linear_null_and_bad_sizes_do_not_touch_the_device():
    with pytest.raises(LaunchError, match="null"):
        K.exl3_linear(None, None, None, None, None, None, 1, 128, 256, 4, Codebook.MUL1, OutDtype.F16)
    assert K.last_launch() == ""
    with pytest.raises(LaunchError, match="multiple of 16"):
        K.exl3_linear(P, P, P, P, P, P, 1, 15, 256, 4, Codebook.MUL1, OutDtype.F32)
    with pytest.raises(LaunchError, match="multiple of 128"):
        K.exl3_linear(P, P, P, P, P, P, 1, 16, 100, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(LaunchError, match="positive"):
        K.exl3_linear(P, P, P, P, P, P, 0, 16, 128, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(LaunchError, match="1..=8"):
        K.exl3_linear(P, P, P, P, P, P, 1, 128, 128, 9, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(LaunchError, match="codebook"):
        K.load().berth_exl3_linear(P, P, P, P, P, P, 1, 128, 128, 4, 3, 0, None) and (_ for _ in ()).throw(
            LaunchError(K.last_error()))
    # size_k = 16 passes the reference's checks; the Hadamard block needs 128
    with pytest.raises(LaunchError, match="multiple of 128"):
        K.exl3_linear(P, P, P, P, P, P, 1, 16, 128, 4, Codebook.MUL1, OutDtype.F16)
    assert K.last_error() != ""


def test_error_is_cleared_by_the_next_failure_and_is_per_family():
    with pytest.raises(LaunchError):
        K.exl3_linear(None, None, None, None, None, None, 1, 128, 256, 4, Codebook.MUL1, OutDtype.F16)
    first = K.last_error()
    with pytest.raises(LaunchError):
        K.ops.silu_mul(P, P, P, 3)
    assert K.last_error() == first            # the ops family has its own slot
    assert "even" in K.ops.last_error()


def test_prefill_validation_order():
    with pytest.raises(LaunchError, match="null"):
        K.prefill_lin.exl3_linear(None, P, P, P, P, P, None, 2, 128, 128, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(LaunchError, match="size_m must be > 1"):
        K.prefill_lin.exl3_linear(P, P, P, P, P, P, None, 1, 128, 128, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(LaunchError, match="multiple of 16"):
        K.prefill_lin.exl3_linear(P, P, P, P, P, P, None, 2, 24, 128, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(LaunchError, match="w_scratch"):
        K.prefill_lin.exl3_linear(P, P, P, P, P, P, None, 145, 128, 128, 4, Codebook.MUL1, OutDtype.F16)
    assert K.prefill_lin.last_launch() == ""
    with pytest.raises(LaunchError, match="bad shape"):
        K.prefill_lin.hgemm(P, P, P, 4, 8, 16, 8, OutDtype.F16)
    with pytest.raises(LaunchError, match="null"):
        K.prefill_lin.hgemm(None, P, P, 4, 8, 16, 16, OutDtype.F16)
    with pytest.raises(LaunchError, match="slice exceeds"):
        K.prefill_lin.reconstruct(P, P, 128, 256, 256, 128, 4, Codebook.MUL1)
    with pytest.raises(LaunchError, match="had columns"):
        K.prefill_lin.had_r_128(P, P, P, True, 1, 100, False)


def test_silu_mul_validation():
    with pytest.raises(LaunchError, match="null"):
        K.ops.silu_mul(None, P, P, 4)
    with pytest.raises(LaunchError, match="positive and even"):
        K.ops.silu_mul(P, P, P, 0)
    assert K.ops.last_launch() == ""


def test_unpack_signs_validation():
    # crates/berth-exl3/src/signs.rs:26-34: odd byte counts are rejected before anything runs
    with pytest.raises(LaunchError, match="su.*not a multiple of 2"):
        K.unpack_signs(P, P, 3)
    with pytest.raises(LaunchError, match="null"):
        K.unpack_signs(None, P, 4)
    K.unpack_signs(None, None, 0)       # empty input: nothing to do


def test_glue_op_validation():
    # crates/berth-kernels/csrc/ops/norm.cu:108-125 and add.cu: refused before any device call
    with pytest.raises(LaunchError, match="rms_norm: null"):
        K.ops.rms_norm(None, P, P, 1, 128, 1e-6)
    with pytest.raises(LaunchError, match="rms_norm: null"):
        K.ops.rms_norm_res_in(P, P, P, None, 1, 128, 1e-6)
    with pytest.raises(LaunchError, match="positive"):
        K.ops.rms_norm(P, P, P, 0, 128, 1e-6)
    with pytest.raises(LaunchError, match="multiple of 4"):
        K.ops.rms_norm(P, P, P, 1, 130, 1e-6)
    with pytest.raises(LaunchError, match="add_f32: null"):
        K.ops.add_f32(P, None, P, 4)
    with pytest.raises(LaunchError, match="n must be positive"):
        K.ops.add_f32(P, P, P, 0)


def test_mgemm_validation():
    with pytest.raises(LaunchError, match="null"):
        K.ops.exl3_mgemm(None, P, P, P, P, P, 1, 128, 128, 4, Codebook.MUL1, OutDtype.F16, 1, 2)
    with pytest.raises(LaunchError, match="sliced mode requires"):
        K.ops.exl3_mgemm(P, P, P, P, P, P, 1, 128, 128, 4, Codebook.MUL1, OutDtype.F16, 1, 2, size_n_list=P)
    with pytest.raises(LaunchError, match="single-input"):
        K.ops.exl3_mgemm(P, P, P, P, P, P, 1, 128, 128, 4, Codebook.MUL1, OutDtype.F16, 2, 2, P, P, P, P, 1)
    with pytest.raises(LaunchError, match="num_had_src requires"):
        K.ops.exl3_mgemm(P, P, P, P, P, P, 1, 128, 128, 4, Codebook.MUL1, OutDtype.F16, 1, 2, num_had_src=1)


def test_fused_mlp_validation():
    P = 0x1000
    lins = [(P, P, P)] * 3
    with pytest.raises(LaunchError, match="null"):
        K.exl3_mlp(None, lins, P, P, P, P, P, 1, 256, 384, 4, Codebook.MUL1)
    with pytest.raises(LaunchError, match="null"):
        K.exl3_mlp(P, [(P, P, P), (P, None, P), (P, P, P)], P, P, P, P, P, 1, 256, 384, 4, Codebook.MUL1)
    with pytest.raises(LaunchError, match="positive"):
        K.exl3_mlp(P, lins, P, P, P, P, P, 0, 256, 384, 4, Codebook.MUL1)
    with pytest.raises(LaunchError, match="multiple of 128"):
        K.exl3_mlp(P, lins, P, P, P, P, P, 1, 256, 200, 4, Codebook.MUL1)
    with pytest.raises(LaunchError, match="1..=8"):
        K.exl3_mlp(P, lins, P, P, P, P, P, 1, 256, 384, 9, Codebook.MUL1)
    assert K.last_launch() == ""


def test_no_alloc_linear_validates_before_any_device_call():
    """berth_exl3_linear_noalloc: the same checks as berth_exl3_linear plus its own limits,
    all ahead of the first device call (dangling pointers, no GPU needed)."""
    with pytest.raises(LaunchError, match="null"):
        K.exl3_linear_noalloc(None, P, P, P, P, P, 1, 128, 256, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(LaunchError, match="multiple of 128"):
        K.exl3_linear_noalloc(P, P, P, P, P, P, 1, 128, 100, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(LaunchError, match="at most 8 rows"):
        K.exl3_linear_noalloc(P, P, P, P, P, P, 9, 128, 256, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(LaunchError, match="counter table"):
        K.exl3_linear_noalloc(P, P, P, P, P, P, 1, 128, 128 * 65537, 4, Codebook.MUL1, OutDtype.F16)
    assert K.last_launch() == ""


def test_every_symbol_the_reference_crate_binds_for_the_path_is_exported():
    """tests/golden/reference_extern_symbols.json lists what the reference's `extern "C"` blocks
    declare (crates/berth-kernels/src/{ffi,prefill_lin,ops}.rs): with all of them exported the
    unchanged Rust modules link against libberth_kernels_hip.so."""
    import json
    lib = K.load()
    listed = json.load(open(os.path.join(ROOT, "tests", "golden", "reference_extern_symbols.json")))
    declared = set(_declared("berth_kernels_hip.h"))
    names = [n for entry in listed.values() for kind in ("always", "test_only") for n in entry[kind]]
    assert len(names) == 25
    for name in names:
        assert hasattr(lib, name), name
        assert name in declared, f"{name} is exported but not declared in include/berth_kernels_hip.h"


def test_tune_keys_reproduce_the_reference_known_answers():
    """crates/berth-kernels/src/lib.rs:223-233 (lm_head key and its salted form) and
    src/ops.rs:738-770 (the two 27B bundle keys): pure host hashes, no device call."""
    lib = K.load()
    key = lib.berth_exl3_gemm_tune_key(1, 5120, 248320, 6, 0, 0, 2, 82, int(Codebook.MUL1))
    assert key == 0x51F40C1BD7CAE3A7
    assert lib.berth_exl3_salt_hash(key) == 0x0C94364FADC0CDF9
    assert lib.berth_ops_mgemm_tune_key(1, 5120, 2048, 4, 1, 0, 2, 82, int(Codebook.MUL1), 1, 8, 1) == 0xD2297A8A33A33F5B
    assert lib.berth_ops_mgemm_tune_key(1, 5120, 1024, 4, 0, 0, 2, 82, int(Codebook.MUL1), 1, 14, 1) == 0x9C25A0752178FB4A
    # m = 1 shares the m = 2 entry of the single-linear key; the bundle key keeps m = 1 apart
    assert lib.berth_exl3_gemm_tune_key(2, 5120, 248320, 6, 0, 0, 2, 82, 2) == key
    assert lib.berth_ops_mgemm_tune_key(2, 5120, 2048, 4, 1, 0, 2, 82, 2, 1, 8, 1) != 0xD2297A8A33A33F5B


def test_gemv_cfg_table_of_the_reference():
    """The rows of crates/berth-kernels/src/prefill_lin.rs:385-442 (cc 2 = Ampere, 3 = Ada,
    mode 1, 4 bpw, mul1, 164 co-resident narrow workgroups)."""
    cfg = K.load().berth_exl3_gemv_cfg
    AMPERE, ADA, MODE, BITS, CB, NARROW = 2, 3, 1, 4, 2, 164
    for m in (3, 5, 8):
        assert cfg(AMPERE, m, 5120, 17408, BITS, CB, MODE, NARROW) == -1      # gate / up
        assert cfg(AMPERE, m, 17408, 5120, BITS, CB, MODE, NARROW) == 0       # down
        assert cfg(AMPERE, m, 6144, 5120, BITS, CB, MODE, NARROW) == 0        # o_proj
        assert cfg(AMPERE, m, 10240, 5120, BITS, CB, MODE, NARROW) == 0       # mtp.fc
    assert cfg(AMPERE, 9, 17408, 5120, BITS, CB, MODE, NARROW) == -1
    assert cfg(AMPERE, 2, 17408, 5120, BITS, CB, MODE, NARROW) == 0
    assert cfg(AMPERE, 3, 17408, 5120, BITS, CB, 0, NARROW) == -1
    assert cfg(AMPERE, 3, 5120, 8192, BITS, CB, MODE, NARROW) == 1
    assert cfg(ADA, 3, 5120, 8192, BITS, CB, MODE, NARROW) == -1
    # forced modes and the other bit rates
    assert cfg(AMPERE, 3, 5120, 8192, BITS, CB, 2, NARROW) == 0 and cfg(AMPERE, 3, 5120, 8320, BITS, CB, 2, NARROW) == 1
    assert cfg(AMPERE, 3, 5120, 17408, BITS, CB, 3, NARROW) == 0 and cfg(AMPERE, 3, 5120, 1024, BITS, CB, 4, NARROW) == 1
    assert cfg(AMPERE, 3, 5120, 17408, 2, CB, MODE, NARROW) == 1 and cfg(AMPERE, 3, 5120, 17408, 5, CB, MODE, NARROW) == -1
    assert cfg(AMPERE, 3, 5120, 17408, 3, 0, MODE, NARROW) == -1 and cfg(AMPERE, 3, 5100, 17408, BITS, CB, MODE, NARROW) == -1


def test_glue_ops_validate_before_any_device_call():
    """Messages of crates/berth-kernels/csrc/ops/{embed,copy,norm}.cu, with dangling pointers."""
    with pytest.raises(LaunchError, match="embed_tokens: null device pointer"):
        K.ops.embed_tokens(None, P, P, 16, 1)
    with pytest.raises(LaunchError, match="embed_tokens_f16: hidden and n must be positive"):
        K.ops.embed_tokens(P, P, P, 0, 1, f16=True)
    with pytest.raises(LaunchError, match="memcpy_d2d: byte count is 0"):
        K.ops.memcpy_d2d(P, P, 0)
    with pytest.raises(LaunchError, match="cat_f16_last: rows and hidden must be positive"):
        K.ops.cat_f16_last(P, P, P, 0, 8)
    with pytest.raises(LaunchError, match="rms_norm: dim must be a multiple of 4"):
        K.ops.rms_norm_f16(P, P, P, 1, 6, 1e-6)
    assert K.ops.last_launch() == ""
