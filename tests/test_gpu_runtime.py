"""The device-runtime library (libberth_hip.so, the stand-in for crates/berth-cuda) through
its C ABI: the cases of the reference runtime's own GPU tests (crates/berth-cuda/tests/gpu.rs:
device report, device and pinned copy round trips, event timing across streams, a code-object
launch that writes a scalar, the dynamic-LDS opt-in), plus the remaining entry points (device
copy, asynchronous fill, a stream waiting for another stream's event, both ways of loading a
code object, a launch with dynamic LDS on a stream of its own, the error texts)."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CODE_OBJECT = os.path.join(ROOT, "tests", "runtime_probe.hsaco")


class Runtime:
    def __init__(self):
        L = C.CDLL(os.path.join(ROOT, "berth_amd", "lib", "libberth_hip.so"))
        vp, u64, sz, u32 = C.c_void_p, C.c_uint64, C.c_size_t, C.c_uint32
        L.berth_hip_error_string.restype = C.c_char_p
        L.berth_hip_error_string.argtypes = [C.c_int]
        L.berth_hip_last_error.restype = C.c_char_p
        L.berth_hip_stream_handle.restype = u64
        for name, args in {
            "context_new": [C.c_int, C.POINTER(vp)], "context_free": [vp], "context_ordinal": [vp],
            "context_multiprocessor_count": [vp, C.POINTER(u32)],
            "context_compute_capability": [vp, C.POINTER(C.c_int), C.c_char_p, sz],
            "context_total_memory": [vp, C.POINTER(u64)], "context_synchronize": [vp],
            "stream_new": [vp, C.POINTER(vp)], "stream_free": [vp], "stream_handle": [vp], "stream_synchronize": [vp],
            "stream_wait_event": [vp, vp], "event_new": [vp, C.POINTER(vp)], "event_free": [vp],
            "event_record": [vp, vp], "event_synchronize": [vp], "event_elapsed_ms": [vp, vp, C.POINTER(C.c_float)],
            "buffer_alloc": [vp, sz, C.POINTER(u64)], "buffer_zeroed": [vp, vp, sz, C.POINTER(u64)],
            "buffer_free": [vp, u64], "copy_from_host": [vp, u64, vp, sz], "copy_to_host": [vp, vp, u64, sz],
            "copy_from_host_async": [vp, u64, vp, sz], "copy_to_host_async": [vp, vp, u64, sz],
            "copy_device": [vp, u64, u64, sz], "memset_async": [vp, u64, C.c_int, sz],
            "pinned_alloc": [vp, sz, C.POINTER(vp)], "pinned_free": [vp, vp],
            "module_load_file": [vp, C.c_char_p, C.POINTER(vp)], "module_load_bytes": [vp, vp, sz, C.POINTER(vp)],
            "module_free": [vp], "module_function": [vp, C.c_char_p, C.POINTER(vp)], "function_free": [vp],
            "function_set_max_dynamic_shared_bytes": [vp, u32],
            "function_launch": [vp, vp] + [u32] * 7 + [C.POINTER(vp)],
        }.items():
            getattr(L, "berth_hip_" + name).argtypes = args
        self.L = L
        self.ctx = C.c_void_p()
        self.ok(L.berth_hip_context_new(0, C.byref(self.ctx)))

    def ok(self, rc):
        assert rc == 0, (rc, self.L.berth_hip_error_string(rc), self.L.berth_hip_last_error())

    def __getattr__(self, name):
        return getattr(self.L, "berth_hip_" + name)

    def stream(self):
        s = C.c_void_p()
        self.ok(self.stream_new(self.ctx, C.byref(s)))
        return s

    def event(self):
        e = C.c_void_p()
        self.ok(self.event_new(self.ctx, C.byref(e)))
        return e

    def alloc(self, nbytes, zero_on=None):
        d = C.c_uint64()
        if zero_on is not None:
            self.ok(self.buffer_zeroed(self.ctx, zero_on, nbytes, C.byref(d)))
        else:
            self.ok(self.buffer_alloc(self.ctx, nbytes, C.byref(d)))
        return d

    def pinned(self, nbytes, dtype):
        p = C.c_void_p()
        self.ok(self.pinned_alloc(self.ctx, nbytes, C.byref(p)))
        arr = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_ubyte)), shape=(nbytes,)).view(dtype)
        return p, arr

    def launch(self, fn, stream, grid, block, lds, *args):
        params = (C.c_void_p * len(args))(*[C.cast(C.pointer(a), C.c_void_p) for a in args])
        return self.function_launch(fn, stream, grid, 1, 1, block, 1, 1, lds, params)


@pytest.fixture(scope="module")
def rt():
    r = Runtime()
    yield r
    r.context_free(r.ctx)


def test_device_reports_the_mi355x(rt):
    assert rt.context_ordinal(rt.ctx) == 0
    cus, gfx, total = C.c_uint32(), C.c_int(), C.c_uint64()
    name = C.create_string_buffer(64)
    rt.ok(rt.context_multiprocessor_count(rt.ctx, C.byref(cus)))
    rt.ok(rt.context_compute_capability(rt.ctx, C.byref(gfx), name, 64))
    rt.ok(rt.context_total_memory(rt.ctx, C.byref(total)))
    assert cus.value == 256 and gfx.value == 950 and name.value.startswith(b"gfx950")
    assert total.value > 250 * (1 << 30)            # 288 GB of HBM3E


def test_memcpy_round_trip_device_and_pinned(rt):
    s = rt.stream()
    n = 1 << 16
    src = np.arange(n, dtype=np.int32) * 3 - 7
    a, b = rt.alloc(n * 4), rt.alloc(n * 4, zero_on=s)
    back = np.full(n, -1, dtype=np.int32)
    rt.ok(rt.copy_to_host(s, back.ctypes.data, b, n * 4))
    assert (back == 0).all()                         # buffer_zeroed
    rt.ok(rt.copy_from_host(s, a, src.ctypes.data, n * 4))
    rt.ok(rt.copy_device(s, b, a, n * 4))
    rt.ok(rt.copy_to_host(s, back.ctypes.data, b, n * 4))
    assert np.array_equal(back, src)
    # pinned buffers and the asynchronous copies; an asynchronous byte fill in between
    p_in, h_in = rt.pinned(n * 4, np.int32)
    p_out, h_out = rt.pinned(n * 4, np.int32)
    assert (h_in == 0).all()
    h_in[:] = src[::-1]
    rt.ok(rt.copy_from_host_async(s, a, p_in, n * 4))
    rt.ok(rt.memset_async(s, b, 0x5A, n * 4))
    rt.ok(rt.copy_to_host_async(s, p_out, b, n * 4))
    rt.ok(rt.stream_synchronize(s))
    assert (h_out.view(np.uint8) == 0x5A).all()
    rt.ok(rt.copy_to_host_async(s, p_out, a, n * 4))
    rt.ok(rt.stream_synchronize(s))
    assert np.array_equal(h_out, src[::-1])
    rt.ok(rt.pinned_free(rt.ctx, p_in))
    rt.ok(rt.pinned_free(rt.ctx, p_out))
    rt.ok(rt.buffer_free(rt.ctx, a))
    rt.ok(rt.buffer_free(rt.ctx, b))
    rt.stream_free(s)


def test_event_elapsed_and_a_stream_waiting_for_another(rt):
    s1, s2 = rt.stream(), rt.stream()
    assert rt.stream_handle(s1) != rt.stream_handle(s2) and rt.stream_handle(s1) != 0
    e0, e1 = rt.event(), rt.event()
    n = 1 << 24
    a, b = rt.alloc(n), rt.alloc(n)
    rt.ok(rt.event_record(e0, s1))
    rt.ok(rt.memset_async(s1, a, 7, n))
    rt.ok(rt.event_record(e1, s1))
    rt.ok(rt.stream_wait_event(s2, e1))              # s2's copy must see s1's fill
    rt.ok(rt.copy_device(s2, b, a, n))
    rt.ok(rt.stream_synchronize(s2))
    rt.ok(rt.event_synchronize(e1))
    ms = C.c_float(-1.0)
    rt.ok(rt.event_elapsed_ms(e0, e1, C.byref(ms)))
    assert 0.0 <= ms.value < 1000.0
    back = np.zeros(n, dtype=np.uint8)
    rt.ok(rt.copy_to_host(s2, back.ctypes.data, b, n))
    assert (back == 7).all()
    for e in (e0, e1):
        rt.event_free(e)
    for d in (a, b):
        rt.ok(rt.buffer_free(rt.ctx, d))
    rt.stream_free(s1)
    rt.stream_free(s2)


def _module(rt, how):
    m = C.c_void_p()
    if how == "file":
        rt.ok(rt.module_load_file(rt.ctx, CODE_OBJECT.encode(), C.byref(m)))
        return m, None
    image = open(CODE_OBJECT, "rb").read()
    keep = C.create_string_buffer(image, len(image))
    rt.ok(rt.module_load_bytes(rt.ctx, keep, len(image), C.byref(m)))
    return m, keep


@pytest.mark.parametrize("how", ["file", "bytes"])
def test_code_object_launch_writes_the_scalar(rt, how):
    assert os.path.exists(CODE_OBJECT), "the code object is not built (python -m berth_amd.build)"
    m, _keep = _module(rt, how)
    fn = C.c_void_p()
    rt.ok(rt.module_function(m, b"fill_i32", C.byref(fn)))
    s = rt.stream()
    out = rt.alloc(4, zero_on=s)
    rt.ok(rt.launch(fn, s, 1, 1, 0, C.c_uint64(out.value), C.c_int(0x5EED)))
    got = np.zeros(1, dtype=np.int32)
    rt.ok(rt.copy_to_host(s, got.ctypes.data, out, 4))
    assert got[0] == 0x5EED
    missing = C.c_void_p()
    assert rt.module_function(m, b"no_such_kernel", C.byref(missing)) != 0
    assert b"hipModuleGetFunction" in rt.last_error()
    rt.function_free(fn)
    rt.ok(rt.buffer_free(rt.ctx, out))
    rt.module_free(m)
    rt.stream_free(s)


def test_launch_with_dynamic_lds_on_its_own_stream(rt):
    m, _ = _module(rt, "file")
    fn = C.c_void_p()
    rt.ok(rt.module_function(m, b"axpy_reversed_lds", C.byref(fn)))
    s = rt.stream()
    n, block = 1000, 256
    x = np.random.default_rng(1).normal(size=n).astype(np.float32)
    y = np.random.default_rng(2).normal(size=n).astype(np.float32)
    dx, dy = rt.alloc(n * 4), rt.alloc(n * 4)
    rt.ok(rt.copy_from_host(s, dx, x.ctypes.data, n * 4))
    rt.ok(rt.copy_from_host(s, dy, y.ctypes.data, n * 4))
    grid = (n + block - 1) // block
    rt.ok(rt.launch(fn, s, grid, block, block * 4, C.c_uint64(dx.value), C.c_uint64(dy.value), C.c_float(2.5), C.c_int(n)))
    got = np.zeros(n, dtype=np.float32)
    rt.ok(rt.copy_to_host(s, got.ctypes.data, dy, n * 4))
    xp = np.zeros(grid * block, dtype=np.float32)
    xp[:n] = x
    want = (np.float32(2.5) * xp.reshape(grid, block)[:, ::-1].reshape(-1)[:n] + y).astype(np.float32)
    assert np.array_equal(got, want)
    # refused configurations come back as error codes with a text
    assert rt.launch(fn, s, 0, block, 0, C.c_uint64(dx.value), C.c_uint64(dy.value), C.c_float(1.0), C.c_int(n)) != 0
    assert rt.launch(fn, s, 1, 2048, 0, C.c_uint64(dx.value), C.c_uint64(dy.value), C.c_float(1.0), C.c_int(n)) != 0
    rt.function_free(fn)
    for d in (dx, dy):
        rt.ok(rt.buffer_free(rt.ctx, d))
    rt.module_free(m)
    rt.stream_free(s)


def test_dynamic_lds_opt_in_allows_more_than_64kib(rt):
    m, _ = _module(rt, "bytes")
    fn = C.c_void_p()
    rt.ok(rt.module_function(m, b"touch_dyn_lds", C.byref(fn)))
    s = rt.stream()
    out = rt.alloc(4, zero_on=s)
    nbytes = 96 * 1024
    rt.ok(rt.function_set_max_dynamic_shared_bytes(fn, nbytes))
    rt.ok(rt.launch(fn, s, 1, 64, nbytes, C.c_uint64(out.value), C.c_int(nbytes)))
    got = np.zeros(1, dtype=np.int32)
    rt.ok(rt.copy_to_host(s, got.ctypes.data, out, 4))
    assert got[0] == 3
    # more than the device has is refused
    assert rt.function_set_max_dynamic_shared_bytes(fn, 1 << 20) != 0 or \
        rt.launch(fn, s, 1, 64, 1 << 20, C.c_uint64(out.value), C.c_int(1 << 20)) != 0
    rt.function_free(fn)
    rt.ok(rt.buffer_free(rt.ctx, out))
    rt.module_free(m)
    rt.stream_free(s)


def test_loading_what_is_not_a_code_object_fails_with_a_text(rt):
    m = C.c_void_p()
    rc = rt.module_load_file(rt.ctx, b"/nonexistent/berth.hsaco", C.byref(m))
    assert rc != 0 and rt.error_string(rc) and b"hipModuleLoad" in rt.last_error()
    assert rt.module_load_bytes(rt.ctx, None, 16, C.byref(m)) != 0          # refused before the driver sees it


def test_launches_on_two_streams_are_ordered_on_the_shared_workspace():
    """The library's split-K workspace serves one launch at a time per device.  Launches of
    different streams used to mix their partial sums silently; now a launch on another stream
    than the device's previous one waits for that stream's work so far.  Many alternating
    launches of two different split-K linears on two non-blocking streams, with no
    synchronisation by the caller in between, must each give the bits of a launch alone."""
    import torch
    from berth_amd import kernels as K
    from berth_amd import synth
    from berth_amd.kernels import Codebook, OutDtype
    from tests.gpu_util import DEV, dev
    rt = Runtime()
    streams = [rt.stream() for _ in range(2)]
    raw = [C.c_void_p(rt.stream_handle(s)) for s in streams]     # the hipStream_t behind each handle
    shapes = [(1, 4096, 8192, 4), (1, 2048, 768, 4)]            # streaming kernel; 1..8-row kernel with split-K
    work = []
    for i, (m, Kk, N, bits) in enumerate(shapes):
        tr, suh, svh = synth.linear(9900 + i, Kk, N, bits)
        x = synth.activations(9910 + i, m, Kk)
        d = {k: dev(v.view(np.uint16)) for k, v in dict(tr=tr, suh=suh, svh=svh, x=x).items()}
        c = torch.zeros((m, N), dtype=torch.float32, device=DEV)
        a_had = torch.zeros((m, Kk), dtype=torch.float16, device=DEV)
        work.append((m, Kk, N, bits, d, c, a_had))

    def launch(i, stream):
        m, Kk, N, bits, d, c, a_had = work[i]
        K.exl3_linear(d["x"].data_ptr(), d["tr"].data_ptr(), c.data_ptr(), d["suh"].data_ptr(), a_had.data_ptr(),
                      d["svh"].data_ptr(), m, Kk, N, bits, Codebook.MUL1, OutDtype.F32, stream)

    want = []
    for i in range(2):
        launch(i, None)
        torch.cuda.synchronize()
        want.append(work[i][5].cpu().numpy().view(np.uint32).copy())
    for rep in range(40):
        for i in range(2):
            work[i][5].fill_(-1.0)
        torch.cuda.synchronize()
        for burst in range(4):
            launch(0, raw[0])
            launch(1, raw[1])
        torch.cuda.synchronize()
        for i in range(2):
            assert np.array_equal(work[i][5].cpu().numpy().view(np.uint32), want[i]), (rep, i)
    for s in streams:
        rt.stream_free(s)
    rt.context_free(rt.ctx)
