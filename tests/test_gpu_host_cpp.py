"""The C++ host layer (berth_amd/csrc/host/engine.hpp: Gpu, DeviceBuffer, Exl3Linear,
RowScratch, MultiLinear, MlpLayer, MoeLayer over the two C ABIs) driven through its check
program on case files, results compared with the CPU oracle.  This is also the
functional test of the device-runtime library (contexts, streams, events,
buffers, copies)."""
import os
import subprocess

import numpy as np
import pytest

from berth_amd import synth
from oracle import oracle as O
from tests.gpu_util import close

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "berth_amd", "lib", "berth_host_check")


def _write_linear(d, name, lin):
    tr, suh, svh = lin
    tr.view(np.uint16).tofile(os.path.join(d, f"{name}.trellis.bin"))
    suh.view(np.uint16).tofile(os.path.join(d, f"{name}.suh.bin"))
    svh.view(np.uint16).tofile(os.path.join(d, f"{name}.svh.bin"))


def _run(kind, d):
    assert os.path.exists(EXE), "berth_host_check is not built (python -m berth_amd.build)"
    r = subprocess.run([EXE, kind, str(d)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    return r.stdout


@pytest.mark.parametrize("rows,fp32,use_rows", [(1, 1, 0), (1, 0, 0), (5, 0, 0), (40, 1, 0), (200, 0, 1), (16, 1, 1)])
def test_cpp_linear(tmp_path, rows, fp32, use_rows):
    Kk, N, bits = 256, 384, 4
    lin = synth.linear(4000 + rows, Kk, N, bits)
    x = synth.activations(4100 + rows, rows, Kk)
    _write_linear(tmp_path, "lin", lin)
    x.view(np.uint16).tofile(tmp_path / "x.bin")
    (tmp_path / "meta.txt").write_text(f"{Kk} {N} {rows} {fp32} {use_rows}\n")
    out = _run("linear", tmp_path)
    assert "linear ok" in out and "elapsed_ms=" in out
    y = np.fromfile(tmp_path / "y.bin", dtype=np.float32 if fp32 else np.float16).reshape(rows, N)
    want, _ = O.linear(x, *lin, Kk, N, bits, 2, out_fp32=bool(fp32))
    assert close(y, want.reshape(rows, N))[0] == 0


@pytest.mark.parametrize("rows,fp32", [(1, 0), (4, 1), (20, 0), (150, 1)])
def test_cpp_bundle(tmp_path, rows, fp32):
    """MultiLinear: three linears on one input as one sliced berth_ops_mgemm, every row-count
    route (one row, 2..8 rows from the device lists, more than 8 rows on the MFMA kernels)."""
    Kk, Ns, bits = 256, (768, 256, 512), 4
    lins = [synth.linear(4500 + rows + i, Kk, n, bits) for i, n in enumerate(Ns)]
    x = synth.activations(4600 + rows, rows, Kk)
    for i, lin in enumerate(lins):
        _write_linear(tmp_path, f"src{i}", lin)
    x.view(np.uint16).tofile(tmp_path / "x.bin")
    (tmp_path / "meta.txt").write_text(f"{Kk} {rows} {fp32} " + " ".join(str(n) for n in Ns) + "\n")
    out = _run("bundle", tmp_path)
    assert "bundle ok" in out and "slices=6 width=256" in out and "sliced x6" in out, out
    for i, lin in enumerate(lins):
        y = np.fromfile(tmp_path / f"y{i}.bin", dtype=np.float32 if fp32 else np.float16).reshape(rows, Ns[i])
        want, _ = O.linear(x, *lin, Kk, Ns[i], bits, 2, out_fp32=bool(fp32))
        assert close(y, want.reshape(rows, Ns[i]))[0] == 0, i


@pytest.mark.parametrize("rows", [1, 24])
def test_cpp_mlp(tmp_path, rows):
    H, I, bits = 256, 384, 3
    gate, up, down = synth.linear(5000, H, I, bits), synth.linear(5003, H, I, bits), synth.linear(5006, I, H, bits)
    x = (synth.activations(5100 + rows, rows, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    for name, lin in (("gate", gate), ("up", up), ("down", down)):
        _write_linear(tmp_path, name, lin)
    x.view(np.uint16).tofile(tmp_path / "x.bin")
    (tmp_path / "meta.txt").write_text(f"{H} {I} {rows}\n")
    assert "mlp ok" in _run("mlp", tmp_path)
    y = np.fromfile(tmp_path / "y.bin", dtype=np.float32).reshape(rows, H)
    g, _ = O.linear(x, *gate, H, I, bits, 2)
    u, _ = O.linear(x, *up, H, I, bits, 2)
    a = O.silu_mul(g, u).reshape(rows, I)
    want, _ = O.linear(a, *down, I, H, bits, 2, out_fp32=True)
    # gate/up round to fp16 on both sides from fp32 sums in different orders: whole-layer bound
    assert np.abs(y - want.reshape(rows, H)).max() <= 2e-3 * np.abs(want).max()


@pytest.mark.parametrize("T,shared", [(1, 0), (12, 1)])
def test_cpp_moe(tmp_path, T, shared):
    H, E, k, I, bits = 256, 6, 2, 128, 4
    experts = [(synth.linear(6000 + 10 * e, H, I, bits), synth.linear(6003 + 10 * e, H, I, bits),
                synth.linear(6006 + 10 * e, I, H, bits)) for e in range(E)]
    sh = (synth.linear(6900, H, I, bits), synth.linear(6903, H, I, bits), synth.linear(6906, I, H, bits))
    wr = synth.router_weight(6999, H, E)
    bias = synth.zipf_bias(6998, E)
    x = (synth.activations(6100 + T, T, H).astype(np.float32) / np.sqrt(H)).astype(np.float16)
    for e, trio in enumerate(experts):
        for name, lin in zip(("gate", "up", "down"), trio):
            _write_linear(tmp_path, f"e{e}.{name}", lin)
    for name, lin in zip(("gate", "up", "down"), sh):
        _write_linear(tmp_path, f"shared.{name}", lin)
    wr.view(np.uint16).tofile(tmp_path / "router.bin")
    bias.tofile(tmp_path / "bias.bin")
    x.view(np.uint16).tofile(tmp_path / "x.bin")
    (tmp_path / "meta.txt").write_text(f"{T} {H} {E} {k} {I} {shared} 1\n")
    assert "moe ok" in _run("moe", tmp_path)
    y = np.fromfile(tmp_path / "y.bin", dtype=np.float32).reshape(T, H)
    idx = np.fromfile(tmp_path / "idx.bin", dtype=np.int32).reshape(T, k)
    want, oi, _ = O.moe_layer(x, wr, experts, k, I, bits, 2, bias=bias, shared=sh if shared else None,
                              shared_I=I if shared else 0)
    assert np.array_equal(idx, oi)
    assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max()
