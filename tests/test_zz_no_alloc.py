"""berth_exl3_linear_noalloc (the entry point that allocates nothing: split-K scratch in a
fixed array inside the library) against berth_exl3_linear on the same inputs, through the C
ABI: two calls in a row, the second on a smaller input, so that what the first call left in
the shared scratch is in the way if anything is."""
import numpy as np
import pytest
import torch

from berth_amd import kernels as K
from berth_amd import synth
from berth_amd.kernels import Codebook, OutDtype
from oracle import oracle as O
from tests.gpu_util import DEV, close, dev, host_u16, knobs

pytestmark = pytest.mark.gpu


def _both(m, Kk, N, bits, seed, out_fp32=True):
    tr, suh, svh = synth.linear(seed, Kk, N, bits)
    x = synth.activations(seed + 1, m, Kk)
    d = {k: dev(v.view(np.uint16)) for k, v in dict(tr=tr, suh=suh, svh=svh, x=x).items()}
    res = []
    for fn in (K.exl3_linear, K.exl3_linear_noalloc):
        c = torch.full((m, N), 7.0, dtype=torch.float32 if out_fp32 else torch.float16, device=DEV)
        a_had = torch.zeros((m, Kk), dtype=torch.float16, device=DEV)
        fn(d["x"].data_ptr(), d["tr"].data_ptr(), c.data_ptr(), d["suh"].data_ptr(), a_had.data_ptr(),
           d["svh"].data_ptr(), m, Kk, N, bits, Codebook.MUL1, OutDtype.F32 if out_fp32 else OutDtype.F16)
        launch = K.last_launch()
        torch.cuda.synchronize()
        res.append((c.cpu().numpy().copy() if out_fp32 else host_u16(c).copy(), host_u16(a_had).copy(), launch))
    return res, (x, tr, suh, svh)


@pytest.mark.parametrize("first,second", [((1, 4096, 1024, 4), (1, 512, 256, 4)),
                                          ((1, 5120, 17408, 4), (1, 2048, 768, 3)),
                                          ((5, 2048, 512, 4), (2, 256, 128, 5))])
def test_no_alloc_matches_the_allocating_entry_point_twice_in_a_row(first, second):
    for i, (m, Kk, N, bits) in enumerate((first, second)):
        (ref, ref_had, ref_launch), (got, got_had, got_launch) = _both(m, Kk, N, bits, 8100 + 17 * i + Kk)[0]
        assert "split_k=1 " not in got_launch or Kk <= 512, got_launch      # the scratch is really in use
        # same kernels on the same split: the same bits
        assert ref_launch.split(" grid=")[0] == got_launch.split(" grid=")[0], (ref_launch, got_launch)
        assert np.array_equal(got_had, ref_had), got_launch
        assert np.array_equal(got.view(np.uint32) if got.dtype == np.float32 else got,
                              ref.view(np.uint32) if ref.dtype == np.float32 else ref), (ref_launch, got_launch)


def test_no_alloc_output_is_within_the_bar_of_the_oracle():
    (_, (got, got_had, launch)), (x, tr, suh, svh) = _both(1, 2048, 768, 4, 8200)
    want, want_had = O.linear(x, tr, suh, svh, 2048, 768, 4, 2, out_fp32=True)
    assert np.array_equal(got_had.reshape(-1), want_had.view(np.uint16).reshape(-1))
    assert close(got, want)[0] == 0, launch


def test_no_alloc_refuses_what_does_not_fit():
    bad = 0xdead000
    with pytest.raises(K.LaunchError, match="at most 8 rows"):
        K.exl3_linear_noalloc(bad, bad, bad, bad, bad, bad, 9, 256, 256, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(K.LaunchError, match="null device pointer"):
        K.exl3_linear_noalloc(None, bad, bad, bad, bad, bad, 1, 256, 256, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(K.LaunchError, match="size_n must be a multiple of 128"):
        K.exl3_linear_noalloc(bad, bad, bad, bad, bad, bad, 1, 256, 200, 4, Codebook.MUL1, OutDtype.F16)
    with pytest.raises(K.LaunchError, match="exceeds the scratch's counter table"):
        K.exl3_linear_noalloc(bad, bad, bad, bad, bad, bad, 1, 128, 128 * 65537, 1, Codebook.MUL1, OutDtype.F16)
    # With the default split (about six workgroups per compute unit) the partial sums of a launch
    # stay under 6.3 MB on 256 compute units; a finer split of eight rows of a wide, deep weight
    # exceeds the 8 MiB and is refused before anything is launched (the pointers are never used).
    with knobs(BERTH_GEMV_WG_PER_CU=16):
        with pytest.raises(K.LaunchError, match="bytes of split-K scratch"):
            K.exl3_linear_noalloc(bad, bad, bad, bad, bad, bad, 8, 16384, 16384, 2, Codebook.MUL1, OutDtype.F32)
    assert K.last_launch() == ""


_CAPTURE_SCRIPT = r"""
import sys
import numpy as np
import torch
sys.path.insert(0, sys.argv[1])
from berth_amd import kernels as K
from berth_amd import synth
from berth_amd.kernels import Codebook, OutDtype

DEV = "cuda:0"
def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).to(DEV)

cases = []
for m, Kk, N, bits, seed in ((1, 4096, 8192, 4, 8300), (1, 512, 256, 4, 8301), (3, 1024, 384, 3, 8302)):
    tr, suh, svh = synth.linear(seed, Kk, N, bits)
    x = synth.activations(seed + 1, m, Kk)
    d = {k: dev(v.view(np.uint16)) for k, v in dict(tr=tr, suh=suh, svh=svh, x=x).items()}
    c = torch.zeros((m, N), dtype=torch.float32, device=DEV)
    a_had = torch.zeros((m, Kk), dtype=torch.float16, device=DEV)
    cases.append((m, Kk, N, bits, d, c, a_had))

def run(fn):
    texts = []
    for m, Kk, N, bits, d, c, a_had in cases:
        fn(d["x"].data_ptr(), d["tr"].data_ptr(), c.data_ptr(), d["suh"].data_ptr(), a_had.data_ptr(),
           d["svh"].data_ptr(), m, Kk, N, bits, Codebook.MUL1, OutDtype.F32, torch.cuda.current_stream().cuda_stream)
        texts.append(K.last_launch())
    return texts

def outputs():
    torch.cuda.synchronize()
    return [c.cpu().numpy().view(np.uint32).copy() for *_, c, _ in cases]

def clear():
    for *_, c, _ in cases:
        c.fill_(-3.0)

# the very first calls of the entry point in this process are the recorded ones
graph = torch.cuda.CUDAGraph()
side = torch.cuda.Stream(device=DEV)
with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):
        texts = run(K.exl3_linear_noalloc)
torch.cuda.synchronize()
assert "exl3_gemv_stream_kernel" in texts[0] and "exl3_gemv_kernel" in texts[1], texts
clear()
run(K.exl3_linear)                      # eager, the allocating entry point: the reference bits
want = outputs()
for replay in range(3):
    clear()
    graph.replay()
    got = outputs()
    for g, w, t in zip(got, want, texts):
        assert np.array_equal(g, w), (replay, t)
    run(K.exl3_linear)                  # eager work of the same library between the replays
    torch.cuda.synchronize()
clear()
run(K.exl3_linear_noalloc)              # and eagerly after the replays
for g, w in zip(outputs(), want):
    assert np.array_equal(g, w)
print("capture ok")
"""


def test_no_alloc_first_call_inside_a_stream_capture_replays_bit_exact(tmp_path):
    """The entry point's stated use: its first calls in a process are recorded into a HIP graph
    (nothing may allocate, synchronise or clear memory there), the graph is replayed three
    times with eager launches of the library in between, and every replay gives the bits of
    berth_exl3_linear.  A process of its own, so that the calls really are the first."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = tmp_path / "capture.py"
    script.write_text(_CAPTURE_SCRIPT)
    r = subprocess.run([sys.executable, str(script), root], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "capture ok" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
