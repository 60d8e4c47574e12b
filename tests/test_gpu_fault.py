"""Failure handling of the split-K tile finisher of the MFMA kernels, forced from the host:
a tile's "partial sums written" counter is pre-set past the number of sharers, so the
finisher's wait can never complete.  It has to give up after its bounded number of polls,
zero the tile's counters, leave the tile unwritten and exit normally; the next call that
would launch an MFMA kernel reports it and launches nothing; the call after that runs as if
nothing had happened.  Every kernel in this test exits by itself."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

from berth_amd import kernels as K
from berth_amd import synth
from berth_amd.kernels import Codebook, LaunchError, OutDtype
from oracle import oracle as O
from tests.gpu_util import DEV, close, dev, knobs
from tests.test_gpu_runtime import Runtime

pytestmark = pytest.mark.gpu

WRITTEN_BASE = 32768        # second half of the counter table: "partial sums written" per tile


def _launch(d, c, a_had, w, rows, Kk, N):
    K.prefill_lin.exl3_linear(d["x"].data_ptr(), d["tr"].data_ptr(), c.data_ptr(), d["suh"].data_ptr(), a_had.data_ptr(),
                              d["svh"].data_ptr(), w, rows, Kk, N, 4, Codebook.MUL1, OutDtype.F32)
    launch = K.prefill_lin.last_launch()
    torch.cuda.synchronize()
    return launch


def test_finisher_gives_up_reports_and_recovers():
    rows, Kk, N = 16, 4096, 256                     # one 32-row tile shared by 16 workgroups
    tr, suh, svh = synth.linear(31, Kk, N, 4)
    x = synth.activations(32, rows, Kk)
    d = {k: dev(v.view(np.uint16)) for k, v in dict(tr=tr, suh=suh, svh=svh, x=x).items()}
    a_had = torch.zeros((rows, Kk), dtype=torch.float16, device=DEV)
    want, _ = O.linear(x, tr, suh, svh, Kk, N, 4, 2, out_fp32=True)

    c = torch.full((rows, N), 777.0, dtype=torch.float32, device=DEV)
    launch = _launch(d, c, a_had, None, rows, Kk, N)
    assert "split_k=16" in launch, launch
    assert close(c.cpu().numpy(), want)[0] == 0

    counters, slots = C.c_void_p(), C.c_int()
    assert K.load().berth_kernels_workspace(None, None, C.byref(counters), C.byref(slots)) == 0
    assert slots.value == 2 * WRITTEN_BASE
    rt = Runtime()
    bogus = np.array([1000], dtype=np.uint32)
    rt.ok(rt.copy_from_host(None, counters.value + 4 * WRITTEN_BASE, bogus.ctypes.data, 4))

    with knobs(BERTH_SPIN_LIMIT=300):
        c.fill_(777.0)
        launch = _launch(d, c, a_had, None, rows, Kk, N)     # the launch itself is accepted and every kernel exits
        assert "exl3_gemm_kernel" in launch
        assert (c.cpu().numpy() == 777.0).all()              # the tile was left unwritten
        with pytest.raises(LaunchError, match="gave up waiting for the split-K partial sums of tile 0"):
            _launch(d, c, a_had, None, rows, Kk, N)
        assert K.prefill_lin.last_launch() == ""
    both = np.zeros(2, dtype=np.uint32)
    rt.ok(rt.copy_to_host(None, both[:1].ctypes.data, counters.value, 4))
    rt.ok(rt.copy_to_host(None, both[1:].ctypes.data, counters.value + 4 * WRITTEN_BASE, 4))
    assert (both == 0).all()                                 # the finisher zeroed the tile's counters
    launch = _launch(d, c, a_had, None, rows, Kk, N)         # reported once; now everything is back to normal
    assert close(c.cpu().numpy(), want)[0] == 0, launch
    rt.context_free(rt.ctx)
