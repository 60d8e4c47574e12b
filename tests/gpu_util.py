"""Helpers shared by the GPU parity tests."""
import contextlib
import os

import numpy as np
import torch

DEV = "cuda:0"


def dev(a: np.ndarray) -> torch.Tensor:
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        a = a.view(np.int16)
    return torch.from_numpy(a).to(DEV)


def host_u16(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def host_f16(t: torch.Tensor) -> np.ndarray:
    return host_u16(t).view(np.float16)


def close(got, want, rtol=2e-3, atol=1e-3):
    """|got - want| <= atol + rtol*|want|, the tolerance the linear outputs are held to."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(got - want)
    lim = atol + rtol * np.abs(want)
    bad = err > lim
    return int(bad.sum()), float((err / lim).max())


@contextlib.contextmanager
def knobs(**kv):
    """Sets BERTH_* environment knobs for the body and makes the library read them (it reads
    the environment once per process, then only when told to)."""
    from berth_amd import kernels as K
    old = {k: os.environ.get(k) for k in kv}
    for k, v in kv.items():
        os.environ[k] = str(v)
    K.reload_env()
    try:
        yield
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
        K.reload_env()
