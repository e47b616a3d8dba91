"""Helpers shared by the parity tests."""
import numpy as np
import torch

# north-star tolerances
FP32_RTOL, FP32_ATOL = 1e-5, 1e-6
FP16_RTOL, FP16_ATOL = 2e-2, 1e-2


def rng(seed):
    return np.random.default_rng(seed)


def dev(x, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(x))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def host(t):
    return t.detach().float().cpu().numpy() if t.dtype == torch.float16 else t.detach().cpu().numpy()


def tol(dtype):
    return (FP16_RTOL, FP16_ATOL) if dtype in (torch.float16, np.float16) else (FP32_RTOL, FP32_ATOL)


def assert_close(got, want, dtype, what="", rtol=None, atol=None):
    r, a = tol(dtype)
    rtol = r if rtol is None else rtol
    atol = a if atol is None else atol
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, "%s: shape %s vs %s" % (what, got.shape, want.shape)
    err = np.abs(got - want)
    bound = atol + rtol * np.abs(want)
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        a_here = float(np.broadcast_to(np.asarray(atol, dtype=np.float64), err.shape)[i])   # atol may be per element
        raise AssertionError("%s: %d / %d elements out of tolerance (rtol=%g atol=%g); worst at %s: got %r want %r"
                             % (what, bad.sum(), bad.size, rtol, a_here, i, got[i], want[i]))
