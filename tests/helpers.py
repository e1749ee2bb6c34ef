"""Shared helpers for the parity tests."""
import numpy as np
import torch

# tolerances of the parity contract: bf16 outputs and fp32 statistics
O_ATOL = 2e-2
O_RTOL = 2e-2
STAT_RTOL = 1e-3


def f32(t):
    return t.detach().float().cpu().numpy()


def assert_close_o(got, want, what=""):
    got = np.asarray(got, np.float32)
    want = np.asarray(want, np.float32)
    assert np.isfinite(got).all(), "%s: non-finite output" % what
    err = np.abs(got - want)
    lim = O_ATOL + O_RTOL * np.abs(want)
    bad = err > lim
    assert not bad.any(), "%s: %d of %d outside tolerance, max err %.4g" % (what, bad.sum(), bad.size, err.max())


def assert_close_stat(got, want, what="", rtol=STAT_RTOL, atol=1e-5):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    same_inf = np.isinf(want) & (got == want)
    err = np.abs(got - want)
    lim = atol + rtol * np.abs(want)
    bad = (err > lim) & ~same_inf
    bad |= np.isnan(got)
    assert not bad.any(), "%s: %d of %d outside tolerance, max err %.4g" % (what, bad.sum(), bad.size, np.nanmax(np.where(same_inf, 0, err)))


def to_dev(dev, *ts):
    return tuple(t.to(dev).contiguous() for t in ts)
