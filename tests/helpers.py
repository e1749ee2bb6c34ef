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
    assert np.isfinite(want).all(), "%s: non-finite expected value (the checker itself is broken)" % what
    assert np.isfinite(got).all(), "%s: non-finite output" % what
    err = np.abs(got - want)
    lim = O_ATOL + O_RTOL * np.abs(want)
    bad = ~(err <= lim)   # a NaN on either side fails
    assert not bad.any(), "%s: %d of %d outside tolerance, max err %.4g" % (what, bad.sum(), bad.size, err.max())


def assert_close_stat(got, want, what="", rtol=STAT_RTOL, atol=1e-5):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert not np.isnan(want).any(), "%s: NaN in the expected value (the checker itself is broken)" % what
    # infinities must agree in place and sign; everything else is compared where both are finite
    inf_w, inf_g = np.isinf(want), np.isinf(got)
    same_inf = inf_w & inf_g & (got == want)
    fin = np.isfinite(want) & np.isfinite(got)
    err = np.zeros(want.shape, np.float64)
    err[fin] = np.abs(got[fin] - want[fin])
    lim = atol + rtol * np.abs(np.where(fin, want, 0.0))
    bad = ~(err <= lim) | ~(fin | same_inf)
    assert not bad.any(), "%s: %d of %d outside tolerance, max err %.4g" % (what, bad.sum(), bad.size, err.max())


def to_dev(dev, *ts):
    return tuple(t.to(dev).contiguous() for t in ts)
