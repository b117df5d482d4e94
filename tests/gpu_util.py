"""Helpers for the GPU parity tests: device upload, canonical comparisons, tolerances."""
import numpy as np
import torch

import oracle_lib as O

DEV = "cuda:0"

# FP32 features: |gpu - oracle| <= 1e-4 * max(|oracle|, floor), FP16: 1e-2.  The floor (1 % of the
# tensor's largest magnitude) keeps elements that are tiny through cancellation from being judged by a
# relative error against ~0.
RTOL_FP32 = 1e-4
RTOL_FP16 = 1e-2


def dev(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def points_input(pts, max_points):
    """-> points tensor [max_points,F] (zero padded, as the reference's loader does) and size tensor."""
    buf = np.zeros((max_points, pts.shape[1]), np.float32)
    n = min(len(pts), max_points)
    buf[:n] = pts[:n]
    return dev(buf), dev(np.array([len(pts)], np.int32))


def assert_features_close(got, want, rtol, what=""):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if want.size == 0:
        return
    floor = 1e-2 * float(np.abs(want).max())
    bound = rtol * np.maximum(np.abs(want), floor)
    err = np.abs(got - want)
    bad = err > bound
    assert not bad.any(), "%s: %d of %d elements off, worst %.3g (bound %.3g) at %s" % (
        what, int(bad.sum()), bad.size, float((err / np.maximum(bound, 1e-300)).max()), rtol,
        np.unravel_index(np.argmax(err / np.maximum(bound, 1e-300)), err.shape))


def canonical(coors, n, *arrays):
    return O.sort_by_zyx(coors, n, *arrays)


def to_np(t):
    return t.detach().cpu().numpy()
