"""The doubled-width backbone in FP32: the 64->128 and 128->128 FP32 kernels on 100 000-row tensors.  Kept in a
file of its own, collected after the other GPU tests, with a time limit: it is the heaviest configuration the
library is asked to run and no benchmark configuration covers it."""
import numpy as np
import pytest

from gpu_util import assert_end_to_end_close, to_np
from sessd3d import backbone as B, frames as F
from test_gpu_pipeline import run_pipeline

pytestmark = pytest.mark.gpu


@pytest.mark.timeout(120, method="thread")
def test_wide_fp32_backbone_matrix_cores_against_valu_kernels():
    """Doubled channel widths in FP32 (the 64->128 and 128->128 FP32 kernels, 100 000-row tensors of up to 51 MB)
    at 60 000 points: too heavy for the scalar oracle, so the matrix-core path is checked against the
    shape-agnostic VALU kernels of the same library: status and site counts exactly, the dense tensors within
    the whole-frame bound."""
    pts = F.lidar_frame(60000, 8)
    layers = B.reference_layers(width_mult=2)
    W = B.random_weights(layers, seed=6, w_std=0.03)
    kw = dict(share_rulebooks=True, skip_pad_rows=True, voxel_cap=40000)
    fast, dense, _ = run_pipeline(pts, layers, W, 60000, 100000, overlap_streams=True, use_graph=True, **kw)
    slow, sdense, _ = run_pipeline(pts, layers, W, 60000, 100000, force_valu=True, **kw)
    assert fast.status() == slow.status()
    counts = [fast.layer_count(l) for l in range(-1, len(layers))]
    assert counts == [slow.layer_count(l) for l in range(-1, len(layers))] and counts[0] == 40000
    a, b = to_np(dense), to_np(sdense)
    assert np.isfinite(a).all() and a.any()
    assert_end_to_end_close(a, b, False, "wide FP32 backbone, MFMA vs VALU")
