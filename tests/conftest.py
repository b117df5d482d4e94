import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "se-ssd-ai-trt_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

# The first frame of the reference's data directory, kept as a fixture (tests/golden/README.md).
KITTI_FRAME0 = os.path.join(ROOT, "tests", "golden", "kitti_000000.bin")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def kitti_frame0():
    import numpy as np
    return np.fromfile(KITTI_FRAME0, np.float32).reshape(-1, 4)


def pytest_terminal_summary(terminalreporter):
    """What the feature comparisons of this session saw at worst (gpu_util.assert_features_close)."""
    import sys
    g = sys.modules.get("gpu_util")
    if g is None or not getattr(g, "WORST_SEEN", None):
        return
    terminalreporter.write_line("feature comparisons, worst over the session:")
    for (k, half), v in sorted(g.WORST_SEEN.items()):
        terminalreporter.write_line("  %-32s %s %.3g" % (k, "fp16" if half else "fp32", v))
