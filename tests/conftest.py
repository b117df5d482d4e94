import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "se-ssd-ai-trt_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

# Real frames the reference ships; only present in the authoring container.  Tests that read them
# are CPU tests and skip when the directory is absent.
KITTI_DIR = "/root/reference/data/kitti_training_velodyne_reduced"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def kitti_frame0():
    import numpy as np
    path = os.path.join(KITTI_DIR, "000000.bin")
    if not os.path.exists(path):
        pytest.skip("KITTI fixture frames not present")
    return np.fromfile(path, np.float32).reshape(-1, 4)
