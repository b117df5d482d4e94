"""The voxelizer entry point that allocates nothing (sessd_voxelgen_enqueue_static: its scratch memory is a static
device array inside the library) against sessd_voxelgen_enqueue on a caller-owned workspace, through the C-ABI:
identical bits, on two calls in a row that share the array, the second with a smaller input."""
import numpy as np
import pytest
import torch

from gpu_util import dev, points_input, to_np
from sessd3d import api, backbone as B, ctypes_defs as D, frames as F

pytestmark = pytest.mark.gpu


def outputs(max_voxels, fill):
    vox = torch.full((max_voxels, 4), float(fill), dtype=torch.float32, device="cuda:0")
    coors = torch.full((max_voxels, 4), int(fill), dtype=torch.int32, device="cuda:0")
    num = torch.full((1,), int(fill), dtype=torch.int32, device="cuda:0")
    return [vox, coors, num]


def both_ways(vg, pts, max_points, max_voxels):
    """-> (outputs with a workspace, outputs on the static scratch, status of either), as host arrays"""
    ins = list(points_input(pts, max_points))
    a, b = outputs(max_voxels, 7), outputs(max_voxels, 9)
    vg.configure(ins, a)
    vg.enqueue(ins, a)                       # workspace: a torch tensor the wrapper owns
    torch.cuda.synchronize()
    st_a = vg.status()
    before = torch.cuda.memory_allocated()
    vg.enqueue_static(ins, b)                # no workspace, nothing allocated
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    st_b = vg.status_static()
    return [to_np(t) for t in a], [to_np(t) for t in b], (st_a, st_b)


def test_static_scratch_voxelizer_equals_the_workspace_one_on_two_calls_in_a_row():
    max_points, max_voxels = 80000, 60000                         # the reference's tensor shapes (params.h:19-20)
    vg = api.VoxelGenerator(max_voxels=max_voxels)
    for npts, seed in ((60000, 3), (9000, 4), (0, 0)):            # the later calls see the earlier ones' leftovers
        pts = F.lidar_frame(npts, seed) if npts else np.zeros((0, 4), np.float32)
        a, b, (st_a, st_b) = both_ways(vg, pts, max_points, max_voxels)
        assert st_a == st_b == 0
        assert a[2][0] == b[2][0] and (npts == 0 or a[2][0] > 1000)
        assert np.array_equal(a[1], b[1]), "coordinates differ (%d points)" % npts
        assert np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32)), "voxel means differ (%d points)" % npts


def test_static_scratch_voxelizer_raises_the_same_flags_and_handles_a_second_handle():
    """A second handle with a binding voxel cap shares the array with the first: overflow flag, dropped cells and
    every output row as with a workspace."""
    pts = F.lidar_frame(20000, 6)
    small = api.VoxelGenerator(max_voxels=3000)
    a, b, (st_a, st_b) = both_ways(small, pts, 20000, 3000)
    assert st_a == st_b == D.SESSD_STATUS_VOXEL_OVERFLOW and a[2][0] == b[2][0] == 3000
    assert np.array_equal(a[1], b[1]) and np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32))
    big = api.VoxelGenerator(max_voxels=20000)
    a, b, (st_a, st_b) = both_ways(big, pts[:5000], 20000, 20000)
    assert st_a == st_b == 0
    assert np.array_equal(a[1], b[1]) and np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32))


def test_static_scratch_voxelizer_rejects_what_does_not_fit():
    vg = api.VoxelGenerator(max_voxels=60000)
    pts = F.lidar_frame(1000, 1)
    ins = list(points_input(pts, 150000))                         # 14.7 MB of scratch: beyond the 8 MiB array
    outs = outputs(60000, 5)
    vg.configure(ins, outs)
    with pytest.raises(api.SessdError, match="static buffer holds"):
        vg.enqueue_static(ins, outs)
    torch.cuda.synchronize()
    assert int(to_np(outs[2])[0]) == 5                            # nothing was launched
