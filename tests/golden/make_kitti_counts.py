"""Recompute tests/golden/kitti_000000_counts.json with numpy only (no oracle, no reference code).

Reads frame 000000 of the reference's data directory (kept beside this script as kitti_000000.bin), voxelises it in float32, and walks the four
strided stages with set arithmetic: an output cell o of a sparse layer is active iff some active
input cell c satisfies c = o*s - p + k for an offset 0 <= k < ksize on every axis; the pairs of a
layer are all (input, output, offset) triples that satisfy it.
"""
import json
import os
import sys

import numpy as np

SRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kitti_000000.bin")


def voxelize(p):
    lo = np.array([0.0, -40.0, -3.0], np.float32)
    hi = np.array([70.4, 40.0, 1.0], np.float32)
    vs = np.array([0.05, 0.05, 0.1], np.float32)
    ok = np.all((p[:, :3] >= lo) & (p[:, :3] < hi), axis=1)
    idx = np.floor((p[ok, :3] - lo) / vs).astype(np.int64)[:, ::-1]
    idx = idx[np.all((idx >= 0) & (idx < np.array([40, 1600, 1408])), axis=1)]
    lin = idx @ np.array([1600 * 1408, 1408, 1])
    _, first, cnt = np.unique(lin, return_index=True, return_counts=True)
    return idx[np.sort(first)], int(min(cnt.max(), 5))


def subm_pairs(cells):
    s = set(map(tuple, cells))
    n = 0
    for dz in (-1, 0, 1):
        for dy in (-1, 0, 1):
            for dx in (-1, 0, 1):
                n += sum((z + dz, y + dy, x + dx) in s for z, y, x in s)
    return n


def sparse(cells, k, s, p, out_shape):
    outs, pairs = set(), 0
    for c in map(tuple, cells):
        for kz in range(k[0]):
            for ky in range(k[1]):
                for kx in range(k[2]):
                    t = [c[a] + p[a] - (kz, ky, kx)[a] for a in range(3)]
                    if all(t[a] % s[a] == 0 and 0 <= t[a] // s[a] < out_shape[a] for a in range(3)):
                        outs.add(tuple(t[a] // s[a] for a in range(3)))
                        pairs += 1
    return np.array(sorted(outs)), pairs


def main():
    p = np.fromfile(SRC, np.float32).reshape(-1, 4)
    cells, maxpts = voxelize(p)
    sites, pairs = [len(cells)], []
    plan = [(2, None), ((3, 3, 3), (2, 2, 2), (1, 1, 1), (21, 800, 704)), (2, None),
            ((3, 3, 3), (2, 2, 2), (1, 1, 1), (11, 400, 352)), (3, None),
            ((3, 3, 3), (2, 2, 2), (0, 1, 1), (5, 200, 176)), (3, None),
            ((3, 1, 1), (2, 1, 1), (0, 0, 0), (2, 200, 176))]
    for step in plan:
        if step[1] is None:
            pairs += [subm_pairs(cells)] * step[0]
        else:
            cells, n = sparse(cells, *step)
            pairs.append(n)
            sites.append(len(cells))
    out = dict(points=len(p), voxels=sites[0], max_points_in_voxel=maxpts,
               active_sites_after_stage=sites, pairs_per_layer=pairs)
    json.dump(out, sys.stdout, indent=2)


if __name__ == "__main__":
    main()
