"""Seeded synthetic inputs: LiDAR frames with scan-line structure and random active-voxel sets.

There is no dataset on the benchmark machine, so frames are simulated: a 64-ring spinning sensor
(elevations -24.8 .. +2 degrees) looks at a ground plane at z = -1.7 m and at vertical obstacle
slabs whose distance is piecewise constant in azimuth (exponentially distributed, mean 15 m).
This keeps what matters for the sparse backbone -- points that are neighbours in the scan fall in
neighbouring voxels -- so the number of active sites shrinks through the strided layers the way it
does on real KITTI frames instead of growing as it does for spatially uncorrelated points.
"""
import numpy as np

from . import backbone as B

N_RINGS = 64
ELEV_MIN_DEG = -24.8
ELEV_MAX_DEG = 2.0
GROUND_Z = -1.7


def lidar_frame(n_points: int, seed: int = 0, full_circle: bool = False, ground_fraction: float = 0.35,
                mean_range: float = 15.0, near_thinning: float = 1.0, pc_range=B.POINT_CLOUD_RANGE) -> np.ndarray:
    """-> float32 [n_points, 4] (x, y, z, intensity), every point inside pc_range, scan order
    (ring by ring from the top ring, azimuth ascending inside a ring)."""
    rng = np.random.default_rng(seed)
    xmin, ymin, zmin, xmax, ymax, zmax = pc_range
    elev = np.deg2rad(ELEV_MIN_DEG + (ELEV_MAX_DEG - ELEV_MIN_DEG) * np.arange(N_RINGS) / (N_RINGS - 1))[::-1]
    half_fov = np.pi if full_circle else np.deg2rad(50.0)
    oversample = 2.2
    for _attempt in range(8):
        steps = int(np.ceil(oversample * n_points / N_RINGS)) + 8
        az = np.linspace(-half_fov, half_fov, steps, endpoint=False)
        # obstacle slabs: piecewise-constant distance / height over azimuth, shared by all rings
        n_seg = max(8, int(steps / 12))
        edges = np.sort(rng.choice(np.arange(1, steps), size=n_seg - 1, replace=False))
        seg_of_step = np.searchsorted(edges, np.arange(steps), side="right")
        seg_dist = np.minimum(2.5 + rng.exponential(mean_range, n_seg), 90.0)
        seg_slope = rng.normal(0.0, 0.6, n_seg)           # slab not exactly facing the sensor
        seg_top = GROUND_Z + rng.uniform(0.3, 3.2, n_seg)   # slab height above ground
        seg_present = rng.uniform(size=n_seg) < 0.8
        pos_in_seg = np.arange(steps) - np.concatenate([[0], edges])[seg_of_step]
        d_obst = seg_dist[seg_of_step] * (1.0 + seg_slope[seg_of_step] * pos_in_seg * (2 * half_fov / steps))
        d_obst = np.where(seg_present[seg_of_step], d_obst, np.inf)
        top = seg_top[seg_of_step]

        e = elev[:, None]                                   # [R,1]
        d_o = d_obst[None, :]                               # horizontal distance of the slab
        z_at_o = d_o * np.tan(e)                            # height where the ray meets the slab
        with np.errstate(divide="ignore", invalid="ignore"):
            d_ground = np.where(e < 0, GROUND_Z / np.tan(e), np.inf)  # horizontal distance to ground hit
        hit_obst = (z_at_o <= top[None, :]) & (z_at_o >= GROUND_Z) & np.isfinite(d_o)
        use_obst = hit_obst & (d_o <= d_ground)
        d = np.where(use_obst, d_o, d_ground) * np.ones((N_RINGS, steps))
        is_ground = ~use_obst & np.isfinite(d)
        valid = np.isfinite(d)
        noise_r = rng.normal(0.0, 0.08, d.shape)
        d = d + noise_r
        x = d * np.cos(az)[None, :]
        with np.errstate(invalid='ignore'):
            y = d * np.sin(az)[None, :]
        z = np.where(is_ground, GROUND_Z + rng.normal(0.0, 0.05, d.shape), d * np.tan(e) + rng.normal(0.0, 0.01, d.shape))
        inside = valid & (x >= xmin) & (x < xmax - 1e-3) & (y >= ymin) & (y < ymax - 1e-3) & \
            (z >= zmin) & (z < zmax - 1e-3)
        # thin the ground so that it carries ground_fraction of the returns
        g_in = inside & is_ground
        o_in = inside & ~is_ground
        n_o, n_g = int(o_in.sum()), int(g_in.sum())
        want_g = int(round(ground_fraction * n_points))
        want_o = n_points - want_g
        if n_o >= want_o and n_g >= want_g:
            keep = np.zeros(d.shape, bool)
            gi = np.flatnonzero(g_in.ravel())
            oi = np.flatnonzero(o_in.ravel())
            # returns are thinned with probability proportional to distance: the near field, where
            # many rays fall into one 5 cm voxel, is what a camera-FOV crop of a real scan lacks
            dflat = np.nan_to_num(d.ravel(), posinf=0.0)
            pg = np.clip(dflat[gi], 1.0, 40.0) ** near_thinning
            po = np.clip(dflat[oi], 1.0, 40.0) ** near_thinning
            keep.ravel()[rng.choice(gi, want_g, replace=False, p=pg / pg.sum())] = True
            keep.ravel()[rng.choice(oi, want_o, replace=False, p=po / po.sum())] = True
            inten = rng.uniform(0.0, 1.0, d.shape)
            pts = np.stack([x, y, z, inten], axis=-1)[keep]   # row-major: ring by ring, azimuth ascending
            return np.ascontiguousarray(pts, np.float32)
        oversample *= 1.6
    raise RuntimeError("lidar_frame: could not reach %d in-range points" % n_points)


def lidar_frames(n_points: int, seeds, threads: int = 8, **kw):
    """lidar_frame(n_points, seed, **kw) for every seed, in order, generated by a pool of threads a few frames
    ahead of the consumer (numpy releases the interpreter lock in the array operations that dominate: 8 threads make
    a 150 000-point frame every 0.1 s instead of every 0.4 s).  A generator: frames are not kept."""
    import collections
    import concurrent.futures as cf
    seeds = list(seeds)
    ahead = max(1, 2 * threads)
    with cf.ThreadPoolExecutor(max_workers=max(1, threads)) as ex:
        pending = collections.deque()
        it = iter(seeds)
        for seed in it:
            pending.append(ex.submit(lidar_frame, n_points, seed, **kw))
            if len(pending) >= ahead:
                break
        while pending:
            frame = pending.popleft().result()
            nxt = next(it, None)
            if nxt is not None:
                pending.append(ex.submit(lidar_frame, n_points, nxt, **kw))
            yield frame


def random_active_voxels(n: int, grid_zyx, seed: int = 0) -> np.ndarray:
    """n unique cells drawn uniformly without replacement from a (z,y,x) grid.
    -> int32 [n,4] rows (0,z,y,x) in draw order."""
    rng = np.random.default_rng(seed)
    Z, Y, X = grid_zyx
    lin = rng.choice(Z * Y * X, size=n, replace=False)
    z, rem = np.divmod(lin, Y * X)
    y, x = np.divmod(rem, X)
    return np.stack([np.zeros_like(z), z, y, x], axis=1).astype(np.int32)


def clustered_active_voxels(n: int, grid_zyx, seed: int = 0, n_blobs: int = 40, sigma=(1.0, 3.0, 3.0)) -> np.ndarray:
    """n unique cells concentrated around random centres: neighbour-rich input for rulebook tests."""
    rng = np.random.default_rng(seed)
    Z, Y, X = grid_zyx
    centres = np.stack([rng.uniform(0, Z, n_blobs), rng.uniform(0, Y, n_blobs), rng.uniform(0, X, n_blobs)], 1)
    got = {}
    while len(got) < n:
        c = centres[rng.integers(0, n_blobs, 4 * n)]
        p = np.rint(c + rng.normal(size=c.shape) * np.asarray(sigma)).astype(np.int64)
        ok = (p[:, 0] >= 0) & (p[:, 0] < Z) & (p[:, 1] >= 0) & (p[:, 1] < Y) & (p[:, 2] >= 0) & (p[:, 2] < X)
        for z, y, x in p[ok]:
            if len(got) >= n:
                break
            got.setdefault((int(z), int(y), int(x)), None)
    k = np.array(list(got.keys()), np.int32)
    return np.concatenate([np.zeros((n, 1), np.int32), k], axis=1)
