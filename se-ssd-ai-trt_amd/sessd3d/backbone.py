"""Static shapes of the SE-SSD SpMiddleFHD 3-D backbone and seeded random weights for it.

Layer list and shapes restate the reference's params.h:19-197 and the wiring at
se-ssd-ai-trt.cpp:1138-1252: ten SubM layers (middle_conv 0,3,9,12,18,21,24,30,33,36) and four
strided sparse layers (6,15,27,39), each followed by BatchNorm1d + ReLU.
"""
from dataclasses import dataclass, field
from typing import List, Tuple

import numpy as np

from . import ctypes_defs as D

# params.h:26-36
POINT_CLOUD_RANGE = (0.0, -40.0, -3.0, 70.4, 40.0, 1.0)  # xmin,ymin,zmin,xmax,ymax,zmax
VOXEL_SIZE = (0.05, 0.05, 0.1)
MAX_NUM_POINTS_PER_VOXEL = 5
VOXEL_FEATURE_NUM = 4
# params.h:19-20
MAX_VOXELS = 60000
MAX_POINTS = 80000
# params.h:194-197
DENSE_SIZE_XYZ = (176, 200, 2)
DENSE_CHANNEL = 64


@dataclass
class Layer:
    name: str
    type: int                       # D.SESSD_LAYER_*
    cin: int
    cout: int
    out_shape: Tuple[int, int, int]  # x,y,z
    ksize: Tuple[int, int, int] = (3, 3, 3)    # z,y,x
    stride: Tuple[int, int, int] = (1, 1, 1)
    padding: Tuple[int, int, int] = (1, 1, 1)

    @property
    def kvol(self):
        return self.ksize[0] * self.ksize[1] * self.ksize[2]


def reference_layers(width_mult: int = 1, subm_per_64_stage: int = 3) -> List[Layer]:
    """The reference's 14 conv layers (params.h:39-192).

    width_mult=2 doubles every channel width after the input (the stress configuration);
    subm_per_64_stage=2 gives the 12-layer variant some descriptions of the network use.
    """
    S, P = D.SESSD_LAYER_SUBM, D.SESSD_LAYER_SPARSE
    w = width_mult
    g1, g2, g3, g4, g5 = (1408, 1600, 41), (704, 800, 21), (352, 400, 11), (176, 200, 5), (176, 200, 2)
    L = [
        Layer("subm0", S, 4, 16 * w, g1),
        Layer("subm3", S, 16 * w, 16 * w, g1),
        Layer("sparse6", P, 16 * w, 32 * w, g2, (3, 3, 3), (2, 2, 2), (1, 1, 1)),
        Layer("subm9", S, 32 * w, 32 * w, g2),
        Layer("subm12", S, 32 * w, 32 * w, g2),
        Layer("sparse15", P, 32 * w, 64 * w, g3, (3, 3, 3), (2, 2, 2), (1, 1, 1)),
    ]
    L += [Layer("subm%d" % i, S, 64 * w, 64 * w, g3) for i in (18, 21, 24)[:subm_per_64_stage]]
    L += [Layer("sparse27", P, 64 * w, 64 * w, g4, (3, 3, 3), (2, 2, 2), (0, 1, 1))]
    L += [Layer("subm%d" % i, S, 64 * w, 64 * w, g4) for i in (30, 33, 36)[:subm_per_64_stage]]
    L += [Layer("sparse39", P, 64 * w, 64 * w, g5, (3, 1, 1), (2, 1, 1), (0, 0, 0))]
    return L


def conv_index(layer: Layer) -> int:
    """Index of the layer inside the reference's `backbone.middle_conv` Sequential (its name's number:
    se-ssd-ai-trt.cpp:1147-1249); the layer's BatchNorm is index + 1."""
    return int("".join(ch for ch in layer.name if ch.isdigit()))


def conv_out_size(n, k, s, p):
    """spconv's output extent for one axis: (n + 2p - k)//s + 1."""
    return (n + 2 * p - k) // s + 1


@dataclass
class Weights:
    w: List[np.ndarray] = field(default_factory=list)      # [K,Cin,Cout] float32
    scale: List[np.ndarray] = field(default_factory=list)  # [Cout]
    shift: List[np.ndarray] = field(default_factory=list)  # [Cout]


def fold_bn(gamma, beta, mean, var, eps=1e-5):
    """se-ssd-ai-trt.cpp:816-824: scale = gamma/sqrt(var+eps), shift = beta - mean*gamma/sqrt(var+eps),
    every operation in float32 (the reference's `sqrt` on a float resolves to the float overload)."""
    gamma, beta, mean, var = (np.asarray(a, np.float32) for a in (gamma, beta, mean, var))
    root = np.sqrt(var + np.float32(eps), dtype=np.float32)
    scale = gamma / root
    shift = beta - (mean * gamma) / root
    return scale.astype(np.float32), shift.astype(np.float32)


def random_weights(layers: List[Layer], seed: int = 0, w_std: float = 0.1, bn: bool = True) -> Weights:
    """Seeded random-init weights of the layer shapes: W ~ N(0, w_std) and, when bn is set, random
    BatchNorm statistics folded into a per-channel scale/shift."""
    rng = np.random.default_rng(seed)
    out = Weights()
    for l in layers:
        out.w.append((rng.standard_normal((l.kvol, l.cin, l.cout)) * w_std).astype(np.float32))
        if bn:
            gamma = rng.uniform(0.5, 1.5, l.cout).astype(np.float32)
            beta = rng.uniform(-0.1, 0.3, l.cout).astype(np.float32)
            mean = rng.uniform(-0.2, 0.2, l.cout).astype(np.float32)
            var = rng.uniform(0.5, 1.5, l.cout).astype(np.float32)
            s, b = fold_bn(gamma, beta, mean, var)
        else:
            s, b = np.ones(l.cout, np.float32), np.zeros(l.cout, np.float32)
        out.scale.append(s)
        out.shift.append(b)
    return out


def layer_specs(layers: List[Layer]):
    """ctypes array of sessd_layer_spec for the C-ABI."""
    arr = (D.LayerSpec * len(layers))()
    for i, l in enumerate(layers):
        arr[i].type = l.type
        arr[i].in_channel = l.cin
        arr[i].out_channel = l.cout
        for a in range(3):
            arr[i].ksize[a] = l.ksize[a]
            arr[i].stride[a] = l.stride[a]
            arr[i].padding[a] = l.padding[a]
            arr[i].out_shape[a] = l.out_shape[a]
    return arr


def voxelgen_desc(max_voxels=MAX_VOXELS, max_pts=MAX_NUM_POINTS_PER_VOXEL,
                  pc_range=POINT_CLOUD_RANGE, voxel_size=VOXEL_SIZE):
    d = D.VoxelGenDesc()
    d.max_num_points_per_voxel = max_pts
    d.max_voxels = max_voxels
    for i in range(6):
        d.point_cloud_range[i] = pc_range[i]
    d.voxel_feature_num = VOXEL_FEATURE_NUM
    for i in range(3):
        d.voxel_size[i] = voxel_size[i]
    return d


def dense_desc(size_xyz=DENSE_SIZE_XYZ, channel=DENSE_CHANNEL):
    d = D.Sparse2DenseDesc()
    for i in range(3):
        d.feature_map_size[i] = size_xyz[i]
    d.feature_map_channel = channel
    return d


WTS_PREFIX = "backbone.middle_conv."


def write_wts(path, blobs) -> None:
    """Writes `{name: array}` in the reference's text weight format (tools/gen_wts.py:86-99): the blob
    count, then per blob `name count` and the big-endian hex of every float32."""
    with open(path, "w") as f:
        f.write("%d\n" % len(blobs))
        for name, v in blobs.items():
            a = np.ascontiguousarray(v, np.float32).reshape(-1)
            f.write("%s %d " % (name, a.size))
            for word in a.view(np.uint32):
                f.write(" %08x" % int(word))
            f.write("\n")


def random_state_dict(layers: List[Layer], seed: int = 0, w_std: float = 0.1):
    """Seeded stand-in for the `backbone.middle_conv.*` entries of an SE-SSD checkpoint: conv weights
    [kz,ky,kx,Cin,Cout] and BatchNorm1d weight/bias/running_mean/running_var (+ num_batches_tracked, which
    the reference's generator also writes and its loader ignores)."""
    rng = np.random.default_rng(seed)
    sd = {}
    for l in layers:
        i = conv_index(l)
        sd["%s%d.weight" % (WTS_PREFIX, i)] = (rng.standard_normal(l.ksize + (l.cin, l.cout)) * w_std).astype(np.float32)
        sd["%s%d.weight" % (WTS_PREFIX, i + 1)] = rng.uniform(0.5, 1.5, l.cout).astype(np.float32)
        sd["%s%d.bias" % (WTS_PREFIX, i + 1)] = rng.uniform(-0.1, 0.3, l.cout).astype(np.float32)
        sd["%s%d.running_mean" % (WTS_PREFIX, i + 1)] = rng.uniform(-0.2, 0.2, l.cout).astype(np.float32)
        sd["%s%d.running_var" % (WTS_PREFIX, i + 1)] = rng.uniform(0.5, 1.5, l.cout).astype(np.float32)
        sd["%s%d.num_batches_tracked" % (WTS_PREFIX, i + 1)] = np.array([1234.0], np.float32)
    return sd


def weights_from_blobs(layers: List[Layer], get, eps: float = 1e-5) -> Weights:
    """`get(name) -> flat float32 array` (a parsed weight file or a dict) -> per-layer [K,Cin,Cout] weights
    and folded BatchNorm scale/shift, by the blob names the reference uses (se-ssd-ai-trt.cpp:1147-1249)."""
    out = Weights()
    for l in layers:
        i = conv_index(l)
        out.w.append(np.asarray(get("%s%d.weight" % (WTS_PREFIX, i)), np.float32).reshape(l.kvol, l.cin, l.cout))
        bn = "%s%d" % (WTS_PREFIX, i + 1)
        s, b = fold_bn(*(np.asarray(get(bn + k), np.float32).reshape(-1)
                         for k in (".weight", ".bias", ".running_mean", ".running_var")), eps=eps)
        out.scale.append(s)
        out.shift.append(b)
    return out
