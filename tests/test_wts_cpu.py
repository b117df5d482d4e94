"""The `.wts` weight-file reader and BatchNorm folding (host side of the library; no GPU call).

Format: writer tools/gen_wts.py:86-99 (`struct.pack('>f', v).hex()` per element), reader
se-ssd-ai-trt.cpp:276-314 (`>> std::hex` into a uint32 reinterpreted as float)."""
import struct

import numpy as np
import pytest

import oracle_lib as O
from sessd3d import api, backbone as B


def test_known_bit_patterns():
    text = "2\na.b 6 3f800000 c0490fdb 00000001 7f800000 80000000 7fc00000\nempty 0 \n"
    w = api.WeightFile(text=text)
    assert w.names() == ["a.b", "empty"]
    v = w["a.b"]
    assert v[0] == 1.0 and v[1] == np.float32(-3.14159274) and v[3] == np.inf
    assert v.view(np.uint32).tolist() == [0x3F800000, 0xC0490FDB, 1, 0x7F800000, 0x80000000, 0x7FC00000]
    assert w["empty"].size == 0
    with pytest.raises(api.SessdError, match="no blob named"):
        w["missing"]


def test_round_trip_of_the_generator_format(tmp_path):
    rng = np.random.default_rng(0)
    blobs = {"backbone.middle_conv.0.weight": rng.standard_normal((3, 3, 3, 4, 16)).astype(np.float32),
             "backbone.middle_conv.1.running_var": rng.uniform(0, 2, 16).astype(np.float32),
             "tiny": np.array([1e-45, -0.0, np.inf, -np.inf, np.nan, 3.4028235e38], np.float32)}
    path = tmp_path / "m.wts"
    B.write_wts(path, blobs)
    lines = open(path).read().split("\n")
    assert lines[0] == "3"
    # the writer's tokens are exactly struct.pack('>f').hex() of the reference's generator
    name, count, *tok = lines[3].split()
    assert (name, count) == ("tiny", "6")
    assert tok == [struct.pack(">f", float(v)).hex() for v in blobs["tiny"][:4]] + ["7fc00000", "7f7fffff"]
    w = api.WeightFile(path=str(path))
    assert w.names() == list(blobs)
    for k, v in blobs.items():
        assert np.array_equal(w[k].view(np.uint32), v.reshape(-1).view(np.uint32)), k
    # independent decode of the same text: big-endian float per token
    back = np.array([struct.unpack(">f", bytes.fromhex(t))[0] for t in lines[2].split()[2:]], np.float32)
    assert np.array_equal(back, w["backbone.middle_conv.1.running_var"])


@pytest.mark.parametrize("text,msg", [
    ("", "positive blob count"), ("0\n", "positive blob count"), ("x\n", "positive blob count"),
    ("2\na 1 3f800000\n", "2 blobs announced, 1 found"), ("1\na 3 3f800000 3f800000\n", "element 2 of 3"),
    ("1\na 1 3g800000\n", "not 32-bit hex"), ("1\na 1 13f800000\n", "not 32-bit hex"), ("1\na -1\n", "element count"),
    ("1\na 1000000000000 3f800000\n", "the file ends before that"),       # 2^40 elements announced: refused, not allocated
    ("1\na 99 3f800000 3f800000\n", "the file ends before that"),
])
def test_malformed_files_are_errors_not_asserts(text, msg):
    with pytest.raises(api.SessdError, match=msg):
        api.WeightFile(text=text)


def test_missing_file():
    with pytest.raises(api.SessdError, match="cannot open"):
        api.WeightFile(path="/nonexistent/dir/model.wts")


def test_uppercase_hex_and_repeated_names():
    w = api.WeightFile(text="2\na 1 3F800000\na 2 40000000 0x40400000\n")
    assert w.names() == ["a"] and w["a"].tolist() == [2.0, 3.0]     # map assignment: the later blob wins


def test_fold_batchnorm_matches_the_oracle_and_the_closed_form():
    rng = np.random.default_rng(5)
    g, b, m = rng.normal(size=(3, 257)).astype(np.float32)
    v = rng.uniform(1e-3, 3, 257).astype(np.float32)
    sc, sh = api.fold_batchnorm(g, b, m, v, 1e-5)
    o_sc, o_sh = O.fold_bn(g, b, m, v, 1e-5)
    assert np.array_equal(sc, o_sc) and np.array_equal(sh, o_sh)
    p_sc, p_sh = B.fold_bn(g, b, m, v, 1e-5)
    assert np.array_equal(sc, p_sc) and np.array_equal(sh, p_sh)
    want = g.astype(np.float64) / np.sqrt(v.astype(np.float64) + 1e-5)
    assert np.allclose(sc, want, rtol=3e-7, atol=0)
    assert np.allclose(sh, b - m * want, rtol=1e-5, atol=1e-6)
    # y = (x - mean)/sqrt(var + eps)*gamma + beta
    x = rng.normal(size=(10, 257)).astype(np.float32)
    assert np.allclose(x * sc + sh, (x - m) / np.sqrt(v + 1e-5) * g + b, rtol=1e-4, atol=1e-5)


def test_weights_from_blobs_shapes_and_names(tmp_path):
    layers = B.reference_layers()
    sd = B.random_state_dict(layers, seed=3)
    assert len(sd) == 14 * 6 and "backbone.middle_conv.39.weight" in sd and "backbone.middle_conv.40.running_var" in sd
    path = tmp_path / "bb.wts"
    B.write_wts(path, sd)
    wf = api.WeightFile(path=str(path))
    W = B.weights_from_blobs(layers, wf.__getitem__)
    for l, w, s in zip(layers, W.w, W.scale):
        assert w.shape == (l.kvol, l.cin, l.cout) and s.shape == (l.cout,)
    # [kz,ky,kx,Cin,Cout] flattened = [K][Cin][Cout] with K = kz*9 + ky*3 + kx (submConv3dlayer.cu:510)
    assert np.array_equal(W.w[0][1 * 9 + 2 * 3 + 0], sd["backbone.middle_conv.0.weight"][1, 2, 0])
    i = B.conv_index(layers[-1])
    assert i == 39 and W.w[-1].shape == (3, 64, 64)


def test_load_frame_reads_kitti_layout(tmp_path):
    rng = np.random.default_rng(9)
    pts = rng.uniform(-50, 50, (1234, 4)).astype(np.float32)
    path = tmp_path / "000007.bin"
    pts.tofile(path)
    buf, n = api.load_frame(str(path), 2000)
    assert n == 1234 and np.array_equal(buf[:n], pts) and not buf[n:].any()
    # bytes that do not fill a point are ignored: points_size = bytes / 4 / sizeof(float) (se-ssd-ai-trt.cpp:1850)
    with open(path, "ab") as f:
        f.write(b"\x01\x02\x03\x04\x05\x06\x07")
    buf2 = np.full((2000, 4), 7.0, np.float32)
    _, n2 = api.load_frame(str(path), 2000, out=buf2)
    assert n2 == 1234 and np.array_equal(buf2[:n2], pts) and not buf2[n2:].any()
    with pytest.raises(api.SessdError, match="holds"):
        api.load_frame(str(path), 1000)                       # does not fit: error, where the reference exits
    with pytest.raises(api.SessdError, match="cannot open"):
        api.load_frame(str(tmp_path / "nope.bin"), 1000)
    empty = tmp_path / "empty.bin"
    empty.write_bytes(b"")
    assert api.load_frame(str(empty), 10)[1] == 0


def test_load_frame_on_the_reference_fixture(kitti_frame0):
    """The first frame of the reference's data directory (kept under tests/golden): 20 285 points."""
    from conftest import KITTI_FRAME0
    buf, n = api.load_frame(KITTI_FRAME0, B.MAX_POINTS)
    assert n == len(kitti_frame0) == 20285 and np.array_equal(buf[:n], kitti_frame0)
