"""Model files (.odl) and checkpoints: the reference's on-disk formats (src/io/model_io.cpp:116-273,
src/io/checkpoint.cpp:13-226) read and written by this repository's host layer.

Pinned three ways: a file written by the compiled reference is committed (tests/golden/ref_mlp.odl) and parsed here
byte by byte with an independent reader; where the compiled reference is present, files cross between the two
implementations in both directions; and the host layer's own files are parsed by the same independent reader.
The CPU tests use the host layer with tensors left on the CPU (no compute); the GPU test loads the reference's file
onto the device and runs the model."""
import os
import struct

import numpy as np
import pytest

import oraclelib as ol

f32 = np.float32
HERE = os.path.dirname(os.path.abspath(__file__))
G = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))
REF_FILE = os.path.join(HERE, "golden", "ref_mlp.odl")
NAMES = ("layer_0.weight", "layer_0.bias", "layer_1.weight", "layer_1.bias")
SHAPES = {"layer_0.weight": (4, 8), "layer_0.bias": (1, 8), "layer_1.weight": (8, 2), "layer_1.bias": (1, 2)}
needs_ref = pytest.mark.skipif(not ol.have_ref(), reason="compiled reference (oracle/_ref) not built here")


def parse_odl(path):
    """name -> (array, dtype code, (device type, device index)); raises on anything but a well-formed file."""
    raw = open(path, "rb").read()
    pos = 0

    def take(fmt):
        nonlocal pos
        vals = struct.unpack_from("<" + fmt, raw, pos)
        pos += struct.calcsize("<" + fmt)
        return vals if len(vals) > 1 else vals[0]

    assert take("I") == 0x4F444C00 and take("I") == 1
    entries = {}
    for _ in range(take("Q")):
        n = take("Q")
        name = raw[pos:pos + n].decode()
        pos += n
        rank = take("Q")
        shape = tuple(take("Q") for _ in range(rank))
        dtype, dev_type, dev_index = take("i"), take("i"), take("i")
        count = int(np.prod(shape)) if shape else 1
        np_dtype = {0: np.float32}.get(dtype)
        assert np_dtype is not None, "only float32 entries are expected in these tests (dtype code %d)" % dtype
        arr = np.frombuffer(raw, np_dtype, count, pos).reshape(shape)
        pos += arr.nbytes
        entries[name] = (arr, dtype, (dev_type, dev_index))
    assert pos == len(raw), "trailing bytes"
    return entries


def split_params(flat):
    out, p = {}, 0
    for n in NAMES:
        k = int(np.prod(SHAPES[n]))
        out[n] = flat[p:p + k].reshape(SHAPES[n])
        p += k
    return out


def test_reference_written_file_parses_to_its_parameters():
    entries = parse_odl(REF_FILE)
    want = split_params(G["io_mlp_params"])
    assert set(entries) == set(NAMES)
    for n in NAMES:
        arr, dtype, dev = entries[n]
        assert arr.shape == SHAPES[n] and dtype == 0 and dev == (0, 0)  # float32, saved from CPU tensors
        assert np.array_equal(arr, want[n])


def test_host_layer_reads_and_writes_the_format_without_a_gpu(tmp_path):
    hc = ol.host_driver(cpu=True)
    back = np.empty(58, f32)
    assert hc.odl_hostcpu_load_mlp(REF_FILE.encode(), 1, None, back, None) == 0
    assert np.array_equal(back, G["io_mlp_params"])
    mine = str(tmp_path / "mine.odl")
    params = np.random.default_rng(2).standard_normal(58).astype(f32)
    assert hc.odl_hostcpu_save_mlp(params, mine.encode()) == 0
    entries = parse_odl(mine)
    want = split_params(params)
    assert set(entries) == set(NAMES)
    for n in NAMES:
        assert np.array_equal(entries[n][0], want[n]) and entries[n][1:] == (0, (0, 0))
    assert os.path.getsize(mine) == os.path.getsize(REF_FILE)  # same layout, entry order aside
    assert hc.odl_hostcpu_load_mlp(mine.encode(), 1, None, back, None) == 0 and np.array_equal(back, params)
    # damaged files are refused with the reference's runtime_error: truncated data, wrong magic, missing file
    raw = open(mine, "rb").read()
    for name, blob in (("short.odl", raw[:-5]), ("magic.odl", b"XXXX" + raw[4:]), ("version.odl", raw[:4] + b"\x02\0\0\0" + raw[8:]),
                       ("count.odl", raw[:8] + struct.pack("<Q", 1 << 40) + raw[16:]), ("empty.odl", b"")):
        bad = str(tmp_path / name)
        open(bad, "wb").write(blob)
        assert hc.odl_hostcpu_load_mlp(bad.encode(), 1, None, back, None) == -2, name
    assert hc.odl_hostcpu_load_mlp(str(tmp_path / "absent.odl").encode(), 1, None, back, None) == -2
    # strict loading refuses a file with a missing or an extra entry; non-strict takes what matches
    def rewrite(keep, extra=False):
        ents = parse_odl(mine)
        blob = struct.pack("<IIQ", 0x4F444C00, 1, len(keep) + (1 if extra else 0))
        for n in list(keep) + (["stranger"] if extra else []):
            arr = ents[n][0] if n in ents else np.zeros((2,), f32)
            blob += struct.pack("<Q", len(n)) + n.encode() + struct.pack("<Q", arr.ndim)
            blob += b"".join(struct.pack("<Q", d) for d in arr.shape) + struct.pack("<iii", 0, 0, 0) + arr.tobytes()
        path = str(tmp_path / ("rw%d%d.odl" % (len(keep), extra)))
        open(path, "wb").write(blob)
        return path.encode()
    assert hc.odl_hostcpu_load_mlp(rewrite(NAMES[:3]), 1, None, back, None) == -2
    assert hc.odl_hostcpu_load_mlp(rewrite(NAMES, extra=True), 1, None, back, None) == -2
    assert hc.odl_hostcpu_load_mlp(rewrite(NAMES, extra=True), 0, None, back, None) == 0 and np.array_equal(back, params)


def test_checkpoint_directory_round_trip_without_a_gpu(tmp_path):
    hc = ol.host_driver(cpu=True)
    params = np.random.default_rng(3).standard_normal(58).astype(f32)
    es, fl, back = np.zeros(2, np.int32), np.zeros(5, f32), np.empty(58, f32)
    path = str(tmp_path / "run7.ckpt")
    assert hc.odl_hostcpu_checkpoint_roundtrip(params, path.encode(), 5, 100, 0.5, 0.001, 0.9, 0.999, 1e-8, es, fl, back) == 0
    assert es.tolist() == [5, 100]
    np.testing.assert_allclose(fl, [0.5, 0.001, 0.9, 0.999, 1e-8], rtol=1e-6)  # written as decimal text
    assert np.array_equal(back, params)
    ckdir = str(tmp_path / "run7")  # "X.ckpt" names the directory "X" (checkpoint.cpp:18-22)
    assert sorted(os.listdir(ckdir)) == ["metadata.json", "model.odl"]
    import json
    meta = json.load(open(os.path.join(ckdir, "metadata.json")))
    assert meta["format_type"] == "origindl_checkpoint" and meta["format_version"] == "1.0"
    assert meta["epoch"] == 5 and meta["step"] == 100 and meta["optimizer_type"] == "Adam"
    assert set(meta["optimizer_config"]) == {"lr", "beta1", "beta2", "eps"}
    assert set(parse_odl(os.path.join(ckdir, "model.odl"))) == set(NAMES)


@needs_ref
def test_files_cross_between_the_reference_and_the_host_layer(tmp_path):
    r, hc = ol.ref(), ol.host_driver(cpu=True)
    params = np.random.default_rng(4).standard_normal(58).astype(f32)
    theirs, mine = str(tmp_path / "theirs.odl"), str(tmp_path / "mine.odl")
    assert r.odl_ref_save_mlp(params, theirs.encode()) == 0
    assert hc.odl_hostcpu_save_mlp(params, mine.encode()) == 0
    a, b = parse_odl(theirs), parse_odl(mine)
    assert set(a) == set(b) and all(np.array_equal(a[n][0], b[n][0]) and a[n][1:] == b[n][1:] for n in a)
    back = np.empty(58, f32)
    assert hc.odl_hostcpu_load_mlp(theirs.encode(), 1, None, back, None) == 0 and np.array_equal(back, params)
    x, y = np.random.default_rng(5).standard_normal((3, 4)).astype(f32), np.empty((3, 2), f32)
    assert r.odl_ref_load_mlp(mine.encode(), 1, x, back, y) == 0 and np.array_equal(back, params)
    # the checkpoint directory of either side reads on the other: same metadata lines, same model file
    es, fl = np.zeros(2, np.int32), np.zeros(5, f32)
    for drv, fn, path in ((r, "odl_ref_checkpoint_roundtrip", tmp_path / "ref.ckpt"),
                          (hc, "odl_hostcpu_checkpoint_roundtrip", tmp_path / "host.ckpt")):
        assert getattr(drv, fn)(params, str(path).encode(), 3, 42, 1.25, 0.01, 0.8, 0.99, 1e-6, es, fl, back) == 0
        assert es.tolist() == [3, 42] and np.array_equal(back, params)
    ref_meta = open(tmp_path / "ref" / "metadata.json").read().splitlines()
    host_meta = open(tmp_path / "host" / "metadata.json").read().splitlines()
    assert sorted(l.rstrip(",") for l in ref_meta) == sorted(l.rstrip(",") for l in host_meta)  # the config map's order is unspecified


@pytest.mark.gpu
def test_reference_file_loads_onto_the_device_and_runs(tmp_path):
    h = ol.host_driver()
    back, y = np.empty(58, f32), np.empty((3, 2), f32)
    assert h.odl_host_load_mlp(REF_FILE.encode(), 1, G["io_mlp_x"], back, y) == 0
    assert np.array_equal(back, G["io_mlp_params"])
    np.testing.assert_allclose(y, G["io_mlp_y"], rtol=1e-5, atol=1e-6)  # the reference's own forward of the same file
    # a checkpoint written and read back by the device build of the driver
    es, fl = np.zeros(2, np.int32), np.zeros(5, f32)
    assert h.odl_host_checkpoint_roundtrip(G["io_mlp_params"], str(tmp_path / "d.ckpt").encode(), 1, 2, 0.25, 0.001, 0.9,
                                           0.999, 1e-8, es, fl, back) == 0
    assert es.tolist() == [1, 2] and np.array_equal(back, G["io_mlp_params"])
