"""The repository's own reader / writer of the reference's tensor file format (saga_amd/src/tensor.cpp
Tensor::save / Tensor::load, graph.cpp Tensors::saveTensors / loadTensors) against the documented layout of
src/tensor.cpp:1382-1550: "sagaT001", u32 type (0 float, 1 half), u32 rank, rank x u32 extents, row-major
payload; written through <path>.tmp + rename; a directory holds one file per named tensor
(src/graph.cpp:60-104).  The byte layout is built here by hand with struct.pack, independently of the writer."""
import os
import struct

import numpy as np
import pytest

from saga_amd import api as S

SHAPES = [(7,), (3, 4), (2, 3, 5), (2, 3, 4, 5), (1, 1, 1, 1)]


def file_bytes(a):
    code = {np.dtype(np.float32): 0, np.dtype(np.float16): 1}[a.dtype]
    return b"sagaT001" + struct.pack("<II", code, a.ndim) + struct.pack(f"<{a.ndim}I", *a.shape) + a.tobytes()


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("shape", SHAPES)
def test_save_writes_the_documented_bytes_and_load_reads_them_back(tmp_path, shape, dtype):
    rng = np.random.default_rng(len(shape))
    a = rng.standard_normal(shape).astype(dtype)
    path = str(tmp_path / "t")
    S.Tensor.from_numpy(a).save(path)
    assert open(path, "rb").read() == file_bytes(a)
    assert not os.path.exists(path + ".tmp")
    t = S.Tensor.load(path, "t")
    assert t.dims == list(shape) and t.dtype == (S.FLOAT if dtype == np.float32 else S.HALF)
    np.testing.assert_array_equal(t.read(), a)


def test_load_reads_a_hand_built_file(tmp_path):
    a = np.arange(24, dtype=np.float32).reshape(2, 3, 4) / 8
    path = str(tmp_path / "hand")
    with open(path, "wb") as f:
        f.write(file_bytes(a) + b"trailing bytes are ignored")
    np.testing.assert_array_equal(S.Tensor.load(path).read(), a)


def test_load_rejects_malformed_files(tmp_path):
    a = np.ones((2, 3), np.float32)
    good = file_bytes(a)
    cases = {
        "short header": good[:12],
        "bad magic": b"sagaT002" + good[8:],
        "unknown type": good[:8] + struct.pack("<I", 2) + good[12:],
        "rank 9": good[:12] + struct.pack("<I", 9) + b"\0" * 64,
        "extents cut": good[:20],
        "payload cut": good[:-4],
    }
    for name, data in cases.items():
        path = str(tmp_path / name.replace(" ", "_"))
        with open(path, "wb") as f:
            f.write(data)
        with pytest.raises(S.SagaError):
            S.Tensor.load(path)
    with pytest.raises(S.SagaError):
        S.Tensor.load(str(tmp_path / "missing"))


def test_save_refuses_integer_tensors(tmp_path):
    with pytest.raises(S.SagaError):
        S.Tensor.from_numpy(np.arange(4, dtype=np.int32)).save(str(tmp_path / "i"))
    assert not os.listdir(tmp_path)


def test_graph_directory_round_trip(tmp_path):
    """saveTensors writes one file per named tensor of the graph; loadTensors of another graph picks them up by
    file name, and nodes created afterwards find their parameters there (src/tensor.cpp:1142-1180)."""
    rng = np.random.default_rng(3)
    w = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    g = S.Graph()
    x = S.Tensor.from_numpy(np.zeros((1, 3, 8, 8), np.float32))
    g.add_node("conv", {"x": x, "w": S.Tensor.from_numpy(w, name="c1-w")}, {"size": 3, "activations": 4}, "c1")
    g.add_node("batchnorm", {"x": x}, {}, "bn1")  # implicit s, b, m, v get the names bn1-s ...
    d = str(tmp_path / "weights")
    g.save_tensors(d)
    names = sorted(os.listdir(d))
    assert "bn1-s" in names and "bn1-v" in names
    for n in names:
        raw = open(os.path.join(d, n), "rb").read()
        assert raw[:8] == b"sagaT001"
    # an implicit batch-norm scale is ones[1, C]
    assert open(os.path.join(d, "bn1-s"), "rb").read() == file_bytes(np.ones((1, 3), np.float32))
    g2 = S.Graph()
    g2.load_tensors(d)
    for n in names:
        got = g2.named_tensor(n)
        assert got is not None
        np.testing.assert_array_equal(got.read(), S.Tensor.load(os.path.join(d, n)).read())
    # a node created after the load takes its parameter from the directory instead of initialising it
    with open(os.path.join(d, "c2-w"), "wb") as f:
        f.write(file_bytes(w))
    g3 = S.Graph()
    g3.load_tensors(d)
    n = g3.add_node("conv", {"x": x}, {"size": 3, "activations": 4}, "c2")
    np.testing.assert_array_equal(n.input("w").read(), w)


def graph_from_directory(net, x, directory):
    """The node list of `net` added to a graph that has loaded `directory`: every parameter is found by its
    name among the loaded tensors (and so becomes a named tensor of the graph, which saveTensors writes)."""
    g = S.Graph()
    g.load_tensors(directory)
    t = {net.input: S.Tensor.from_numpy(x)}
    for nd in net.nodes:
        ins = {k: t[v] for k, v in nd["in"].items() if v in t}
        t[nd["out"]] = g.add_node(nd["type"], ins, nd["attrs"], nd["name"]).y()
    node = g.add_node("catclassifier", {"x": t[net.output]})
    t["labels"] = node.y().grad()
    return g, t


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [S.FLOAT, S.HALF])
def test_device_tensors_save_in_logical_order_and_reload(tmp_path, dt):
    """A directory of hand-built tensor files initialises a network on the GPU (loadTensors + lookup by name);
    after two training steps Graph::saveTensors(dir, ctx) writes the parameters as they are on the device -
    fp16 filters live there in channels-last order, the file is row-major in logical N,C,H,W order - and a
    second context that loads that directory computes bit-identical inference results."""
    from saga_amd import networks as N
    net = N.resnet20(4, dtype=dt)
    rng = np.random.default_rng(8)
    x = rng.standard_normal((4, 3, 32, 32)).astype(N.np_dtype(dt))
    d0 = tmp_path / "initial"
    d0.mkdir()
    for k, v in net.params.items():
        is_bn = k.endswith(("-s", "-m", "-v")) or (k.endswith("-b") and k[:-2] + "-s" in net.params)
        with open(d0 / k, "wb") as f:
            f.write(file_bytes(np.asarray(v).astype(np.float32 if is_bn else N.np_dtype(dt))))
    ctx = S.Context()
    g, t = graph_from_directory(net, x, str(d0))
    p = ctx.create_program(g, 4, training=True, learning_rate=1e-2)
    infer = ctx.create_program(g, 4, training=False)
    ctx.resolve(t["labels"]).write(rng.integers(0, 10, (4, 1)).astype(np.int32))
    logits = ctx.resolve(t[net.output])
    # the files initialised the device: same inference result as the same weights handed over explicitly
    infer.run(1)
    ctx_b = S.Context()
    gb, tb = N.build_graph(net, x)
    pb = ctx_b.create_program(gb, 4, training=False)
    lb = ctx_b.resolve(tb[net.output])
    pb.run(1)
    np.testing.assert_array_equal(logits.read(), lb.read())
    p.run(2)
    infer.run(1)
    want_logits = logits.read()
    d = str(tmp_path / "w")
    g.save_tensors(d, ctx)
    assert sorted(os.listdir(d)) == sorted(net.params)
    for k in ("s1-conv-w", "s3_0-conv-p-w", "fc-w", "fc-b", "s2_0-bn-1-s", "s2_0-bn-1-m"):
        dev = ctx.resolve(g.named_tensor(k)).read()
        assert not np.array_equal(dev.astype(np.float32), np.asarray(net.params[k], np.float32).reshape(dev.shape)), k
        assert open(os.path.join(d, k), "rb").read() == file_bytes(np.ascontiguousarray(dev)), k
    ctx2 = S.Context()
    g2, t2 = graph_from_directory(N.resnet20(4, dtype=dt, seed=99), x, d)
    p2 = ctx2.create_program(g2, 4, training=False)
    out = ctx2.resolve(t2[net.output])
    p2.run(1)
    np.testing.assert_array_equal(out.read(), want_logits)
