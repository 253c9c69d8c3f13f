"""ONNX loader (Graph::load / Tensor::loadProtoBuf), CPU part: the graphs the loader builds from
the fixture files under tests/golden/onnx (written by tests/golden/make_onnx_fixtures.py - three by
PyTorch's ONNX serializer, one field by field) have the nodes, attributes, parameter tensors and
shapes the files describe, by the mapping of the reference's loader (src/onnx.cpp:373-743)."""
import os
import struct

import numpy as np
import pytest

from saga_amd import api as S

ONNX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "onnx")


def model_path(name):
    return os.path.join(ONNX, name, name + ".onnx")


def load(name):
    return S.Graph.load(model_path(name))


def types(g):
    return [line.split(" | ")[0] for line in g.describe()]


def test_tensor_files():
    """input_0.pb / output_0.pb: raw_data tensors with packed dims."""
    for name, ishape, oshape in [("mini_resnet", [2, 3, 16, 16], [2, 10]), ("handmade", [1, 4, 8, 8], [1, 5])]:
        d = os.path.join(ONNX, name, "test_data_set_0")
        x = S.Tensor.load_protobuf(os.path.join(d, "input_0.pb"))
        y = S.Tensor.load_protobuf(os.path.join(d, "output_0.pb"))
        assert x.dims == ishape and y.dims == oshape and x.dtype == S.FLOAT
        raw = open(os.path.join(d, "input_0.pb"), "rb").read()
        # the payload of the raw_data field is the last ishape-many floats before the name field
        n = int(np.prod(ishape))
        at = raw.index(b"\x42\x07input_0") - 4 * n
        np.testing.assert_array_equal(x.read().reshape(-1), np.frombuffer(raw[at:at + 4 * n], np.float32))


def test_mini_resnet_structure():
    g = load("mini_resnet")
    t = types(g)
    # the fc node brings no reshape of its own: Flatten already produced a rank-2 tensor
    assert t.count("conv") == 6 and t.count("batchnorm") == 6 and t.count("add") == 2
    assert t.count("maxpool") == 1 and t.count("avgpool") == 1 and t.count("fc") == 1 and t.count("reshape") == 1
    lines = g.describe()
    stem = lines[0]
    assert stem.startswith("conv | ") and "pad=1" in stem and "stride=1" in stem
    assert ":float[2, 3, 16, 16]" in stem and "[8, 3, 3, 3]" in stem and stem.endswith("float[2, 8, 16, 16]")
    pool = next(l for l in lines if l.startswith("maxpool"))
    assert "pad=1" in pool and "size=3" in pool and "stride=2" in pool and pool.endswith("[2, 8, 8, 8]")
    gap = next(l for l in lines if l.startswith("avgpool"))
    assert "global=true" in gap.lower() or "global=1" in gap
    assert gap.endswith("[2, 16, 1, 1]")
    down = [l for l in lines if l.startswith("conv") and "stride=2" in l]
    assert len(down) == 2  # the 3x3 and the 1x1 projection of the down-sampling block
    fc = next(l for l in lines if l.startswith("fc"))
    assert "transW=" in fc and "[10, 16]" in fc and fc.endswith("float[2, 10]")
    bn = next(l for l in lines if l.startswith("batchnorm"))
    assert "epsilon=" in bn and all(f" {s}=" in " " + bn.split(" | ")[1] for s in "xsbmv")
    ins, outs = g.inputs(), g.outputs()
    assert len(ins) == 1 and ins[0].dims == [2, 3, 16, 16]
    assert len(outs) == 1 and outs[0].dims == [2, 10]


def test_mini_squeezenet_structure():
    g = load("mini_squeezenet")
    t = types(g)
    assert t.count("concat") == 3 and t.count("softmax") == 1 and t.count("maxpool") == 2
    lines = g.describe()
    first = lines[0]
    assert "pad=0" in first and "stride=2" in first and " b=" in first  # bias attached as input b
    cat = next(l for l in lines if l.startswith("concat"))
    assert " x0=" in " " + cat and " x1=" in cat and cat.endswith("[2, 16, 8, 8]")
    assert g.outputs()[0].dims == [2, 10]


def test_handmade_structure_and_values():
    """Unpacked repeated fields, float_data / int64_data initializers, symbolic batch dimension,
    initializers that are also listed as inputs."""
    g = load("handmade")
    lines = g.describe()
    assert types(g) == ["conv", "leakyrelu", "conv", "conv", "sum", "dropout", "avgpool", "reshape", "fc", "add"]
    assert "pad=1" in lines[0] and "stride=1" in lines[0]
    assert "alpha=0.1" in lines[1]
    assert " x2=" in lines[4]
    assert "size=4" in lines[6] and "stride=4" in lines[6] and lines[6].endswith("[1, 6, 2, 2]")
    assert lines[7].endswith("[1, 24]")
    ins = g.inputs()
    assert [i.dims for i in ins] == [[1, 4, 8, 8]]  # w1 and shape are parameters, N counts as 1
    # float_data written one value per field and int64_data with a negative varint
    raw = open(model_path("handmade"), "rb").read()
    w1 = g.named_tensor("w1").read()
    first = struct.unpack("<f", raw[raw.index(b"\x25") + 1:raw.index(b"\x25") + 5])[0]
    assert w1.shape == (6, 4, 3, 3) and np.isfinite(w1).all() and np.abs(w1).max() > 0
    assert any(np.isclose(first, v) for v in w1.reshape(-1)[:4])
    np.testing.assert_array_equal(g.named_tensor("shape").read(), [0, -1])


def test_errors_return_null(tmp_path):
    """Missing files, truncated files and unknown operators fail with a message, not a crash."""
    with pytest.raises(S.SagaError):
        S.Graph.load(str(tmp_path / "missing.onnx"))
    raw = open(model_path("mini_vgg"), "rb").read()
    cut = tmp_path / "cut.onnx"
    cut.write_bytes(raw[:len(raw) // 2])
    with pytest.raises(S.SagaError):
        S.Graph.load(str(cut))
    bad = tmp_path / "bad.onnx"
    bad.write_bytes(raw.replace(b"MaxPool", b"MaxFool"))
    with pytest.raises(S.SagaError):
        S.Graph.load(str(bad))
    with pytest.raises(S.SagaError):
        S.Tensor.load_protobuf(str(tmp_path / "missing.pb"))
