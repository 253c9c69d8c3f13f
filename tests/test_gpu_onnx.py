"""ONNX models run on the hip engine: what the reference's `saga onnx <model>` does
(test/test_onnx.cpp:14-94) - load the model, build an inference program in NCHW and in NHWC,
feed test_data_set_0/input_0.pb, compare the output with output_0.pb by the reference's criterion
(sum of squared errors <= 1e-3) and by this build's fp32 bar (1e-4 of the largest expected value).
The model-zoo files the reference names are not in its repository; the fixtures under
tests/golden/onnx stand in for them (expected outputs computed by PyTorch on the CPU)."""
import os

import numpy as np
import pytest

from saga_amd import api as S
from tests.gpu_util import rel_err

pytestmark = pytest.mark.gpu

ONNX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "onnx")


@pytest.mark.parametrize("layout", [S.LAYOUT_NCHW, S.LAYOUT_NHWC], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("name", ["mini_resnet", "mini_squeezenet", "mini_vgg", "handmade"])
def test_onnx_model(name, layout):
    base = os.path.join(ONNX, name)
    g = S.Graph.load(os.path.join(base, name + ".onnx"))
    ctx = S.Context()
    gin, gout = g.inputs(), g.outputs()
    assert len(gin) == 1 and len(gout) == 1
    p = ctx.create_program(g, 1, training=False, tensor_layout=layout)
    x, y = ctx.resolve(gin[0]), ctx.resolve(gout[0])
    p.finalize()
    want_in = S.Tensor.load_protobuf(os.path.join(base, "test_data_set_0", "input_0.pb"))
    want_out = S.Tensor.load_protobuf(os.path.join(base, "test_data_set_0", "output_0.pb"))
    assert x.dims == want_in.dims and y.dims == want_out.dims
    x.write(want_in.read())
    p.run(1)
    got, want = y.read().astype(np.float32), want_out.read()
    sse = float(((got - want) ** 2).sum())
    e = rel_err(got, want)
    print(f"  {name}: SSE {sse:.3e}, rel max-abs err {e:.3e}, engine sse() {want_out.sse(y):.3e}")
    assert np.isfinite(got).all()
    assert sse <= 1e-3 and want_out.sse(y) <= 1e-3
    assert e <= 1e-4
    if name == "mini_squeezenet":  # softmax output
        np.testing.assert_allclose(got.sum(axis=1), 1.0, atol=1e-5)
        np.testing.assert_array_equal(got.argmax(axis=1), want.argmax(axis=1))


def _fixture_module():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_onnx_fixtures", os.path.join(ONNX, "..", "make_onnx_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("half", [False, True], ids=["fp32", "fp16"])
def test_onnx_resnet50_full_size(tmp_path, half):
    """A full ResNet-50 v1.5 (the operator sequence of the model zoo's resnet50-v1-12.onnx, random
    weights) exported by PyTorch into a temporary file, loaded and run at 224x224.  fp32: NCHW
    program against PyTorch's CPU result.  fp16: the same weights stored as FLOAT16, NHWC program on
    the matrix-core path, against PyTorch's fp32 result on the fp16-rounded weights."""
    import torch
    fx = _fixture_module()
    torch.manual_seed(11)
    gen = torch.Generator().manual_seed(12)
    m = fx.ResNet50().eval()
    fx.randomize_bn(m, gen)
    batch = 4 if half else 2
    x = torch.randn(batch, 3, 224, 224, generator=gen)
    if half:
        m = m.half()
        x = x.half()
        # the serializer only traces: run the export on the GPU, where every fp16 operator exists
        blob = fx.export(m.cuda(), x.cuda())
        m = m.cpu().float()
        x = x.float()
    else:
        blob = fx.export(m, x)
    with torch.no_grad():
        want = m(x).numpy()
    path = tmp_path / "resnet50.onnx"
    path.write_bytes(blob)
    g = S.Graph.load(str(path))
    t = [line.split(" | ")[0] for line in g.describe()]
    assert t.count("conv") == 53 and t.count("batchnorm") == 53 and t.count("add") == 16 and t.count("fc") == 1
    ctx = S.Context()
    p = ctx.create_program(g, 1, training=False)
    xi, yo = ctx.resolve(g.inputs()[0]), ctx.resolve(g.outputs()[0])
    assert xi.dtype == (S.HALF if half else S.FLOAT)
    p.finalize()
    xi.write(x.numpy())
    p.run(1)
    got = yo.read().astype(np.float32)
    e = rel_err(got, want)
    print(f"  ResNet-50 from ONNX ({'fp16' if half else 'fp32'}): rel max-abs err {e:.3e}, max |ref| {np.abs(want).max():.3f}")
    assert e <= (2e-2 if half else 1e-4)
    if not half:
        np.testing.assert_array_equal(got.argmax(axis=1), want.argmax(axis=1))
