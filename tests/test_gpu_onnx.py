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
