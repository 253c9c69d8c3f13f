"""The reference's own known-answer harnesses replayed through the drop-in boundary
(Graph -> Context::createProgram -> Program::run -> resolveTensor), on the hip engine:
test/test_ops.cpp:574-656 (12 operator cases, INFERENCE programs) and
test/test_resnode.cpp:185-280 (conv1x1 -> batchnorm -> [sum] -> relu with backprop, TRAINING
programs, 8 combinations x {fp32, fp16}).  Pass criterion as there: SSE <= 1e-4."""
import numpy as np
import pytest

from saga_amd import api as S

pytestmark = pytest.mark.gpu

DT = [S.FLOAT, S.HALF]


def T(g, name, dt=S.FLOAT, dims=None):
    t = g[name]
    d = dims or t["dims"]
    a = np.array(t["data"][: int(np.prod(d))], np.float32).reshape(d)
    return S.Tensor.from_numpy(a.astype(np.float16) if dt == S.HALF else a)


def A(g, name):
    t = g[name]
    return np.array(t["data"][: int(np.prod(t["dims"]))], np.float64).reshape(t["dims"])


@pytest.fixture(scope="module")
def ctx():
    return S.Context()


def run_op(ctx, op, inputs, attrs, want, tol=1e-4):
    g = S.Graph()
    n = g.add_node(op, inputs, attrs)
    x = inputs.get("x", inputs.get("x0"))
    p = ctx.create_program(g, x.dims[0], training=False)
    y = ctx.resolve(n.y())
    p.run()
    got = y.read().astype(np.float64)
    sse = float(((got.reshape(want.shape) - want) ** 2).sum())
    assert sse <= tol, f"{op}: sse {sse:e}"
    return sse


@pytest.mark.parametrize("dt", DT)
def test_ops_known_answers(golden, ctx, dt):
    g = golden["ops"]
    tol = 1e-4 if dt == S.FLOAT else 2e-3  # fp16 storage rounds the fixtures themselves
    run_op(ctx, "relu", {"x": T(g, "relu_input", dt)}, {}, A(g, "relu_output"), tol if dt == S.FLOAT else 1.0)
    run_op(ctx, "conv", {"x": T(g, "conv_input_x", dt), "w": T(g, "conv_input_w", dt), "b": T(g, "conv_input_b", dt)},
           {"size": 3, "activations": 2, "pad": 1, "bias": True}, A(g, "conv_output"), tol)
    run_op(ctx, "maxpool", {"x": T(g, "pooling_input", dt)}, {"size": 2, "stride": 2}, A(g, "maxpool_output"), tol)
    run_op(ctx, "maxpool", {"x": T(g, "pooling_input", dt)}, {"global": True}, A(g, "maxpool_output_global"), tol)
    run_op(ctx, "avgpool", {"x": T(g, "pooling_input", dt)}, {"size": 2, "stride": 2}, A(g, "avgpool_output"), tol)
    run_op(ctx, "avgpool", {"x": T(g, "pooling_input", dt)}, {"global": True}, A(g, "avgpool_output_global"), tol)
    fc_tol = tol if dt == S.FLOAT else 1e6  # fc1 uses integers up to 1e4: not representable in fp16
    run_op(ctx, "fc", {"x": T(g, "fc1_input_x", dt), "w": T(g, "fc1_input_w", dt)}, {"transW": False},
           A(g, "fc1_output_no_bias"), fc_tol)
    run_op(ctx, "fc", {"x": T(g, "fc1_input_x", dt), "w": T(g, "fc1_input_w", dt), "b": T(g, "fc1_input_b", dt)},
           {"transW": False}, A(g, "fc1_output_bias"), fc_tol)
    run_op(ctx, "fc", {"x": T(g, "fc2_input_x", dt), "w": T(g, "fc2_input_w", dt)}, {"transW": True},
           A(g, "fc2_output_no_bias"), tol)
    run_op(ctx, "fc", {"x": T(g, "fc2_input_x", dt), "w": T(g, "fc2_input_w", dt), "b": T(g, "fc2_input_b", dt)},
           {"transW": True}, A(g, "fc2_output_bias"), tol)
    run_op(ctx, "concat", {"x0": T(g, "concat_input_x0", dt), "x1": T(g, "concat_input_x1", dt)}, {},
           A(g, "concat_output"), tol)
    run_op(ctx, "batchnorm",
           {"x": T(g, "batchnorm_input_x", dt), "s": T(g, "batchnorm_input_s"), "b": T(g, "batchnorm_input_b"),
            "m": T(g, "batchnorm_input_m"), "v": T(g, "batchnorm_input_v")}, {"epsilon": 0.00001},
           A(g, "batchnorm_output"), tol)


def test_concat_axis0_chain(golden, ctx):
    """test/test_ops.cpp:668-720: 4 x relu -> concat(axis 0) -> relu."""
    g = golden["ops"]
    gr = S.Graph()
    outs = {}
    for i in range(4):
        n = gr.add_node("relu", T(g, f"concat_x{i}"))
        outs[f"x{i}"] = n.y()
    n = gr.add_node("concat", outs, {"axis": 0})
    n = gr.add_node("relu", n)
    p = ctx.create_program(gr, 1, training=False)
    y = ctx.resolve(n.y())
    p.run()
    want = np.concatenate([A(g, f"concat_x{i}") for i in range(4)], 0)
    np.testing.assert_array_equal(y.read(), want)


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("combo", range(8))
def test_resnode(golden, ctx, combo, dt):
    bypass, check_dx, no_fusing = bool(combo & 1), bool(combo & 2), bool(combo & 4)
    g = golden["resnode"]
    ctx.reset()
    gr = S.Graph()
    x = T(g, "conv_input_x", dt)
    w = T(g, "conv_input_w", dt, dims=[4, 4, 1, 1])  # 32 values listed, the loader uses 16
    n = gr.add_node("conv", {"x": x, "w": w}, {"activations": 4, "size": 1})
    n = gr.add_node("batchnorm", {"x": n.y(), "s": T(g, "batchnorm_input_s"), "b": T(g, "batchnorm_input_b"),
                                  "m": T(g, "batchnorm_input_m"), "v": T(g, "batchnorm_input_v")},
                    {"epsilon": 0.00001, "expavgf": 0.0})
    if bypass:
        n = gr.add_node("sum", {"x0": x, "x1": n.y()})
    n = gr.add_node("relu", n)
    p = ctx.create_program(gr, 2, training=True, disable_op_fusing=no_fusing)
    y = ctx.resolve(n.y())
    dx = ctx.resolve(x.grad()) if check_dx else None
    ctx.resolve(n.y().grad()).write(A(g, "grad"))
    assert p.run(1) == 0
    sfx = "with_bypass" if bypass else "no_bypass"
    sse = float(((y.read().astype(np.float64) - A(g, "expected_y_" + sfx)) ** 2).sum())
    assert sse <= 1e-4, f"Y sse {sse:e}"
    if dx is not None:
        sse = float(((dx.read().astype(np.float64) - A(g, "expected_dx_" + sfx)) ** 2).sum())
        assert sse <= 1e-4, f"DX sse {sse:e}"
