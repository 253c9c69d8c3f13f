"""Pins the CPU oracle to the known-answer vectors the reference's own tests hold
(test/test_ops.cpp:574-656 and test/test_resnode.cpp:185-253), with the reference's own
tolerance: sum of squared errors <= 1e-4 (test/test_ops.cpp:535-537)."""
import numpy as np
import pytest

from oracle import ref


def T(g, name):
    t = g[name]
    return np.array(t["data"][: int(np.prod(t["dims"]))], np.float32).reshape(t["dims"])


def sse(a, b):
    return float(((np.asarray(a, np.float64) - np.asarray(b, np.float64)) ** 2).sum())


def test_relu(golden):
    g = golden["ops"]
    assert sse(ref.act_fwd(T(g, "relu_input")), T(g, "relu_output")) <= 1e-4


def test_conv_bias(golden):
    g = golden["ops"]
    y = ref.conv2d_fwd(T(g, "conv_input_x"), T(g, "conv_input_w"), pad=1)
    y = ref.bias_add(y, T(g, "conv_input_b"))
    assert sse(y, T(g, "conv_output")) <= 1e-4


def test_pooling(golden):
    g = golden["ops"]
    x = T(g, "pooling_input")
    assert sse(ref.maxpool_fwd(x, 2, 0, 2), T(g, "maxpool_output")) <= 1e-4
    assert sse(ref.maxpool_fwd(x, 8, 0, 1), T(g, "maxpool_output_global")) <= 1e-4
    assert sse(ref.avgpool_fwd(x, 2, 0, 2), T(g, "avgpool_output")) <= 1e-4
    assert sse(ref.avgpool_fwd(x, 8, 0, 1), T(g, "avgpool_output_global")) <= 1e-4


def test_fc(golden):
    g = golden["ops"]
    y = ref.fc_fwd(T(g, "fc1_input_x"), T(g, "fc1_input_w"), transW=False)
    assert sse(y, T(g, "fc1_output_no_bias")) <= 1e-4
    assert sse(y + T(g, "fc1_input_b")[None, :], T(g, "fc1_output_bias")) <= 1e-4
    y = ref.fc_fwd(T(g, "fc2_input_x"), T(g, "fc2_input_w"), transW=True)
    assert sse(y, T(g, "fc2_output_no_bias")) <= 1e-4
    assert sse(y + T(g, "fc2_input_b")[None, :], T(g, "fc2_output_bias")) <= 1e-4


def test_concat(golden):
    g = golden["ops"]
    y = np.concatenate([T(g, "concat_input_x0"), T(g, "concat_input_x1")], axis=1)
    assert sse(y, T(g, "concat_output")) <= 1e-4


def test_batchnorm_inference(golden):
    g = golden["ops"]
    y = ref.bn_infer(T(g, "batchnorm_input_x"), T(g, "batchnorm_input_s"), T(g, "batchnorm_input_b"),
                     T(g, "batchnorm_input_m"), T(g, "batchnorm_input_v"), eps=1e-5)
    assert sse(y, T(g, "batchnorm_output")) <= 1e-4


@pytest.mark.parametrize("bypass", [True, False])
def test_resnode(golden, bypass):
    """conv1x1 -> batchnorm(train) -> [sum with x] -> relu, then backprop of `grad`
    (test/test_resnode.cpp:203-250).  The no-bypass fixtures were produced in fp16, so the
    fp32 oracle sits ~2e-5 SSE away from them; still inside the reference's 1e-4."""
    g = golden["resnode"]
    x = T(g, "conv_input_x")
    w = T(g, "conv_input_w")  # 32 values listed for dims {4,4,1,1}: the loader uses the first 16
    s, b = T(g, "batchnorm_input_s"), T(g, "batchnorm_input_b")
    dy = T(g, "grad")
    c = ref.conv2d_fwd(x, w)
    bn, sm, sv, _, _ = ref.bn_train_fwd(c, s, b, eps=1e-5)
    pre = bn + x if bypass else bn
    y = ref.act_fwd(pre)
    exp_y = T(g, "expected_y_with_bypass" if bypass else "expected_y_no_bypass")
    assert sse(y, exp_y) <= 1e-4
    dpre = ref.act_bwd(pre, y, dy)
    dbn, ds, db = ref.bn_bwd(c, dpre, s, sm, sv)
    dx = ref.conv2d_bwd_data(dbn, w, x.shape)
    if bypass:
        dx = dx + dpre
    exp_dx = T(g, "expected_dx_with_bypass" if bypass else "expected_dx_no_bypass")
    assert sse(dx, exp_dx) <= 1e-4
