"""Pins for the parts of the oracle that no reference-held vector covers: identities the
mathematics fixes (adjoints, closed forms, conservation laws, finite differences) and library
routines the special cases reduce to (torch CPU conv / pooling / batch-norm / cross-entropy)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ref

rng = np.random.default_rng(7)


def rnd(*shape):
    return rng.standard_normal(shape).astype(np.float32)


CONV_CASES = [
    # N, C, H, W, K, R, pad, stride, group[, dilation]
    (2, 8, 9, 9, 6, 3, 1, 1, 1),
    (2, 6, 11, 10, 4, 3, 1, 2, 1),
    (1, 3, 15, 15, 5, 7, 3, 2, 1),
    (2, 8, 8, 8, 8, 1, 0, 2, 1),
    (2, 8, 7, 7, 4, 3, 0, 1, 2),
    (1, 4, 6, 6, 4, 5, 2, 1, 1),
    # dilated filters (shape rule src/node.cpp:50, 66-75): the GPU operator tests take the oracle's word for these
    (2, 5, 11, 12, 4, 3, 2, 1, 1, 2),
    (2, 4, 13, 13, 6, 3, 3, 2, 1, 3),
    (1, 6, 12, 10, 4, 3, 1, 1, 2, 2),
    (2, 3, 14, 14, 4, 5, 4, 2, 1, 2),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_against_torch_and_adjoint(case):
    N, C, H, W, K, R, pad, stride, group = case[:9]
    dil = case[9] if len(case) > 9 else 1
    x, w = rnd(N, C, H, W), rnd(K, C // group, R, R)
    y = ref.conv2d_fwd(x, w, pad, stride, dil, group)
    yt = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), None, stride, pad, dil, group)
    assert y.shape == tuple(yt.shape)
    np.testing.assert_allclose(y, yt.numpy(), rtol=1e-5, atol=1e-5)
    dy = rnd(*y.shape)
    dx = ref.conv2d_bwd_data(dy, w, x.shape, pad, stride, dil, group)
    dw = ref.conv2d_bwd_filter(x, dy, w.shape, pad, stride, dil, group)
    # <conv(x,w),dy> = <x,bwd_data(dy,w)> = <w,bwd_filter(x,dy)>
    lhs = float((y.astype(np.float64) * dy).sum())
    assert abs(lhs - float((x.astype(np.float64) * dx).sum())) <= 1e-4 * max(1, abs(lhs))
    assert abs(lhs - float((w.astype(np.float64) * dw).sum())) <= 1e-4 * max(1, abs(lhs))
    xt = torch.from_numpy(x).double().requires_grad_()
    wt = torch.from_numpy(w).double().requires_grad_()
    F.conv2d(xt, wt, None, stride, pad, dil, group).backward(torch.from_numpy(dy).double())
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-5, atol=1e-5)
    # beta = 1 accumulates
    y2 = ref.conv2d_fwd(x, w, pad, stride, dil, group, y=y, beta=1.0)
    np.testing.assert_allclose(y2, 2 * y, rtol=1e-6, atol=1e-6)


def test_transposed_conv_is_bwd_data():
    # src/cuda/cuda_dnn.cpp:542-574 ; weight dims [Cx, Cy, R, S] (src/node.cpp:99-110)
    x, w = rnd(2, 6, 5, 5), rnd(6, 4, 2, 2)
    Ho = ref.tconv_out(5, 2, 0, 2)
    y = ref.conv2d_bwd_data(x, w, (2, 4, Ho, Ho), 0, 2)
    yt = F.conv_transpose2d(torch.from_numpy(x), torch.from_numpy(w), None, 2, 0)
    np.testing.assert_allclose(y, yt.numpy(), rtol=1e-5, atol=1e-5)
    x, w = rnd(1, 4, 4, 4), rnd(4, 3, 3, 3)
    Ho = ref.tconv_out(4, 3, 1, 2, 1)
    y = ref.conv2d_bwd_data(x, w, (1, 3, Ho, Ho), 1, 2)
    yt = F.conv_transpose2d(torch.from_numpy(x), torch.from_numpy(w), None, 2, 1, output_padding=1)
    np.testing.assert_allclose(y, yt.numpy(), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("transW", [False, True])
def test_fc_adjoint(transW):
    x = rnd(5, 7)
    w = rnd(3, 7) if transW else rnd(7, 3)
    y = ref.fc_fwd(x, w, transW)
    np.testing.assert_allclose(y, x @ (w.T if transW else w), rtol=1e-5, atol=1e-5)
    dy = rnd(*y.shape)
    np.testing.assert_allclose(ref.fc_bwd_x(dy, w, transW), dy @ (w if transW else w.T), rtol=1e-5, atol=1e-5)
    dw = ref.fc_bwd_w(x, dy, transW)
    np.testing.assert_allclose(dw, (dy.T @ x) if transW else (x.T @ dy), rtol=1e-5, atol=1e-5)


def test_bias_bwd():
    dy = rnd(3, 4, 5, 5)
    np.testing.assert_allclose(ref.bias_bwd(dy), dy.sum((0, 2, 3)), rtol=1e-5, atol=1e-5)


def test_bn_train_matches_torch_and_running_stats():
    x, s, b = rnd(4, 5, 3, 3), rnd(5), rnd(5)
    rm, rv = rnd(5), np.abs(rnd(5)) + 0.5
    y, sm, sv, nrm, nrv = ref.bn_train_fwd(x, s, b, rm, rv, 1e-5, 0.1)
    trm, trv = torch.from_numpy(rm.copy()), torch.from_numpy(rv.copy())
    xt = torch.from_numpy(x).requires_grad_()
    st, bt = torch.from_numpy(s).requires_grad_(), torch.from_numpy(b).requires_grad_()
    yt = F.batch_norm(xt, trm, trv, st, bt, True, 0.1, 1e-5)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(nrm, trm.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(nrv, trv.numpy(), rtol=1e-5, atol=1e-6)  # unbiased variance
    np.testing.assert_allclose(sm, x.mean((0, 2, 3)), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(sv, 1 / np.sqrt(x.var((0, 2, 3)) + 1e-5), rtol=1e-5)
    dy = rnd(*x.shape)
    yt.backward(torch.from_numpy(dy))
    dx, ds, db = ref.bn_bwd(x, dy, s, sm, sv)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(ds, st.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("k,pad,stride", [(2, 0, 2), (3, 1, 2), (3, 1, 1), (7, 0, 1)])
def test_pooling_against_torch(k, pad, stride):
    x = rnd(2, 3, 7, 7)
    y, idx = ref.maxpool_fwd(x, k, pad, stride, with_idx=True)
    yt, it = F.max_pool2d(torch.from_numpy(x), k, stride, pad, return_indices=True)
    np.testing.assert_array_equal(y, yt.numpy())
    np.testing.assert_array_equal(idx, it.numpy().astype(np.int32))
    a = ref.avgpool_fwd(x, k, pad, stride)
    at = F.avg_pool2d(torch.from_numpy(x), k, stride, pad, count_include_pad=True)
    np.testing.assert_allclose(a, at.numpy(), rtol=1e-5, atol=1e-6)
    dy = rnd(*y.shape)
    dx = ref.maxpool_bwd(x, dy, k, pad, stride)
    assert abs(dx.sum() - dy.sum()) < 1e-3  # max-pool backward conserves the gradient mass
    xt = torch.from_numpy(x).requires_grad_()
    F.max_pool2d(xt, k, stride, pad).backward(torch.from_numpy(dy))
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-5, atol=1e-6)
    xt = torch.from_numpy(x).requires_grad_()
    F.avg_pool2d(xt, k, stride, pad, count_include_pad=True).backward(torch.from_numpy(dy))
    np.testing.assert_allclose(ref.avgpool_bwd(dy, x.shape, k, pad, stride), xt.grad.numpy(), rtol=1e-5, atol=1e-6)


def test_maxpool_tie_takes_first_index():
    x = np.zeros((1, 1, 4, 4), np.float32)
    y, idx = ref.maxpool_fwd(x, 2, 0, 2, with_idx=True)
    np.testing.assert_array_equal(idx.reshape(-1), [0, 2, 8, 10])


@pytest.mark.parametrize("mode", ["relu", "sigmoid", "tanh", "swish"])
def test_activation_derivative(mode):
    x = rnd(200).astype(np.float64)
    x = x[np.abs(x) > 1e-2].astype(np.float32)
    y = ref.act_fwd(x, mode)
    dx = ref.act_bwd(x, y, np.ones_like(x), mode)
    h = 1e-3
    fd = (ref.act_fwd(x + h, mode).astype(np.float64) - ref.act_fwd(x - h, mode)) / (2 * h)
    np.testing.assert_allclose(dx, fd, rtol=2e-2, atol=2e-3)


def test_relu_propagates_nan():
    assert np.isnan(ref.act_fwd(np.array([np.nan], np.float32))[0])


def test_catclassifier():
    x = rnd(6, 11)
    x[2, 3] = x[2, 7] = x[2].max() + 1  # tie: first index wins (strict '>')
    pred = ref.catclassifier_fwd(x)
    np.testing.assert_array_equal(pred, np.argmax(x, axis=1))
    assert pred[2] == 3
    label = rng.integers(0, 11, 6).astype(np.int32)
    dx, loss = ref.catclassifier_bwd(x, pred, label, 1.0 / 6)
    xt = torch.from_numpy(x).double().requires_grad_()
    lt = F.cross_entropy(xt, torch.from_numpy(label).long(), reduction="none")
    np.testing.assert_allclose(loss, lt.detach().numpy(), rtol=1e-5, atol=1e-6)
    lt.mean().backward()
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(dx.sum(1), 0, atol=1e-6)  # softmax gradient rows sum to zero


def test_loss_and_stats():
    # hand-computed: v = [1, -2, 3] and [0.5, 0.5, 4]
    x = np.array([[2.0, 0.0, 4.0], [1.0, 2.5, 4.0]], np.float32)
    t = np.array([[1.0, 2.0, 1.0], [0.5, 2.0, 0.0]], np.float32)
    dx, mmss = ref.loss_bwd(x, t, 0.5)
    np.testing.assert_allclose(dx, [[0.5, -1.0, 1.5], [0.25, 0.25, 2.0]])
    np.testing.assert_allclose(mmss[0], [-2.0, 3.0, 2.0 / 3, 14.0 / 3], rtol=1e-6)
    # all residuals positive: the minimum is the reference's padded zero, not 0.5
    np.testing.assert_allclose(mmss[1], [0.0, 4.0, 5.0 / 3, 16.5 / 3], rtol=1e-6)
    a = rnd(3, 4, 5, 6)
    b = rnd(3, 4, 5, 6)
    dx, mmss = ref.loss_bwd(a, b, 0.25)
    v = (a - b).reshape(3, -1)
    np.testing.assert_allclose(dx.reshape(3, -1), v * 0.25, rtol=1e-6)
    np.testing.assert_allclose(mmss, np.stack([np.minimum(v.min(1), 0), np.maximum(v.max(1), 0), v.mean(1), (v * v).mean(1)], 1),
                               rtol=1e-5, atol=1e-6)
    st = ref.tensor_stats(a)
    np.testing.assert_allclose(st, [min(a.min(), 0), max(a.max(), 0), a.mean(), a.var()], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(ref.tensor_stats(np.abs(a) + 1)[0], 0.0)  # strictly positive data still report min 0


def test_softmax():
    x = rnd(2, 5, 3, 3)
    y = ref.softmax(x)
    np.testing.assert_allclose(y.sum(1), 1, rtol=1e-5)
    np.testing.assert_allclose(y, F.softmax(torch.from_numpy(x), 1).numpy(), rtol=1e-5, atol=1e-7)


def test_half_conversion_matches_numpy():
    bits = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    L = ref.lib()
    sel = bits[::7]
    f = np.array([L.so_half_to_float(int(b)) for b in sel], np.float32)
    want = sel.view(np.float16).astype(np.float32)
    nan = np.isnan(want)  # NaN payloads may be quieted in transit; only NaN-ness is compared
    assert np.isnan(f[nan]).all()
    np.testing.assert_array_equal(f[~nan].view(np.uint32), want[~nan].view(np.uint32))
    vals = np.concatenate([rnd(2000) * 10.0 ** rng.integers(-8, 6, 2000), [0.0, -0.0, 65504, 65520, 1e-8, np.inf]])
    vals = vals.astype(np.float32)
    got = np.array([L.so_float_to_half(float(v)) for v in vals], np.uint16)
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(got, vals.astype(np.float16).view(np.uint16))


def test_adam_first_step_closed_form():
    # t = 1: m_hat = g, v_hat = g^2 -> dw = -lr * g * rsqrt(g^2 + 1e-8) - lr*lambda*w
    w0, g = rnd(100), rnd(100)
    w, m, v = w0.copy(), np.zeros(100, np.float32), np.zeros(100, np.float32)
    flags = ref.adam_f32(w, g, m, v, 1, 1e-3, 0.01)
    exp = w0 - 1e-3 * g / np.sqrt(g.astype(np.float64) ** 2 + 1e-8) - 1e-3 * 0.01 * w0
    np.testing.assert_allclose(w, exp, rtol=1e-5, atol=1e-6)
    assert not flags.any()
    np.testing.assert_allclose(m, 0.1 * g, rtol=1e-6)
    np.testing.assert_allclose(v, 0.001 * g * g, rtol=1e-4)  # (1 - 0.999f) in float


def test_adam_nonfinite_skips_and_flags():
    w, g = np.ones(4, np.float32), np.array([1, np.inf, np.nan, 2], np.float32)
    m, v = np.zeros(4, np.float32), np.zeros(4, np.float32)
    flags = ref.adam_f32(w, g, m, v, 1, 0.1)
    assert list(flags) == [0, 1, 1]
    assert w[1] == 1 and w[2] == 1 and w[0] != 1 and w[3] != 1 and m[1] == 0


def test_adam_mixed_matches_f32_path_and_flags():
    w0 = rnd(64).astype(np.float16)
    g = (rnd(64) * 64).astype(np.float16)
    w16 = w0.view(np.uint16).copy()
    m, v, c = np.zeros(64, np.float32), np.zeros(64, np.float32), w0.astype(np.float32)
    flags = ref.adam_mixed(w16, g.view(np.uint16).copy(), m, v, c, 1, 1e-2, 64.0)
    wf, mf, vf = w0.astype(np.float32), np.zeros(64, np.float32), np.zeros(64, np.float32)
    ref.adam_f32(wf, g.astype(np.float32) / 64, mf, vf, 1, 1e-2)
    np.testing.assert_allclose(c, wf, rtol=1e-6, atol=1e-7)
    np.testing.assert_array_equal(w16, wf.astype(np.float16).view(np.uint16))
    assert not flags.any()
    gbad = np.array([0x7800, 0x7c00, 0x7e00, 0x3c00], np.uint16)  # big, inf, nan, 1.0
    w16 = np.zeros(4, np.uint16)
    m, v, c = (np.zeros(4, np.float32) for _ in range(3))
    flags = ref.adam_mixed(w16, gbad, m, v, c, 1, 1e-2, 1.0)
    assert list(flags) == [1, 1, 1]
    assert c[1] == 0 and c[2] == 0 and c[0] != 0 and c[3] != 0


def test_loss_scale_rule():
    # src/cuda/cuda_program.cpp:295-302: inf/nan halves; range>1 (never on one GPU) x0.9; else x1.02
    assert ref.loss_scale_update(1024, [0, 1, 0]) == 512
    assert ref.loss_scale_update(1024, [1, 0, 1]) == 512
    assert ref.loss_scale_update(1000, [1, 0, 0]) == np.float32(1020.0)
    assert ref.loss_scale_update(1000, [2, 0, 0]) == np.float32(900.0)


def test_spatial_transform_against_torch_and_closed_forms():
    """Pins so_spatial_transform: (1) torch's affine_grid + grid_sample with align_corners=True and
    zero padding is the same published rule, implemented independently; (2) the identity matrix
    on an equal-sized output is a copy; (3) resizing a linear ramp with the identity matrix gives
    the same ramp sampled at the new pixel centres; (4) a shift of one input pixel moves the image
    and fills with zeros."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, 2, 7, 9)).astype(np.float32)
    theta = np.tile(np.array([[1, 0, 0], [0, 1, 0]], np.float32), (3, 1, 1))
    theta += rng.normal(0, 0.25, theta.shape).astype(np.float32)  # rotations, zooms, shifts beyond the border
    for oh, ow in [(7, 9), (12, 5), (20, 31)]:
        grid = F.affine_grid(torch.from_numpy(theta), (3, 2, oh, ow), align_corners=True)
        want = F.grid_sample(torch.from_numpy(x), grid, mode="bilinear", padding_mode="zeros", align_corners=True)
        np.testing.assert_allclose(ref.spatial_transform(x, theta, oh, ow), want.numpy(), atol=2e-5)  # torch keeps the grid in fp32
    ident = np.tile(np.array([[1, 0, 0], [0, 1, 0]], np.float32), (3, 1, 1))
    np.testing.assert_allclose(ref.spatial_transform(x, ident, 7, 9), x, atol=1e-6)
    ramp = np.broadcast_to(np.arange(8, dtype=np.float32), (1, 1, 4, 8)).copy()
    up = ref.spatial_transform(ramp, ident[:1], 4, 15)
    np.testing.assert_allclose(up[0, 0, 2], np.linspace(0, 7, 15), atol=1e-5)
    shift = ident[:1].copy()
    shift[0, 0, 2] = 2.0 / (9 - 1)  # one input pixel to the right in normalised units
    moved = ref.spatial_transform(x[:1], shift, 7, 9)
    np.testing.assert_allclose(moved[..., :-1], x[:1, ..., 1:], atol=1e-5)
    np.testing.assert_allclose(moved[..., -1], 0, atol=1e-5)
