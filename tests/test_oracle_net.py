"""Pins oracle/net.py, the whole-network checker every network-level GPU test and smoke() compare against.

OracleNet's composition rules (the order of operators per node, gradient fan-in, the loss_scale/N factor of the
classifier, batch-norm running statistics, Adam over all parameters for t > 1, the loss-scale rule) are compared
with an independent statement of the same network: torch-CPU autograd in double precision for forward, every
parameter gradient and the running statistics, and a numpy Adam written from the reference kernel's formula
(src/cuda/cuda_kernels.cu:159-230, bias terms src/cuda/cuda_optimizer.cpp:79-80) for the updates.
A mistake in the oracle's composition (a dropped fan-in term, a wrong scale, a stale bias term) fails here,
on the CPU, before any GPU test trusts it.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ref
from oracle.net import OracleNet
from saga_amd import api as S
from saga_amd import networks as N

B1, B2, EPS = 0.9, 0.999, 1e-8


def tiny_net(dtype, batch=4, seed=11):
    """One of every node kind OracleNet handles: strided conv + bias, batch norm, a tensor with two consumers
    (gradient fan-in), sum, relu, padded max pooling, transposed conv + bias, concat, padded average
    pooling, global average pooling, fc + bias."""
    net = N.Net("tiny", batch, (3, 12, 12), 5, dtype)
    b = N.Builder(net, seed)
    # (a bias directly in front of a batch norm has a zero gradient: the relu / the padded 3x3 keep them alive)
    c1 = b.conv(net.input, "c1", 8, 3, 2, 1, bias=True)            # 8 x 6 x 6
    r1 = b.bn(b.relu(c1), "bn1")
    b2 = b.bn(b.conv(r1, "c2", 8, 3, 1, 1), "bn2")
    r2 = b.relu(b.sum(b2, r1))                                      # r1 feeds c2 and the sum
    mp = b.pool("maxpool", r2, 3, 2, 1)                             # 8 x 3 x 3
    up = b.conv(mp, "up", 6, 2, 2, 0, bias=True, transpose=True)   # 6 x 6 x 6
    cat = b.concat([r2, up])                                        # 14 x 6 x 6, r2 has two consumers too
    c3 = b.relu(b.bn(b.conv(cat, "c3", 10, 3, 1, 1), "bn3"))
    ap = b.pool("avgpool", c3, 3, 1, 1)                             # divisor counts the padding
    gp = b.pool("avgpool", ap, global_=True)
    net.output = b.fc(gp, "fc", 5)
    # parameters away from their trivial initial values, so that every term of every gradient is exercised
    for k in list(net.params):
        if k.endswith(("-bt", "-b")) and not k.startswith("bn"):
            net.params[k] = (b.rng.standard_normal(net.params[k].shape) * 0.2).astype(np.float32)
        elif k.endswith("-s"):
            net.params[k] = b.rng.uniform(0.5, 1.5, net.params[k].shape).astype(np.float32)
        elif k.startswith("bn") and k.endswith("-b"):
            net.params[k] = (b.rng.standard_normal(net.params[k].shape) * 0.3).astype(np.float32)
        elif k.endswith("-m"):
            net.params[k] = (b.rng.standard_normal(net.params[k].shape) * 0.1).astype(np.float32)
        elif k.endswith("-v"):
            net.params[k] = b.rng.uniform(0.5, 1.5, net.params[k].shape).astype(np.float32)
    return net


class TorchNet:
    """The same node list in torch double; parameters are leaf tensors named as in the description."""

    def __init__(self, net, params=None, expavg=0.1):
        self.net, self.expavg = net, expavg
        src = net.params if params is None else params
        self.p = {k: torch.tensor(np.asarray(v, np.float64)) for k, v in src.items()}
        for k in net.trainable:
            self.p[k].requires_grad_(True)

    def forward(self, x, training):
        a = {self.net.input: torch.tensor(np.asarray(x, np.float64))}
        get = lambda n: a[n] if n in a else self.p[n]
        for node in self.net.nodes:
            ty, i, at, out = node["type"], node["in"], node["attrs"], node["out"]
            if ty == "conv":
                bias = get(i["b"]).reshape(-1) if "b" in i else None
                if at.get("transpose"):
                    y = F.conv_transpose2d(get(i["x"]), get(i["w"]), bias, at.get("stride", 1), at.get("pad", 0),
                                           at.get("outputpad", 0))
                else:
                    y = F.conv2d(get(i["x"]), get(i["w"]), bias, at.get("stride", 1), at.get("pad", 0))
            elif ty == "batchnorm":
                m, v = self.p[i["m"]].reshape(-1), self.p[i["v"]].reshape(-1)  # updated in place when training
                y = F.batch_norm(get(i["x"]), m, v, get(i["s"]).reshape(-1), get(i["b"]).reshape(-1), training,
                                 self.expavg, 1e-5)
                if training:
                    self.p[i["m"]], self.p[i["v"]] = m.reshape(1, -1), v.reshape(1, -1)
            elif ty == "relu":
                y = F.relu(get(i["x"]))
            elif ty == "maxpool":
                x_ = get(i["x"])
                k = x_.shape[2] if at.get("global") else at.get("size", 1)
                y = F.max_pool2d(x_, k, at.get("stride", 1), at.get("pad", 0))
            elif ty == "avgpool":
                x_ = get(i["x"])
                k = x_.shape[2] if at.get("global") else at.get("size", 1)
                y = F.avg_pool2d(x_, k, at.get("stride", 1), at.get("pad", 0), count_include_pad=True)
            elif ty == "sum":
                y = get(i["x0"]) + get(i["x1"])
            elif ty == "concat":
                y = torch.cat([get(i[f"x{j}"]) for j in range(len(i))], dim=at.get("axis", 1))
            elif ty == "fc":
                w = get(i["w"])
                y = get(i["x"]).flatten(1) @ (w.T if at.get("transW") else w)
                if "b" in i:
                    y = y + get(i["b"]).reshape(1, -1)
            elif ty == "reshape":
                y = get(i["x"]).reshape([int(v) for v in at["shape"]])
            elif ty == "loss":
                y = get(i["x"])
            else:
                raise NotImplementedError(ty)
            a[out] = y
        self.acts = a
        return a[self.net.output]

    def grads(self, x, labels, scale=1.0):
        """d(scale * mean cross entropy)/d(parameter) for every trainable parameter; logits; per-sample loss."""
        for k in self.net.trainable:
            self.p[k].grad = None
        logits = self.forward(x, True)
        per_sample = F.cross_entropy(logits, torch.tensor(labels.reshape(-1).astype(np.int64)), reduction="none")
        (per_sample.mean() * scale).backward()
        return ({k: self.p[k].grad.numpy().copy() for k in self.net.trainable}, logits.detach().numpy(),
                per_sample.detach().numpy())


    def l2_grads(self, x, scale=1.0):
        """d(scale * strength / (2 N) * sum (y - target)^2)/d(parameter) for a network ending in an L2 loss node,
        whose own gradient is then (y - target) * strength / N * scale; returns (gradients, y)."""
        for k in self.net.trainable:
            self.p[k].grad = None
        y = self.forward(x, True)
        node = [n for n in self.net.nodes if n["type"] == "loss"][0]
        r = y - self.p[node["in"]["target"]]
        (r.pow(2).sum() * (0.5 * node["attrs"].get("strength", 1.0) / y.shape[0] * scale)).backward()
        return {k: self.p[k].grad.numpy().copy() for k in self.net.trainable}, y.detach().numpy()


def worst(got, want):
    """per-tensor relative max-abs error, the measure the parity bars are stated in"""
    want = np.asarray(want, np.float64)
    return float(np.abs(np.asarray(got, np.float64).reshape(want.shape) - want).max()) / max(float(np.abs(want).max()),
                                                                                          1e-30)


def batch(net, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((net.batch,) + tuple(net.in_shape)).astype(np.float32)
    labels = rng.integers(0, net.classes, (net.batch, 1)).astype(np.int32)
    return x, labels


def test_inference_forward_against_torch_double():
    net = tiny_net(S.FLOAT)
    x, _ = batch(net, 1)
    got = OracleNet(net).forward(x, training=False)
    want = TorchNet(net).forward(x, False).detach().numpy()
    e = worst(got, want)
    print(f"inference logits: {e:.2e}")
    assert e <= 2e-6
    assert np.array_equal(OracleNet(net).predict(x), want.argmax(1))


def test_training_forward_backward_and_running_stats_against_torch_double():
    net = tiny_net(S.FLOAT)
    x, labels = batch(net, 2)
    o = OracleNet(net, bn_expavg=0.1)
    o.forward(x, training=True)
    grads, loss, pred = o.backward(labels)
    t = TorchNet(net)
    tg, tlogits, tloss = t.grads(x, labels)
    errs = {"logits": worst(o.acts[net.output], tlogits), "loss": worst(loss, tloss)}
    for name in net.nodes:
        errs["act " + name["out"]] = worst(o.acts[name["out"]], t.acts[name["out"]].detach().numpy())
    assert set(grads) == set(net.trainable)
    for k in net.trainable:
        errs["d " + k] = worst(grads[k], tg[k])
    for k in net.params:
        if k.endswith(("-m", "-v")):
            errs["running " + k] = worst(o.p[k], t.p[k].detach().numpy())
    print({k: f"{v:.1e}" for k, v in errs.items()})
    bad = {k: v for k, v in errs.items() if v > 2e-5}
    assert not bad, bad
    assert np.array_equal(pred, tlogits.argmax(1))


@pytest.mark.parametrize("loss_scale", [4.0, 1024.0])
def test_half_network_gradient_scale_is_loss_scale_over_n(loss_scale, monkeypatch):
    """fp16 programs multiply the classifier's gradient by loss_scale / N (src/cuda/cuda_dnn.cpp:1297-1315).
    With the fp16 rounding of stored tensors switched off the oracle must equal autograd of
    loss_scale * mean cross-entropy."""
    monkeypatch.setattr(ref, "round_half", lambda a: np.asarray(a, np.float32))
    net = tiny_net(S.HALF)
    x, labels = batch(net, 3)
    o = OracleNet(net, loss_scale=loss_scale)
    assert o.half
    o.forward(x, training=True)
    grads, loss, _ = o.backward(labels)
    tg, _, tloss = TorchNet(net).grads(x, labels, scale=loss_scale)
    errs = {k: worst(grads[k], tg[k]) for k in net.trainable}
    errs["loss"] = worst(loss, tloss)  # the per-sample loss is not scaled
    bad = {k: v for k, v in errs.items() if v > 2e-5}
    assert not bad, bad


def test_default_loss_scale_is_the_batch_size():
    # src/cuda/cuda_common.cpp:339-353
    assert OracleNet(tiny_net(S.HALF, batch=6)).loss_scale == 6.0


def numpy_adam(w, g, m, v, t, lr, lam):
    """src/cuda/cuda_kernels.cu:159-189 in float32, bias terms as src/cuda/cuda_optimizer.cpp:79-80."""
    f = np.float32
    b1t, b2t = f(1.0 / (1.0 - B1 ** t)), f(1.0 / (1.0 - B2 ** t))
    m[:] = f(B1) * m + (f(1.0) - f(B1)) * g
    v[:] = f(B2) * v + (f(1.0) - f(B2)) * g * g
    w[:] = w - f(lr) * (m * b1t) / np.sqrt(v * b2t + f(EPS)) - f(lr) * f(lam) * w


def test_five_fp32_train_steps_against_autograd_plus_numpy_adam():
    """Five steps on changing batches: gradients from torch double autograd at the oracle's own current
    parameters, the update from the numpy Adam above; pins Adam for t > 1, the weight decay term and the
    order forward -> backward -> update."""
    net = tiny_net(S.FLOAT)
    lr, lam = 1e-2, 0.01
    o = OracleNet(net, lr=lr, l2=lam)
    w = {k: np.array(net.params[k], np.float32).reshape(-1) for k in net.trainable}
    m = {k: np.zeros_like(w[k]) for k in net.trainable}
    v = {k: np.zeros_like(w[k]) for k in net.trainable}
    run = {k: np.array(net.params[k], np.float64) for k in net.params if k.endswith(("-m", "-v"))}
    worst_w = worst_g = 0.0
    for step in range(1, 6):
        x, labels = batch(net, 100 + step)
        params = {k: (w[k].reshape(net.params[k].shape) if k in w else run[k]) for k in net.params}
        t = TorchNet(net, params)
        tg, _, _ = t.grads(x, labels)
        for k in run:
            run[k] = t.p[k].detach().numpy()
        _, _, grads, flags = o.train_step(x, labels)
        assert not flags.any()
        for k in net.trainable:
            worst_g = max(worst_g, worst(grads[k], tg[k]))
            numpy_adam(w[k], tg[k].astype(np.float32).reshape(-1), m[k], v[k], step, lr, lam)
            e = worst(o.p[k], w[k])
            worst_w = max(worst_w, e)
            assert e <= 1e-5, (step, k, e)
        assert o.t == step
    print(f"5 steps: worst gradient error {worst_g:.1e}, worst weight error {worst_w:.1e}")
    assert worst_g <= 5e-5
    # the weights moved by much more than the agreement asked for
    moved = max(worst(w[k], np.array(net.params[k]).reshape(-1)) for k in net.trainable)
    assert moved > 1e-2


def numpy_adam_mixed(w16, g16, m, v, c, t, lr, scale, lam):
    """src/cuda/cuda_kernels.cu:191-230: fp16 gradient bits tested for exponent >= 0x1e (range) and all ones
    (inf / nan: the element is skipped); fp32 master copy c; the fp16 weight is the rounded master."""
    f = np.float32
    flags = np.zeros(3, np.uint32)
    bits = g16.view(np.uint16)
    big = (bits & 0x7800) == 0x7800
    nonfinite = (bits & 0x7C00) == 0x7C00
    if big.any():
        flags[0] = 1
    if (nonfinite & ((bits & 0x3FF) != 0)).any():
        flags[2] = 1
    if (nonfinite & ((bits & 0x3FF) == 0)).any():
        flags[1] = 1
    ok = ~nonfinite
    b1t, b2t = f(1.0 / (1.0 - B1 ** t)), f(1.0 / (1.0 - B2 ** t))
    dw = g16.astype(np.float32)[ok] * (f(1.0) / f(scale))
    mm = f(B1) * m[ok] + (f(1.0) - f(B1)) * dw
    vv = f(B2) * v[ok] + (f(1.0) - f(B2)) * dw * dw
    cc = c[ok]
    cc = cc - f(lr) * (mm * b1t) / np.sqrt(vv * b2t + f(EPS)) - f(lr) * f(lam) * cc
    m[ok], v[ok], c[ok] = mm, vv, cc
    w16[ok] = cc.astype(np.float16)
    return flags


def test_mixed_precision_steps_overflow_skips_and_loss_scale_rule():
    """An fp16 network driven with a loss scale large enough that the first steps overflow: the oracle's
    adam() must skip exactly the non-finite elements, halve the scale while any gradient is non-finite
    and grow it by 1.02 afterwards (src/cuda/cuda_program.cpp:295-307)."""
    net = tiny_net(S.HALF)
    lr = 1e-3
    o = OracleNet(net, lr=lr, loss_scale=2.0 ** 22)
    st = {}
    for k in net.trainable:
        w32 = o.p[k].reshape(-1).astype(np.float32)
        st[k] = dict(w16=w32.astype(np.float16), m=np.zeros_like(w32), v=np.zeros_like(w32), c=w32.copy())
    scale = np.float32(2.0 ** 22)
    halved = grown = 0
    for step in range(1, 9):
        x, labels = batch(net, 200 + step)
        before = {k: o.p[k].copy() for k in net.trainable}
        _, _, grads, flags = o.train_step(x, labels)
        want_flags = np.zeros(3, np.uint32)
        for k in net.trainable:
            s = st[k]
            if o._is_bn_param(k):
                g = np.asarray(grads[k], np.float32).reshape(-1)
                if not np.isfinite(g).all():
                    # fp32 Adam: non-finite elements are skipped and flagged (src/cuda/cuda_kernels.cu:168-175)
                    want_flags[1] |= np.isinf(g).any()
                    want_flags[2] |= np.isnan(g).any()
                ok = np.isfinite(g)
                ww, mm, vv = s["c"][ok], s["m"][ok], s["v"][ok]
                numpy_adam(ww, g[ok], mm, vv, step, lr, 0.0)
                s["c"][ok], s["m"][ok], s["v"][ok] = ww, mm, vv
                e = worst(o.p[k], s["c"])
            else:
                with np.errstate(over="ignore"):
                    g16 = np.asarray(grads[k], np.float32).reshape(-1).astype(np.float16)
                want_flags |= numpy_adam_mixed(s["w16"], g16, s["m"], s["v"], s["c"], step, lr, scale, 0.0)
                e = worst(o.p[k], s["w16"].astype(np.float32))
                skipped = ~np.isfinite(g16.astype(np.float32))
                if skipped.any():  # skipped elements keep their weight
                    assert np.array_equal(o.p[k].reshape(-1)[skipped], before[k].reshape(-1)[skipped])
            assert e <= 1e-5, (step, k, e)
        assert np.array_equal(flags.astype(bool), want_flags.astype(bool)), (step, flags, want_flags)
        if want_flags[1] or want_flags[2]:
            scale = np.float32(float(scale) * 0.5)
            halved += 1
        else:
            scale = np.float32(float(scale) * 1.02)
            grown += 1
        assert o.loss_scale == scale, (step, o.loss_scale, scale)
    assert halved >= 2 and grown >= 2, (halved, grown)


def test_per_pixel_softmax_head_against_torch():
    """The `softmax` node (over the channels at every pixel, inference only) on top of a convolution."""
    net = N.Net("head", 2, (4, 6, 5), 3, S.FLOAT)
    b = N.Builder(net, 5)
    net.output = b.unary("softmax", b.conv(net.input, "c", 3, 1, 1, 0, bias=True))
    net.params["c-bt"] = (b.rng.standard_normal((1, 3)) * 0.5).astype(np.float32)
    x, _ = batch(net, 9)
    got = OracleNet(net).forward(x, training=False)
    w = torch.tensor(net.params["c-w"].astype(np.float64))
    want = torch.softmax(F.conv2d(torch.tensor(x.astype(np.float64)), w, torch.tensor(net.params["c-bt"].astype(np.float64)).reshape(-1)), 1)
    assert worst(got, want.numpy()) <= 1e-6
    np.testing.assert_allclose(got.sum(1), 1.0, atol=1e-6)


def off_zero(net, rng):
    for k in net.trainable:
        if k.endswith(("-b", "-bt")):
            net.params[k] = (rng.standard_normal(net.params[k].shape) * 0.2).astype(np.float32)


@pytest.mark.parametrize("loss_scale", [1.0, 8.0])
def test_conv_harness_graph_loss_reshape_transw_against_torch_double(loss_scale):
    """The graph of the reference's `conv` command (test/test_conv.cpp:96-140): the three node kinds the
    other networks do not use - fc with transposed weights, reshape, the L2 loss node as the start of the
    backward pass - against autograd of strength / (2 N) * sum (y - target)^2 times the loss scale, which
    the node applies in fp32 programs too (src/cuda/cuda_dnn.cpp:1433-1443)."""
    net, x = N.conv_harness(S.FLOAT)
    off_zero(net, np.random.default_rng(3))
    [n for n in net.nodes if n["type"] == "loss"][0]["attrs"]["strength"] = 1.5
    o = OracleNet(net, loss_scale=loss_scale)
    assert OracleNet(net).loss_scale == 1.0  # program batch size 1 with two rows in the tensors
    o.forward(x, training=True)
    grads, mmss, pred = o.backward()
    assert pred is None and set(grads) == set(net.trainable)
    t = TorchNet(net)
    tg, ty = t.l2_grads(x, loss_scale)
    errs = {"y": worst(o.acts[net.output], ty), "loss y": worst(o.acts[net.loss], ty)}
    for n in net.nodes:
        errs["act " + n["out"]] = worst(o.acts[n["out"]], t.acts[n["out"]].detach().numpy())
    for k in net.trainable:
        errs["d " + k] = worst(grads[k], tg[k])
    r = (ty - x.astype(np.float64)).reshape(2, -1)
    want_mmss = np.stack([np.minimum(r.min(1), 0), np.maximum(r.max(1), 0), r.mean(1), (r * r).mean(1)], 1)
    errs["mmss"] = worst(mmss, want_mmss)
    print({k: f"{v:.1e}" for k, v in errs.items()})
    bad = {k: v for k, v in errs.items() if v > 2e-6}
    assert not bad, bad
    # the transposed fc weight really is [out, in]
    assert net.params["fc1-w"].shape == (20, 20) and net.params["node1-w"].shape == (5, 1, 3, 3)
    assert net.params["node2-w"].shape == (5, 1, 3, 3)


def test_conv_harness_graph_trains_like_autograd_plus_numpy_adam():
    """Twenty fp32 steps of the conv harness graph: oracle weights against torch double gradients fed to the
    numpy Adam, and the mean squared error falls."""
    net, x = N.conv_harness(S.FLOAT)
    lr = 1e-2
    o = OracleNet(net, lr=lr)
    w = {k: np.array(net.params[k], np.float32).reshape(-1) for k in net.trainable}
    m = {k: np.zeros_like(w[k]) for k in net.trainable}
    v = {k: np.zeros_like(w[k]) for k in net.trainable}
    mse = []
    for step in range(1, 21):
        params = {k: (w[k].reshape(net.params[k].shape) if k in w else net.params[k]) for k in net.params}
        tg, _ = TorchNet(net, params).l2_grads(x)
        mmss, _, grads, flags = o.train_step(x)
        mse.append(float(mmss[:, 3].mean()))
        for k in net.trainable:
            numpy_adam(w[k], tg[k].astype(np.float32).reshape(-1), m[k], v[k], step, lr, 0.0)
            assert worst(o.p[k], w[k]) <= 1e-5, (step, k)
    assert mse[-1] < 0.8 * mse[0], mse
