"""Program-level behaviour of the hip engine that the known-answer harnesses do not reach:

 * the dynamic loss-scale controller's overflow branch (src/cuda/cuda_program.cpp:295-307, forced by the
   reference in test/test_mp.cpp:60-70 with targets beyond the fp16 range): scale x 0.5 while any gradient is
   inf / NaN, the optimizer skipping exactly the non-finite elements, flags cleared for the next step,
   x 1.02 afterwards - step by step against the CPU oracle network;
 * the `window` node (src/cuda/cuda_dnn.cpp:2549-2587): an alias of its input at an element offset;
 * anomaly detection (src/cuda/cuda_program.cpp:163-240) reporting a planted NaN.
"""
import numpy as np
import pytest

from oracle import ref
from oracle.net import OracleNet
from saga_amd import api as S
from saga_amd import networks as N
from tests.gpu_util import rel_err

pytestmark = pytest.mark.gpu


def mlp(batch, dtype, seed=21):
    """fc 24 -> 16 + bias, relu, fc 16 -> 10 + bias (the classifier head of a network, nothing else)."""
    net = N.Net("mlp", batch, (24,), 10, dtype)
    b = N.Builder(net, seed)
    net.output = b.fc(b.relu(b.fc(net.input, "fc1", 16)), "fc2", 10)
    return net


def test_loss_scale_overflow_branch_against_oracle():
    net = mlp(8, S.HALF)
    rng = np.random.default_rng(5)
    lr, scale0 = 1e-2, 2.0 ** 24
    ctx = S.Context()
    x0 = rng.standard_normal((8, 24)).astype(np.float16)
    g, t = N.build_graph(net, x0)
    p = ctx.create_program(g, 8, training=True, learning_rate=lr, initial_loss_scale=scale0)
    xin, labels_t = ctx.resolve(t[net.input]), ctx.resolve(t["labels"])
    names = list(net.trainable)
    dev_w = {k: ctx.resolve(t[k]) for k in names}
    dev_g = {k: ctx.resolve(t[k].grad()) for k in names}
    o = OracleNet(net, lr=lr, loss_scale=scale0)
    assert p.loss_scale() == scale0
    halved = grown = partial_skips = 0
    for step in range(14):
        x = rng.standard_normal((8, 24)).astype(np.float16)
        labels = rng.integers(0, 10, (8, 1)).astype(np.int32)
        xin.write(x)
        labels_t.write(labels)
        before = {k: dev_w[k].read().astype(np.float32) for k in names}
        scale_before = p.loss_scale()
        assert p.run(1) == 0
        _, _, ograds, oflags = o.train_step(x.astype(np.float32), labels)
        overflow = bool(oflags[1] or oflags[2])
        # the controller: identical float arithmetic on both sides
        assert p.loss_scale() == float(o.loss_scale), (step, p.loss_scale(), o.loss_scale, oflags)
        assert p.loss_scale() == float(np.float32(scale_before * (0.5 if overflow else 1.02)))
        halved += overflow
        grown += not overflow
        for k in names:
            got_g = dev_g[k].read().astype(np.float32)
            want_g = np.asarray(ograds[k], np.float32).reshape(got_g.shape)
            with np.errstate(over="ignore", invalid="ignore"):
                want_g16 = want_g.astype(np.float16).astype(np.float32)
            bad = ~np.isfinite(want_g16)
            # the same elements overflow on the device (inf and NaN both count as non-finite)
            assert np.array_equal(~np.isfinite(got_g), bad), (step, k)
            after = dev_w[k].read().astype(np.float32)
            # skipped: weight bit-identical to before the step; finite gradients: the weight follows the oracle
            assert np.array_equal(after[bad], before[k][bad]), (step, k, "a non-finite element was updated")
            if bad.any() and not bad.all():
                partial_skips += 1
            want_w = o.p[k].reshape(after.shape)
            e = rel_err(after, want_w)
            assert e <= 2e-3, (step, k, e)
            moved = np.abs(after - before[k])[~bad]
            if moved.size and np.abs(want_g16[~bad]).max() > 0:
                assert moved.max() > 0, (step, k, "no finite element moved")
    print(f"loss scale: {halved} halvings, {grown} growth steps, {partial_skips} partially skipped tensors, "
          f"final {p.loss_scale():.4g}")
    assert halved >= 3 and grown >= 3 and partial_skips >= 1


def test_loss_scale_reference_case_target_beyond_fp16():
    """test/test_mp.cpp: fp16 fc 1 -> 1 with weight 0.1 on x = 0.1 and an L2 loss against a target.  Target 2e4:
    finite gradient, the weight moves by the learning rate (Adam's first step), the scale grows.  Target 7e4 is
    inf in fp16: the gradient is -inf, the weight must not move and the scale halves."""
    for target, moves in ((2e4, True), (7e4, False)):
        ctx = S.Context()
        g = S.Graph()
        x = S.Tensor.from_numpy(np.array([[0.1]], np.float16))
        w = S.Tensor.from_numpy(np.array([[0.1]], np.float16))
        with np.errstate(over="ignore"):
            tgt = S.Tensor.from_numpy(np.array([[target]], np.float32).astype(np.float16))
        n = g.add_node("fc", {"x": x, "w": w}, {"outputs": 1, "bias": False}, "fc1")
        g.add_node("loss", {"x": n.y(), "target": tgt})
        p = ctx.create_program(g, 1, training=True, learning_rate=0.01)
        wl, dw = ctx.resolve(w), ctx.resolve(w.grad())
        s0 = p.loss_scale()
        assert s0 == 1.0  # the reference's default: the batch size (src/cuda/cuda_common.cpp:339-353)
        assert p.run(1) == 0
        got_w, got_dw = float(wl.read()[0, 0]), float(dw.read()[0, 0])
        if moves:
            assert np.isfinite(got_dw) and abs(got_dw - (-2e3)) <= 2.0   # dy = (0.01 - 2e4), dw = x * dy
            assert abs(got_w - 0.11) <= 1e-3
            assert p.loss_scale() == float(np.float32(1.02))
        else:
            assert np.isinf(got_dw)
            assert got_w == float(np.float16(0.1))
            assert p.loss_scale() == 0.5
            # the flags were cleared: a finite step follows with growth
            ctx.resolve(tgt).write(np.array([[1.0]], np.float16))
            assert p.run(1) == 0
            assert p.loss_scale() == float(np.float32(0.5 * 1.02))
            assert float(wl.read()[0, 0]) != float(np.float16(0.1))


@pytest.mark.parametrize("layout", [S.LAYOUT_NCHW, S.LAYOUT_NHWC])
@pytest.mark.parametrize("dt", [S.FLOAT, S.HALF])
def test_window_node_is_an_offset_alias(dt, layout):
    rng = np.random.default_rng(9)
    a = rng.standard_normal((2, 6, 7, 8)).astype(np.float16 if dt == S.HALF else np.float32)
    shape, off = [2, 3, 4, 5], [0, 2, 1, 3]
    want = np.maximum(a[:, 2:5, 1:5, 3:8].astype(np.float32) * 2.0, 0.0)
    ctx = S.Context()
    g = S.Graph()
    x = S.Tensor.from_numpy(a)
    n = g.add_node("sum", {"x0": x, "x1": x})          # a produced tensor: the window aliases device memory
    n = g.add_node("window", n, {"shape": shape, "offset": off})
    assert n.y().dims == shape
    n = g.add_node("relu", n)
    p = ctx.create_program(g, 2, training=False, tensor_layout=layout)
    y = ctx.resolve(n.y())
    assert p.run(1) == 0
    got = y.read().astype(np.float32)
    assert got.shape == tuple(shape)
    np.testing.assert_array_equal(got, want.astype(a.dtype).astype(np.float32))


def test_window_node_gradient_lands_inside_the_window():
    """Training: the window's gradient is the same offset alias of its input's gradient (the reference leaves the
    input gradient outside the window unwritten, so only the window is compared)."""
    rng = np.random.default_rng(10)
    a = rng.standard_normal((2, 4, 6, 6)).astype(np.float32)
    dy = rng.standard_normal((2, 2, 3, 4)).astype(np.float32)
    ctx = S.Context()
    g = S.Graph()
    x = S.Tensor.from_numpy(a)
    n0 = g.add_node("relu", x)
    nw = g.add_node("window", n0, {"shape": [2, 2, 3, 4], "offset": [0, 1, 2, 1]})
    n1 = g.add_node("relu", nw)
    p = ctx.create_program(g, 2, training=True)
    y, dmid = ctx.resolve(n1.y()), ctx.resolve(n0.y().grad())
    ctx.resolve(n1.y().grad()).write(dy)
    assert p.run(1) == 0
    win = np.maximum(a, 0)[:, 1:3, 2:5, 1:5]
    np.testing.assert_array_equal(y.read(), win)
    np.testing.assert_array_equal(dmid.read()[:, 1:3, 2:5, 1:5], dy * (win > 0))


@pytest.mark.parametrize("where", ["input", "weight"])
def test_anomaly_detection_reports_a_planted_nan(where, monkeypatch, capfd):
    monkeypatch.setenv("SAGA_HIP_ANOMALY_THROW", "1")
    net = N.resnet20(4, dtype=S.FLOAT)
    rng = np.random.default_rng(12)
    x = rng.standard_normal((4, 3, 32, 32)).astype(np.float32)
    if where == "input":
        x[2, 1, 7, 9] = np.nan
    else:
        net.params["s3_1-conv-2-w"][5, 3, 1, 1] = np.nan
    ctx = S.Context()
    g, t = N.build_graph(net, x)
    p = ctx.create_program(g, 4, training=True, learning_rate=1e-3, anomaly_detect=True)
    ctx.resolve(t["labels"]).write(rng.integers(0, 10, (4, 1)).astype(np.int32))
    with pytest.raises(S.SagaError) as err:
        p.run(1)
    assert "Anomaly in tensor" in str(err.value)
    out = capfd.readouterr().err
    assert "*** Anomaly in tensor" in out and "(input)" in out
    if where == "weight":
        assert "s3_1-conv-2" in str(err.value) or "s3_1-conv-2" in out


def test_sparse_first_writer_is_moved_behind_the_dense_one(monkeypatch, tmp_path):
    """The gradient of a downsampling block's input has two writers: the projection's backward data (1x1 at
    stride 2, one pixel in four) and the block's first convolution (dense).  In graph order the projection writes
    first; the engine moves it behind the dense writer (three blocks in ResNet-50), which changes nothing but the
    order of the two and the side that accumulates - same writers per tensor, same gradients."""
    import re
    writers, grads = {}, {}
    names = ["s1-conv-w", "s3_1-conv-p-w", "s4_1-conv-1-w", "s5_1-bn-p-s"]
    for reorder in (True, False):
        if not reorder:
            monkeypatch.setenv("SAGA_HIP_NO_WRITER_REORDER", "1")
        net = N.resnet50(4, image=64)
        rng = np.random.default_rng(11)
        x = rng.standard_normal((4, 3, 64, 64)).astype(np.float32)
        ctx = S.Context()
        g, t = N.build_graph(net, x)
        p = ctx.create_program(g, net.batch, training=True, learning_rate=1e-4, initial_loss_scale=1024.0)
        ctx.resolve(t["labels"]).write(rng.integers(0, 1000, 4).astype(np.int32))
        dev = {k: ctx.resolve(t[k].grad()) for k in names}
        path = tmp_path / f"ops_{reorder}.txt"
        p.dump(str(path), False)
        w = {}
        for line in open(path):
            m = re.match(r"#\s*\d+: (\+?)dx:(T\d+) = convbwddata(?:\.bn)?\(w:(T\d+)", line)
            if m:
                w.setdefault(m.group(2), []).append((m.group(3), m.group(1) == "+"))
        writers[reorder] = w
        p.run(1)
        grads[reorder] = {k: dev[k].read().astype(np.float32) for k in names}
    on, off = writers[True], writers[False]
    assert on.keys() == off.keys()
    moved = [k for k in on if on[k] != off[k]]
    assert len(moved) == 3, moved
    for k in on:
        assert sorted(v[0] for v in on[k]) == sorted(v[0] for v in off[k])          # the same writers
    for k in moved:
        assert [v[0] for v in on[k]] == [v[0] for v in off[k]][::-1]
        assert [v[1] for v in on[k]] == [False, True] == [v[1] for v in off[k]]      # the first overwrites, the second adds
    for k in names:
        e = rel_err(grads[True][k], grads[False][k])
        print(f"  grad {k}: reordered against graph order {e:.3e}")
        assert e <= 1e-2, (k, e)
