"""Checkpoint and resume: weights + batch-norm statistics carried over as tensors, Adam's moments, step
counts, fp32 master weights and the loss scale through the optimizer state file.  Three steps, save, a new
context, load, two more steps must end bit-identical to five steps in one go (every kernel is deterministic)."""
import numpy as np
import pytest

from saga_amd import api as S
from saga_amd import networks as N

pytestmark = pytest.mark.gpu


def setup(net, x, labels, loss_scale):
    ctx = S.Context()
    g, t = N.build_graph(net, x)
    p = ctx.create_program(g, net.batch, training=True, learning_rate=1e-3, initial_loss_scale=loss_scale)
    ctx.resolve(t["labels"]).write(labels)
    state = {k: ctx.resolve(t[k]) for k in net.params}
    return ctx, p, state


@pytest.mark.parametrize("make,loss_scale", [(lambda: N.lenet(16), 0.0), (lambda: N.resnet20(16), 4096.0)],
                         ids=["lenet-fp32", "resnet20-fp16-mixed"])
def test_resume_is_bit_identical(make, loss_scale, tmp_path):
    net = make()
    rng = np.random.default_rng(13)
    x = rng.standard_normal((net.batch,) + tuple(net.in_shape)).astype(np.float32)
    labels = rng.integers(0, net.classes, (net.batch, 1)).astype(np.int32)

    _, p, state = setup(net, x, labels, loss_scale)
    p.run(5)
    straight = {k: v.read().copy() for k, v in state.items()}
    straight_scale = p.loss_scale()

    net_a = make()
    _, pa, state_a = setup(net_a, x, labels, loss_scale)
    pa.run(3)
    path = tmp_path / "adam.state"
    pa.save_optimizer(path)
    after3 = {k: v.read().copy() for k, v in state_a.items()}

    net_b = make()
    for k in net_b.params:  # the tensors a Graph::saveTensors / loadTensors round trip would carry
        net_b.params[k] = after3[k].astype(np.float32).reshape(np.asarray(net_b.params[k]).shape)
    _, pb, state_b = setup(net_b, x, labels, loss_scale)
    pb.load_optimizer(path)
    assert pb.loss_scale() == pa.loss_scale()
    pb.run(2)
    assert pb.loss_scale() == straight_scale
    for k in straight:
        np.testing.assert_array_equal(state_b[k].read(), straight[k], err_msg=k)

    # without the optimizer state the resumed run differs (so the file is what made it identical)
    net_c = make()
    for k in net_c.params:
        net_c.params[k] = after3[k].astype(np.float32).reshape(np.asarray(net_c.params[k]).shape)
    _, pc, state_c = setup(net_c, x, labels, loss_scale)
    pc.run(2)
    assert any(not np.array_equal(state_c[k].read(), straight[k]) for k in net.trainable)


def test_optimizer_state_rejects_a_different_program(tmp_path):
    rng = np.random.default_rng(1)
    net = N.lenet(4)
    x = rng.standard_normal((4,) + tuple(net.in_shape)).astype(np.float32)
    labels = rng.integers(0, 10, (4, 1)).astype(np.int32)
    _, p, _ = setup(net, x, labels, 0.0)
    p.run(1)
    path = tmp_path / "adam.state"
    p.save_optimizer(path)
    other = N.resnet20(4, dtype=S.FLOAT)
    xo = rng.standard_normal((4,) + tuple(other.in_shape)).astype(np.float32)
    _, po, _ = setup(other, xo, labels, 0.0)
    with pytest.raises(Exception, match="optimizer state"):
        po.load_optimizer(path)
    (tmp_path / "junk").write_bytes(b"not a state file")
    with pytest.raises(Exception, match="optimizer state"):
        po.load_optimizer(tmp_path / "junk")
