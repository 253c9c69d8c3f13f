"""HIP-graph replay of the step against operation-by-operation execution.

With SAGA_HIP_GRAPH=1 the engine, after two plain steps, records the runs of graph-safe operations of a
program into HIP graphs and replays them.  Every kernel is deterministic, so a run with graphs must reproduce a run without them
bit for bit: same losses after every step (each read is a synchronisation and host work between two
replays), same weights at the end."""
import os

import numpy as np
import pytest

from saga_amd import api as S
from saga_amd import networks as N

pytestmark = pytest.mark.gpu


def small_unet():
    net = N.unet(2, image=32, classes=8, widths=(8, 16, 32, 64), bottleneck=128)
    b = N.Builder(net, 99)
    b.shape[net.output] = (8, 32, 32)
    net.output = b.fc(b.pool("avgpool", net.output, global_=True), "cls", 8)
    return net


def train(net, steps, graphs, params, loss_scale):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((net.batch,) + tuple(net.in_shape)).astype(np.float32)
    labels = rng.integers(0, net.classes, (net.batch, 1)).astype(np.int32)
    os.environ["SAGA_HIP_GRAPH"] = "1" if graphs else "0"
    try:
        ctx = S.Context()
        g, t = N.build_graph(net, x)
        p = ctx.create_program(g, net.batch, training=True, learning_rate=1e-3, initial_loss_scale=loss_scale)
        loss, logits = ctx.resolve(t["loss"]), ctx.resolve(t[net.output])
        ctx.resolve(t["labels"]).write(labels)
        dev = {k: ctx.resolve(t[k]) for k in params}
        trace = []
        for _ in range(steps):
            p.run(1)
            trace.append((loss.read().copy(), logits.read().copy(), p.loss_scale()))
        p.run(3)  # several replays back to back inside one run() as well
        trace.append((loss.read().copy(), logits.read().copy(), p.loss_scale()))
        return trace, {k: v.read().copy() for k, v in dev.items()}
    finally:
        os.environ.pop("SAGA_HIP_GRAPH", None)


CASES = [
    ("lenet fp32", lambda: N.lenet(16), ["c1-w", "fc2-w", "fc1-b"], 0.0),
    ("resnet20 fp16", lambda: N.resnet20(16), ["s1-conv-w", "s4_2-conv-2-w", "fc-w", "s2_0-bn-1-s"], 32768.0),
    ("resnet20 fp32", lambda: N.resnet20(8, dtype=S.FLOAT), ["s1-conv-w", "fc-w"], 0.0),
    ("unet fp16", small_unet, ["down0a-w", "up3-t-w", "up2-t-b", "head-w"], 256.0),
]


@pytest.mark.parametrize("name,make,params,loss_scale", CASES, ids=[c[0] for c in CASES])
def test_graph_replay_matches_eager_training(name, make, params, loss_scale, capfd, monkeypatch):
    monkeypatch.setenv("SAGA_HIP_GRAPH_VERBOSE", "1")
    eager, w_eager = train(make(), 7, False, params, loss_scale)
    assert "into a graph" not in capfd.readouterr().err
    graph, w_graph = train(make(), 7, True, params, loss_scale)
    assert "into a graph" in capfd.readouterr().err, "the graph run recorded nothing"
    assert len(eager) == len(graph)
    for i, (a, b) in enumerate(zip(eager, graph)):
        np.testing.assert_array_equal(a[0], b[0], err_msg=f"{name}: loss after step {i}")
        np.testing.assert_array_equal(a[1], b[1], err_msg=f"{name}: logits after step {i}")
        assert a[2] == b[2], f"{name}: loss scale after step {i}"
    # the steps do change the result, so equal traces are not equal by standing still
    assert not np.array_equal(eager[0][1], eager[-1][1])
    for k in params:
        np.testing.assert_array_equal(w_eager[k], w_graph[k], err_msg=f"{name}: weights {k}")


def test_graph_replay_matches_eager_inference_shared_weights():
    """An inference program replayed from graphs while a training program of the same context keeps
    changing the weights and re-using the arena between the replays."""
    def go(graphs):
        os.environ["SAGA_HIP_GRAPH"] = "1" if graphs else "0"
        try:
            net = N.resnet20(16)
            rng = np.random.default_rng(5)
            x = rng.standard_normal((net.batch,) + tuple(net.in_shape)).astype(np.float32)
            labels = rng.integers(0, net.classes, (net.batch, 1)).astype(np.int32)
            ctx = S.Context()
            g, t = N.build_graph(net, x)
            tr = ctx.create_program(g, net.batch, training=True, learning_rate=1e-3, initial_loss_scale=1024.0)
            inf = ctx.create_program(g, net.batch, training=False)
            logits = ctx.resolve(t[net.output])
            ctx.resolve(t["labels"]).write(labels)
            out = []
            for _ in range(6):
                tr.run(1)
                inf.run(1)
                out.append(logits.read().copy())
            return out
        finally:
            os.environ.pop("SAGA_HIP_GRAPH", None)

    a, b = go(False), go(True)
    for i, (u, v) in enumerate(zip(a, b)):
        np.testing.assert_array_equal(u, v, err_msg=f"inference logits after round {i}")
    assert not np.array_equal(a[0], a[-1])
