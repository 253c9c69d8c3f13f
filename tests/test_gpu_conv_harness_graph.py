"""The training graph of the reference's `conv` command (test/test_conv.cpp:96-140: strided conv + bias -> relu ->
fc with transposed weights + bias -> relu -> reshape -> transposed conv + bias -> L2 loss against the input) built
through the API from SEEDED weights and trained on the hip engine next to the CPU oracle, step by step.  The
command itself draws its weights from a clock-seeded generator (src/tensor.cpp:1081-1085) and can only be judged
by "the error fell" (tests/test_gpu_reference_harness.py); this is its deterministic twin."""
import numpy as np
import pytest

from oracle.net import OracleNet
from saga_amd import api as S
from saga_amd import networks as N
from tests.gpu_util import rel_err

pytestmark = pytest.mark.gpu

LR = 1e-2
STEPS = 400
EXACT_STEPS = 25  # steps over which the two trajectories have not yet had time to drift apart


class Run:
    def __init__(self, dtype, seed):
        self.net, self.x = N.conv_harness(dtype, seed)
        self.ctx = S.Context()
        g, t = N.build_graph(self.net, self.x)
        # the harness creates its program with batch size 1 although the tensors hold two samples
        self.p = self.ctx.create_program(g, 1, training=True, learning_rate=LR)
        self.y = self.ctx.resolve(t[self.net.loss])
        self.mmss = self.ctx.resolve(t[self.net.loss + "-mmss"])
        self.w = {k: self.ctx.resolve(t[k]) for k in self.net.trainable}
        self.dw = {k: self.ctx.resolve(t[k].grad()) for k in self.net.trainable}
        self.g, self.t = g, t

    def step(self):
        self.p.run(1)
        return self.mmss.read().reshape(2, 4).astype(np.float64)


@pytest.mark.parametrize("seed", [6, 7])
@pytest.mark.parametrize("dtype", [S.FLOAT, S.HALF], ids=["fp32", "fp16"])
def test_conv_harness_graph_against_the_oracle_step_by_step(dtype, seed):
    half = dtype == S.HALF
    r = Run(dtype, seed)
    o = OracleNet(r.net, lr=LR)
    assert o.loss_scale == 1.0
    tol = 2e-2 if half else 1e-4
    wtol = 2e-2 if half else 1e-5
    worst = {"y": 0.0, "mmss": 0.0, "grad": 0.0, "weight": 0.0}
    mse_dev, mse_ora = [], []
    for step in range(1, STEPS + 1):
        mmss = r.step()
        o_mmss, _, o_grads, flags = o.train_step(r.x)
        mse_dev.append(float(mmss[:, 3].mean()))
        mse_ora.append(float(o_mmss[:, 3].mean()))
        if half:
            assert abs(r.p.loss_scale() - float(o.loss_scale)) <= 1e-6 * float(o.loss_scale), step
        if step <= EXACT_STEPS:
            worst["y"] = max(worst["y"], rel_err(r.y.read().astype(np.float32), o.acts[r.net.loss]))
            # min / max / mean / mean square of the residual, as one tensor: the mean is a difference of
            # nearly equal sums and is held to the bar relative to the row's largest entry
            worst["mmss"] = max(worst["mmss"], rel_err(mmss, o_mmss))
            for k in r.net.trainable:
                g = r.dw[k].read().astype(np.float32).reshape(o_grads[k].shape)
                worst["grad"] = max(worst["grad"], rel_err(g, o_grads[k]))
                w = r.w[k].read().astype(np.float32).reshape(o.p[k].shape)
                e = rel_err(w, o.p[k])
                worst["weight"] = max(worst["weight"], e)
    print(f"seed {seed} {'fp16' if half else 'fp32'}: first {EXACT_STEPS} steps worst errors "
          + ", ".join(f"{k} {v:.2e}" for k, v in worst.items()))
    print("  mean squared error, engine vs oracle, at steps 1, 25, 100, 200, 400: "
          + ", ".join(f"{mse_dev[i - 1]:.4g}/{mse_ora[i - 1]:.4g}" for i in (1, 25, 100, 200, 400)))
    assert worst["y"] <= tol and worst["mmss"] <= tol and worst["grad"] <= tol, worst
    # Adam's first steps move every weight by about lr whatever the gradient's size, so an element whose
    # gradient is rounding noise may go the other way: weights are held to the bar plus two such steps
    big = max(float(np.abs(o.p[k]).max()) for k in r.net.trainable)
    assert worst["weight"] <= wtol + (2.5 * LR * EXACT_STEPS / big if half else 0.0), worst
    # later the trajectories are allowed to drift, the training result is not: both fall, to similar errors
    assert np.isfinite(mse_dev).all()
    assert mse_dev[-1] <= 0.5 * mse_dev[0] and mse_ora[-1] <= 0.5 * mse_ora[0]
    assert abs(mse_dev[-1] - mse_ora[-1]) <= 0.25 * max(mse_ora[-1], mse_ora[0] * 0.02)


@pytest.mark.parametrize("seed", [6, 7, 8])
def test_conv_harness_graph_fp16_converges_like_fp32(seed):
    """The same seeded weights (rounded to fp16 for both runs) trained in fp32 and in mixed precision, whose
    loss scale starts at the program's batch size - 1 - and grows 2 % per step: the fp16 run must reach the
    error of the fp32 run, not lag behind it."""
    r32, r16 = Run(S.FLOAT, seed), Run(S.HALF, seed)
    for k, v in r32.net.params.items():
        r32.ctx.resolve(r32.t[k]).write(v.astype(np.float16).astype(np.float32))
    m32, m16 = [], []
    for _ in range(STEPS):
        m32.append(float(r32.step()[:, 3].mean()))
        m16.append(float(r16.step()[:, 3].mean()))
    marks = (1, 10, 50, 100, 200, 300, 400)
    print(f"seed {seed}: mean squared error fp32 / fp16 at steps {marks}: "
          + ", ".join(f"{m32[i - 1]:.4g}/{m16[i - 1]:.4g}" for i in marks))
    print(f"  loss scale of the fp16 run after {STEPS} steps: {r16.p.loss_scale():.4g}")
    assert np.isfinite(m16).all() and np.isfinite(m32).all()
    assert abs(m16[0] - m32[0]) <= 2e-2 * m32[0]
    assert m16[-1] <= 0.5 * m16[0]
    assert m16[-1] <= 1.5 * m32[-1] + 0.02 * m32[0]
