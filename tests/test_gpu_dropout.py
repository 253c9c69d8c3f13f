"""Dropout (reference: cudnnDropoutForward / Backward, src/cuda/cuda_dnn.cpp:1486-1574): inference aliases it
away, training scales the kept elements by 1 / (1 - prob).  cuDNN's random stream is closed, so the masks
cannot be compared with the reference's (parity unpinned); what the rule fixes is checked: the kept fraction,
exact zeros and exact scaling, a mask that depends only on the key and the logical element (not on layout),
a new mask per call, and a backward pass that uses the mask of the forward pass it answers."""
import ctypes as C

import numpy as np
import pytest
import torch

from saga_amd import api as S
from saga_amd import kernels as K
from tests.gpu_util import dev, host, rnd

pytestmark = pytest.mark.gpu


def run_fwd(x, dtype, layout, prob, seed, offset):
    xd = dev(x, dtype, layout)
    yd = dev(np.full(x.shape, 7.0, np.float32), dtype, layout)
    K.check(K.lib().saga_hip_dropout_fwd(C.byref(K.view(xd)), C.byref(K.view(yd)), prob, seed, offset, K.stream_ptr()))
    return host(yd)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_dropout_rule(dtype):
    rng = np.random.default_rng(3)
    shape, prob = (4, 16, 24, 24), 0.3
    x = rnd(rng, *shape, dtype=dtype) + 3.0  # no zeros in x: a zero in y is a dropped element
    x = x.astype(np.float16).astype(np.float32) if dtype == torch.float16 else x
    y = run_fwd(x, dtype, "nchw", prob, 11, 1)
    keep = y != 0
    n = keep.size
    assert abs(keep.mean() - (1 - prob)) < 4 * np.sqrt(prob * (1 - prob) / n)
    tol = 1e-6 if dtype == torch.float32 else 1e-3
    np.testing.assert_allclose(y[keep], (x / (1 - prob))[keep], rtol=tol)
    # per channel and per sample the fraction holds too (no stripes)
    assert np.abs(keep.mean(axis=(0, 2, 3)) - (1 - prob)).max() < 0.06
    assert np.abs(keep.mean(axis=(1, 2, 3)) - (1 - prob)).max() < 0.03
    # the mask belongs to (key, logical element): same in channels-last memory, new for another call or seed
    np.testing.assert_array_equal(run_fwd(x, dtype, "nhwc", prob, 11, 1) != 0, keep)
    other = run_fwd(x, dtype, "nchw", prob, 11, 2) != 0
    assert 0.3 < (other != keep).mean() < 0.55  # two independent masks differ on 2p(1-p) = 42 % of the elements
    assert 0.3 < ((run_fwd(x, dtype, "nchw", prob, 12, 1) != 0) != keep).mean() < 0.55
    # neighbouring elements are uncorrelated
    a, b = keep[..., :-1].ravel().astype(np.float64), keep[..., 1:].ravel().astype(np.float64)
    assert abs(np.corrcoef(a, b)[0, 1]) < 0.02
    # prob 0 is the identity
    np.testing.assert_array_equal(run_fwd(x, dtype, "nchw", 0.0, 11, 1), x)

    # backward with the forward's key: dx = dy * mask / (1 - prob), accumulated with beta
    dy = rnd(rng, *shape, dtype=dtype) + 3.0
    dyd = dev(dy, dtype, "nhwc")
    dxd = dev(np.ones(shape, np.float32), dtype, "nhwc")
    K.check(K.lib().saga_hip_dropout_bwd(C.byref(K.view(dyd)), C.byref(K.view(dxd)), prob, 11, 1, 1.0, K.stream_ptr()))
    dx = host(dxd)
    want = np.where(keep, host(dyd) / (1 - prob), 0.0) + 1.0
    np.testing.assert_allclose(dx, want, rtol=tol * 10, atol=tol * 10)
    assert K.lib().saga_hip_dropout_fwd(C.byref(K.view(dyd)), C.byref(K.view(dxd)), 1.0, 1, 1, K.stream_ptr()) == -1


def test_dropout_in_a_training_program_and_aliased_away_for_inference():
    rng = np.random.default_rng(5)
    B, F = 32, 256
    x = (rng.standard_normal((B, F)).astype(np.float32) + 4.0)
    w = (rng.standard_normal((F, 10)) * 0.05).astype(np.float32)
    g = S.Graph()
    tx = S.Tensor.from_numpy(x, name="x")
    tw = S.Tensor.from_numpy(w, name="w")
    d = g.add_node("dropout", tx, {"prob": 0.25})
    fc = g.add_node("fc", {"x": d.y(), "w": tw}, {"outputs": 10})
    cls = g.add_node("catclassifier", {"x": fc.y()})
    labels = rng.integers(0, 10, (B, 1)).astype(np.int32)

    ctx = S.Context()
    p = ctx.create_program(g, B, training=True, learning_rate=1e-3)
    yd, dxd = ctx.resolve(d.y()), ctx.resolve(tx.grad())
    ctx.resolve(cls.y().grad()).write(labels)
    masks = []
    for _ in range(3):
        p.run(1)
        y, dx = yd.read(), dxd.read()
        keep = y != 0
        assert abs(keep.mean() - 0.75) < 4 * np.sqrt(0.1875 / keep.size)
        np.testing.assert_allclose(y[keep], (x / 0.75)[keep], rtol=1e-6)
        # the gradient reaches exactly the elements the forward pass kept
        np.testing.assert_array_equal(dx != 0, keep)
        masks.append(keep)
    assert (masks[0] != masks[1]).mean() > 0.2 and (masks[1] != masks[2]).mean() > 0.2  # a new mask every step

    ctx2 = S.Context()
    pi = ctx2.create_program(g, B, training=False)
    logits = ctx2.resolve(fc.y())
    pi.run(1)
    np.testing.assert_allclose(logits.read(), x @ ctx2.resolve(tw).read().reshape(F, 10), rtol=2e-4, atol=2e-4)
