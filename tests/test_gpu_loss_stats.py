"""The L2 `loss` node and the `stats` node (reference: src/cuda/cuda_dnn.cpp:1358-1482, :2638-2680 and the
kernels src/cuda/cuda_kernels.cu:252-473) through the C ABI and through a training program."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import ref
from saga_amd import api as S
from saga_amd import kernels as K
from tests.gpu_util import assert_close, dev, host, rnd

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("xdt,tdt", [(torch.float32, torch.float32), (torch.float16, torch.float32), (torch.float16, torch.float16)])
@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
@pytest.mark.parametrize("shape", [(3, 5, 6, 7), (4, 1000, 1, 1), (2, 8, 33, 9)])
def test_loss_bwd(shape, layout, xdt, tdt):
    rng = np.random.default_rng(7)
    x, t = rnd(rng, *shape, dtype=xdt), rnd(rng, *shape, dtype=tdt) + 0.25
    if tdt == torch.float16:
        t = t.astype(np.float16).astype(np.float32)
    xd, td = dev(x, xdt, layout), dev(t, tdt, layout)
    dxd = dev(np.full(shape, 9.0, np.float32), xdt, layout)
    mmss = torch.full((shape[0], 4), 9.0, dtype=torch.float32, device="cuda")
    K.check(K.lib().saga_hip_loss_bwd(C.byref(K.view(xd)), C.byref(K.view(td)), C.byref(K.view(dxd)), K.ptr(mmss), 0.125,
                                      K.stream_ptr()))
    dx_ref, mmss_ref = ref.loss_bwd(x, t, 0.125)
    assert_close(host(dxd), dx_ref, xdt, "loss dx")
    assert_close(mmss.cpu().numpy(), mmss_ref, torch.float32, "mmss")
    if xdt == torch.float32:
        assert K.lib().saga_hip_loss_bwd(C.byref(K.view(xd)), C.byref(K.view(dev(t, torch.float16, layout))),
                                         C.byref(K.view(dxd)), K.ptr(mmss), 1.0, K.stream_ptr()) == -3


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("layout,padc", [("nchw", 0), ("nhwc", 0), ("nhwc", 8)])
@pytest.mark.parametrize("shape,shift", [((2, 16, 9, 9), 0.0), ((1, 3, 300, 301), 2.0), ((5, 7, 1, 1), -3.0)])
def test_tensor_stats(shape, shift, layout, padc, dtype):
    rng = np.random.default_rng(8)
    x = rnd(rng, *shape, dtype=dtype) + shift
    x = x.astype(np.float16).astype(np.float32) if dtype == torch.float16 else x
    xd = dev(x, dtype, layout, padc)
    out = torch.zeros(4, dtype=torch.float32, device="cuda")
    n = K.lib().saga_hip_tensor_stats_workspace_size()
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    assert K.lib().saga_hip_tensor_stats(C.byref(K.view(xd)), K.ptr(out), None, 0, K.stream_ptr()) == -4
    K.check(K.lib().saga_hip_tensor_stats(C.byref(K.view(xd)), K.ptr(out), K.ptr(ws), n, K.stream_ptr()))
    got, want = out.cpu().numpy(), ref.tensor_stats(x)
    np.testing.assert_allclose(got[:3], want[:3], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got[3], want[3], rtol=1e-4, atol=1e-6)


def test_loss_and_stats_nodes_in_a_training_program():
    """fc -> loss against a target, with a stats node on the fc output: one Adam step moves the weights against
    the gradient the loss node leaves, mmss and stats match the oracle."""
    rng = np.random.default_rng(9)
    B, F, O = 16, 32, 8
    x = rng.standard_normal((B, F)).astype(np.float32)
    w = (rng.standard_normal((F, O)) * 0.2).astype(np.float32)
    tgt = rng.standard_normal((B, O)).astype(np.float32)
    g = S.Graph()
    tx, tw, tt = S.Tensor.from_numpy(x, name="x"), S.Tensor.from_numpy(w, name="w"), S.Tensor.from_numpy(tgt, name="target")
    fc = g.add_node("fc", {"x": tx, "w": tw}, {"outputs": O})
    loss = g.add_node("loss", {"x": fc.y(), "target": tt}, {"strength": 2.0})
    st = g.add_node("stats", {"x": fc.y()})
    ctx = S.Context()
    p = ctx.create_program(g, B, training=True, learning_rate=1e-2)
    y, mmss, stats = ctx.resolve(loss.y()), ctx.resolve(loss.output("mmss")), ctx.resolve(st.y())
    dw, wd = ctx.resolve(tw.grad()), ctx.resolve(tw)
    p.run(1)
    out = x @ w
    np.testing.assert_allclose(y.read().reshape(B, O), out, rtol=1e-4, atol=1e-5)
    # the reference multiplies by the program's loss scale in every precision (src/cuda/cuda_dnn.cpp:1428-1443),
    # and that scale starts at the sum of the batch sizes (src/cuda/cuda_common.cpp:338-353): in an fp32 program,
    # where nothing divides it out again, the gradient is strength * (y - target)
    dx_ref, mmss_ref = ref.loss_bwd(out, tgt, 2.0 / B * B)
    np.testing.assert_allclose(mmss.read().reshape(B, 4), mmss_ref, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(stats.read().reshape(4), ref.tensor_stats(out), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dw.read().reshape(F, O), x.T @ dx_ref, rtol=1e-4, atol=1e-5)
    # Adam's first step: every weight moves by lr against the sign of its gradient
    step = wd.read().reshape(F, O) - w
    gsign = np.sign(x.T @ dx_ref)
    big = np.abs(x.T @ dx_ref) > 1e-4
    np.testing.assert_allclose(step[big], (-1e-2 * gsign)[big], rtol=1e-3)
