"""The hot path at the benchmark's FULL sizes (batch 256), where the CPU oracle cannot run the
whole problem in seconds: size-independent properties, plus the oracle on a slice of the batch
wherever samples are independent.

 * convolution: y(x, 2w) = 2 y(x, w) bit for bit on normal fp16 results (fp32 accumulation, one
   rounding: scaling by a power of two commutes with it); the adjoint identity <y, dy> = <x, dx> = <w, dw> ties
   forward, backward-data and backward-filter together; forward and backward-data of the first
   images against the oracle (samples do not interact);
 * batch norm (training): per-channel mean and variance of the output are b and s^2; the
   gradient has zero sum and zero correlation with the normalised input per channel;
 * max pooling: every dy lands on exactly one input position; on a batch norm's input, values and
   first-maximum position codes against torch on the whole tensor;
 * ResNet-50 b256 at 224x224 through the engine: inference logits of the first images against
   the oracle network (running statistics make samples independent), finite loss and a
   loss-scale step after one training step.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import ref
from oracle.net import OracleNet
from saga_amd import api as S
from saga_amd import kernels as K
from saga_amd import networks as N
from tests.gpu_util import assert_close, host, rel_err

pytestmark = pytest.mark.gpu

HALF = torch.float16
N256 = 256


def nhwc(t):
    return t.contiguous(memory_format=torch.channels_last)


def dot(a, b):
    return float((a.double() * b.double()).sum())


# Cin, H, Cout, R, stride, pad: the conv microbenchmark shape, a strided 3x3 (class-split backward
# data), a 1x1 stride 2 (classes without taps), a deep 1x1, the RGB stem (thin-input path) and the 1x1 that
# widens 64 channels to 256 (the streaming kernel)
FULL_CONVS = [(64, 56, 64, 3, 1, 1), (128, 56, 128, 3, 2, 1), (256, 56, 512, 1, 2, 0), (1024, 14, 256, 1, 1, 0),
              (3, 224, 64, 7, 2, 3), (64, 56, 256, 1, 1, 0)]


@pytest.mark.parametrize("shape", FULL_CONVS)
def test_conv_full_batch_properties(shape):
    Cc, H, Kk, R, stride, pad = shape
    g = torch.Generator(device="cuda").manual_seed(Cc + Kk)
    x = nhwc(torch.randn(N256, Cc, H, H, dtype=HALF, device="cuda", generator=g))
    w = nhwc(torch.randn(Kk, Cc, R, R, dtype=HALF, device="cuda", generator=g) * (2.0 / (Cc * R * R)) ** 0.5)
    P = 1 + (H + 2 * pad - R) // stride
    y = nhwc(torch.zeros(N256, Kk, P, P, dtype=HALF, device="cuda"))
    y2 = torch.zeros_like(y)
    K.conv2d(K.CONV_FWD, x, w, y, pad, stride)
    K.conv2d(K.CONV_FWD, x, nhwc(w * 2), y2, pad, stride)
    # bit for bit wherever the fp16 result is a normal number (subnormals round on a fixed grid)
    normal = y.abs() >= 2.0 ** -13
    assert bool(normal.float().mean() > 0.99)
    assert torch.equal(y2[normal], (y * 2)[normal]), "forward is not linear in the filter bit for bit"

    # first two images against the oracle
    y_ref = ref.conv2d_fwd(host(x[:2]), host(w), pad, stride)
    assert_close(host(y[:2]), y_ref, HALF, "y[:2]")

    dy = nhwc(torch.randn(N256, Kk, P, P, dtype=HALF, device="cuda", generator=g))
    dw = torch.zeros_like(w)
    K.conv2d(K.CONV_BWD_FILTER, x, dy, dw, pad, stride)
    lhs = dot(y, dy)
    # y and dw are rounded to fp16 element-wise: relative noise of the sums ~ 2^-11 / sqrt(terms)
    assert abs(dot(w, dw) - lhs) <= 2e-3 * abs(lhs) + 1e-2 * float(dw.double().abs().sum()) * 2 ** -11
    if Cc >= 8:
        dx = torch.zeros_like(x)
        K.conv2d(K.CONV_BWD_DATA, dy, w, dx, pad, stride)
        assert abs(dot(x, dx) - lhs) <= 2e-3 * abs(lhs)
        dx_ref = ref.conv2d_bwd_data(host(dy[:2]), host(w), (2, Cc, H, H), pad, stride)
        assert_close(host(dx[:2]), dx_ref, HALF, "dx[:2]")
        # beta = 1 adds to what is there
        K.conv2d(K.CONV_BWD_DATA, dy, w, dx, pad, stride, beta=1.0)
        assert_close(host(dx[:1]), 2 * dx_ref[:1], HALF, "dx beta=1")


@pytest.mark.parametrize("shape", FULL_CONVS)
def test_conv_bwd_filter_full_batch_elementwise(shape):
    """Backward filter at the real launch geometry (the reduction over 256 images split over hundreds of blocks,
    then the fixed-order second pass), compared element by element with the oracle.
    1. dy is non-zero in two images only, so dw must equal the oracle's dw of those two images; three pairs that
       fall into different parts of the split.  Every element of dw is checked, and blocks that see only zeros
       must contribute nothing.
    2. dy dense: dw[k0:k1, c0:c1] depends only on x[:, c0:c1] and dy[:, k0:k1], which the oracle handles over all
       256 images; first, last and a middle block of channels."""
    Cc, H, Kk, R, stride, pad = shape
    g = torch.Generator(device="cuda").manual_seed(3 * Cc + Kk)
    x = nhwc(torch.randn(N256, Cc, H, H, dtype=HALF, device="cuda", generator=g))
    P = 1 + (H + 2 * pad - R) // stride
    dy = nhwc(torch.randn(N256, Kk, P, P, dtype=HALF, device="cuda", generator=g))
    dw = nhwc(torch.zeros(Kk, Cc, R, R, dtype=HALF, device="cuda"))
    worst = 0.0
    for pair in ((0, 255), (37, 128), (101, 202)):
        sparse = torch.zeros_like(dy)
        for n in pair:
            sparse[n] = dy[n]
        dw.fill_(7.0)  # beta = 0 must overwrite
        K.conv2d(K.CONV_BWD_FILTER, x, sparse, dw, pad, stride)
        idx = list(pair)
        want = ref.conv2d_bwd_filter(host(x[idx]), host(dy[idx]), (Kk, Cc, R, R), pad, stride)
        worst = max(worst, assert_close(host(dw), want, HALF, f"dw, dy non-zero in images {pair}", tol=2e-3))
    K.conv2d(K.CONV_BWD_FILTER, x, dy, dw, pad, stride)
    cb, kb = min(8, Cc), 8
    for c0, k0 in ((0, 0), (Cc - cb, Kk - kb), ((Cc // 2 // cb) * cb, (Kk // 2 // kb) * kb + 3 if Kk > 16 else 0)):
        k0 = min(k0, Kk - kb)
        want = ref.conv2d_bwd_filter(host(x[:, c0:c0 + cb]), host(dy[:, k0:k0 + kb]), (kb, cb, R, R), pad, stride)
        worst = max(worst, assert_close(host(dw[k0:k0 + kb, c0:c0 + cb]), want, HALF,
                                        f"dw[{k0}:{k0 + kb}, {c0}:{c0 + cb}] over all images", tol=2e-3))
    print(f"bwd-filter {shape}: worst element error {worst:.2e} of the largest element")


def test_conv_fp32_nchw_full_batch():
    """The fp32 NCHW half of the convolution microbenchmark at its real size (N=256, 64 -> 64, 56x56, 3x3):
    the adjoint identity across the three passes, the first two images of forward and backward data against
    the oracle, and backward filter element-wise with dy non-zero in two images."""
    Cc, H, Kk, R, stride, pad = 64, 56, 64, 3, 1, 1
    F32 = torch.float32
    g = torch.Generator(device="cuda").manual_seed(77)
    x = torch.randn(N256, Cc, H, H, dtype=F32, device="cuda", generator=g)
    w = torch.randn(Kk, Cc, R, R, dtype=F32, device="cuda", generator=g) * (2.0 / (Cc * R * R)) ** 0.5
    y = torch.zeros(N256, Kk, H, H, dtype=F32, device="cuda")
    K.conv2d(K.CONV_FWD, x, w, y, pad, stride)
    assert_close(host(y[:2]), ref.conv2d_fwd(host(x[:2]), host(w), pad, stride), F32, "y[:2]")
    assert_close(host(y[-1:]), ref.conv2d_fwd(host(x[-1:]), host(w), pad, stride), F32, "y[-1]")
    dy = torch.randn(N256, Kk, H, H, dtype=F32, device="cuda", generator=g)
    dx, dw = torch.zeros_like(x), torch.zeros_like(w)
    K.conv2d(K.CONV_BWD_DATA, dy, w, dx, pad, stride)
    K.conv2d(K.CONV_BWD_FILTER, x, dy, dw, pad, stride)
    lhs = dot(y, dy)
    assert abs(dot(x, dx) - lhs) <= 1e-5 * abs(lhs)
    assert abs(dot(w, dw) - lhs) <= 1e-5 * abs(lhs)
    assert_close(host(dx[:2]), ref.conv2d_bwd_data(host(dy[:2]), host(w), (2, Cc, H, H), pad, stride), F32, "dx[:2]")
    for pair in ((0, 255), (90, 171)):
        sparse = torch.zeros_like(dy)
        for n in pair:
            sparse[n] = dy[n]
        dw.fill_(7.0)
        K.conv2d(K.CONV_BWD_FILTER, x, sparse, dw, pad, stride)
        idx = list(pair)
        want = ref.conv2d_bwd_filter(host(x[idx]), host(dy[idx]), (Kk, Cc, R, R), pad, stride)
        assert_close(host(dw), want, F32, f"dw, dy non-zero in images {pair}")


# the up-convolutions of the U-Net configuration at their real channel widths and sizes, one image:
# Cin, H, Cout (2x2, stride 2)
UNET_UPCONVS = [(1024, 16, 512), (512, 32, 256), (256, 64, 128), (128, 128, 64)]


@pytest.mark.parametrize("shape", UNET_UPCONVS)
def test_transposed_conv_real_widths(shape):
    """Transposed convolution (src/cuda/cuda_dnn.cpp:542-574): forward = backward data with x in the dy role,
    dW = backward filter with (dy, x) exchanged, dX = forward convolution of dy - each against the oracle."""
    Cin, H, Cout = shape
    rng = np.random.default_rng(Cin)
    from tests.gpu_util import dev, rnd
    x = rnd(rng, 1, Cin, H, H, dtype=HALF)
    w = rnd(rng, Cin, Cout, 2, 2, dtype=HALF, scale=(2.0 / (Cout * 4)) ** 0.5)  # [Cx, Cy, R, S], src/node.cpp:99-110
    Ho = ref.tconv_out(H, 2, 0, 2)
    y_ref = ref.conv2d_bwd_data(x, w, (1, Cout, Ho, Ho), 0, 2)
    xd, wd = dev(x, HALF, "nhwc"), dev(w, HALF, "nhwc")
    yd = dev(np.zeros_like(y_ref), HALF, "nhwc")
    K.conv2d(K.CONV_BWD_DATA, xd, wd, yd, 0, 2)
    e1 = assert_close(host(yd), y_ref, HALF, "transposed conv y")
    dy = rnd(rng, 1, Cout, Ho, Ho, dtype=HALF)
    dyd = dev(dy, HALF, "nhwc")
    dwd = dev(np.zeros_like(w), HALF, "nhwc")
    K.conv2d(K.CONV_BWD_FILTER, dyd, xd, dwd, 0, 2)
    e2 = assert_close(host(dwd), ref.conv2d_bwd_filter(dy, x, w.shape, 0, 2), HALF, "transposed conv dw")
    dxd = dev(np.zeros_like(x), HALF, "nhwc")
    K.conv2d(K.CONV_FWD, dyd, wd, dxd, 0, 2)
    e3 = assert_close(host(dxd), ref.conv2d_fwd(dy, w, 0, 2), HALF, "transposed conv dx")
    print(f"transposed conv {shape}: y {e1:.1e}, dw {e2:.1e}, dx {e3:.1e}")


def test_batchnorm_full_size_invariants():
    Cc, H = 64, 112  # the largest batch-norm input of ResNet-50: 411 MB
    g = torch.Generator(device="cuda").manual_seed(7)
    x = nhwc(torch.randn(N256, Cc, H, H, dtype=HALF, device="cuda", generator=g) * 1.7 + 0.4)
    y, dy, dx = torch.zeros_like(x), nhwc(torch.randn(x.shape, dtype=HALF, device="cuda", generator=g)), torch.zeros_like(x)
    f = lambda v: torch.tensor(v, dtype=torch.float32, device="cuda")
    rng = np.random.default_rng(3)
    s, b = f(1 + 0.3 * rng.standard_normal(Cc)), f(0.2 * rng.standard_normal(Cc))
    m, v, sm, sv, ds, db = f(np.zeros(Cc)), f(np.ones(Cc)), f(np.zeros(Cc)), f(np.zeros(Cc)), f(np.zeros(Cc)), f(np.zeros(Cc))
    ws = K.bn_workspace(x)
    L = K.lib()
    K.check(L.saga_hip_bn_train_fwd(C.byref(K.view(x)), None, C.byref(K.view(y)), K.ptr(s), K.ptr(b), K.ptr(m), K.ptr(v),
                                    K.ptr(sm), K.ptr(sv), 1e-5, 0.1, 0, K.ptr(ws), ws.numel(), None))
    yd = y.double()
    mean, var = yd.mean((0, 2, 3)), yd.var((0, 2, 3), unbiased=False)
    assert float((mean - b.double()).abs().max()) <= 2e-3
    assert float((var / (s.double() ** 2) - 1).abs().max()) <= 5e-3
    xd = x.double()
    assert float((sm.double() - xd.mean((0, 2, 3))).abs().max()) <= 1e-4
    assert float((sv.double() * torch.sqrt(xd.var((0, 2, 3), unbiased=False) + 1e-5) - 1).abs().max()) <= 1e-4

    K.check(L.saga_hip_bn_bwd(C.byref(K.view(x)), None, C.byref(K.view(dy)), C.byref(K.view(dx)), None, K.ptr(s), K.ptr(sm),
                              K.ptr(sv), K.ptr(ds), K.ptr(db), 0.0, 0.0, 0.0, 0, K.ptr(ws), ws.numel(), None))
    dxd = dx.double()
    xhat = (xd - sm.double().view(1, -1, 1, 1)) * sv.double().view(1, -1, 1, 1)
    n = N256 * H * H
    scale = float(dxd.abs().mean()) * n
    assert float(dxd.sum((0, 2, 3)).abs().max()) <= 2e-4 * scale          # sum over the batch of dx is 0
    assert float((dxd * xhat).sum((0, 2, 3)).abs().max()) <= 2e-4 * scale  # and so is its correlation with x^
    assert float((db.double() - dy.double().sum((0, 2, 3))).abs().max()) <= 1e-3 * float(db.abs().max())
    assert float((ds.double() - (dy.double() * xhat).sum((0, 2, 3))).abs().max()) <= 1e-3 * float(ds.abs().max()) + 1.0


def test_maxpool_full_size_routes_every_gradient_once():
    Cc, H = 64, 112
    g = torch.Generator(device="cuda").manual_seed(11)
    x = nhwc(torch.relu(torch.randn(N256, Cc, H, H, dtype=HALF, device="cuda", generator=g)))  # many ties at 0
    P = 56
    y = nhwc(torch.zeros(N256, Cc, P, P, dtype=HALF, device="cuda"))
    L = K.lib()
    K.check(L.saga_hip_pool_fwd(K.POOL_MAX, C.byref(K.view(x)), C.byref(K.view(y)), None, 3, 1, 2, None))
    assert torch.equal(y, nhwc(torch.nn.functional.max_pool2d(x.float(), 3, 2, 1).to(HALF)))
    dy = nhwc(torch.ones(N256, Cc, P, P, dtype=HALF, device="cuda"))  # ones: dx counts the windows won
    dx = torch.zeros_like(x)
    K.check(L.saga_hip_pool_bwd(K.POOL_MAX, C.byref(K.view(x)), C.byref(K.view(y)), C.byref(K.view(dy)),
                                C.byref(K.view(dx)), 3, 1, 2, 0.0, None))
    assert float(dx.double().sum()) == float(N256 * Cc * P * P)
    assert float(dx.max()) <= 4  # a position lies in at most 2 x 2 windows
    # a position that won a window holds that window's maximum
    # (row h lies in the windows h // 2 and (h + 1) // 2)
    won = dx > 0
    ia = torch.arange(H, device="cuda") // 2
    ib = torch.clamp((torch.arange(H, device="cuda") + 1) // 2, max=P - 1)
    holds = torch.zeros_like(won)
    for r in (ia, ib):
        for c in (ia, ib):
            holds |= x == y[:, :, r][:, :, :, c]
    assert bool(holds[won].all())


def test_maxpool_on_batch_norm_full_size_values_and_first_maximum_codes():
    """saga_hip_maxpool_fwd_codes_bn on the stem's tensor (256 x 64 x 112 x 112).  Scales that are powers of two
    make fma(x, scale, shift) exact before its one rounding to fp32, so torch's multiply-add is the same number
    and the normalised tensor can be built outside the library: pooled values bit for bit, and every position
    code equal to the FIRST maximum of its window (relu leaves zeros in every window: ties everywhere)."""
    Cc, H, P = 64, 112, 56
    g = torch.Generator(device="cuda").manual_seed(12)
    x = nhwc(torch.randn(N256, Cc, H, H, dtype=HALF, device="cuda", generator=g))
    sc = (2.0 ** torch.randint(-2, 3, (Cc,), generator=torch.Generator().manual_seed(3)).float())
    sc[1::3] = -sc[1::3]  # negative scales: the maximum sits at the minimum of x
    sh = torch.randn(Cc, generator=torch.Generator().manual_seed(4))
    ss = torch.cat([sc, sh]).cuda()
    y = nhwc(torch.zeros(N256, Cc, P, P, dtype=HALF, device="cuda"))
    codes = torch.full((N256, P, P, Cc), 255, dtype=torch.uint8, device="cuda")
    L = K.lib()
    K.check(L.saga_hip_maxpool_fwd_codes_bn(C.byref(K.view(x)), C.byref(K.view(y)), K.ptr(codes), 3, 1, 2, K.ptr(ss),
                                            K.BN_RELU, None))
    z = torch.relu(x.float() * sc.cuda()[None, :, None, None] + sh.cuda()[None, :, None, None]).to(HALF)
    assert torch.equal(y, nhwc(torch.nn.functional.max_pool2d(z.float(), 3, 2, 1).to(HALF)))
    # the nine window positions as nine strided views of the padded tensor; torch.max reports the first maximum
    zp = torch.nn.functional.pad(z, (1, 1, 1, 1), value=float("-inf"))
    best = torch.full_like(y, float("-inf"))
    first = torch.zeros(y.shape, dtype=torch.uint8, device="cuda")
    for k in range(9):
        v = zp[:, :, k // 3:k // 3 + 2 * P:2, k % 3:k % 3 + 2 * P:2]
        take = v > best
        best = torch.where(take, v, best)
        first = torch.where(take, torch.full_like(first, k), first)
    assert torch.equal(best, y)
    assert torch.equal(codes.permute(0, 3, 1, 2), first)


def test_resnet50_b256_through_the_engine():
    net = N.resnet50(N256, image=224)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((N256, 3, 224, 224)).astype(np.float16)
    labels = rng.integers(0, 1000, (N256, 1)).astype(np.int32)
    ctx = S.Context()
    graph, t = N.build_graph(net, x)
    train = ctx.create_program(graph, N256, training=True, learning_rate=1e-4, initial_loss_scale=1024.0)
    infer = ctx.create_program(graph, N256, training=False)
    ctx.resolve(t["labels"]).write(labels)
    logits, loss, pred = ctx.resolve(t[net.output]), ctx.resolve(t["loss"]), ctx.resolve(t["pred"])

    # inference first (the training step will move the weights): first two images against the oracle
    infer.run(1)
    got = logits.read().astype(np.float32)[:2]
    small = N.resnet50(2, image=224)
    small.params = net.params
    o = OracleNet(small)
    want = o.forward(x[:2].astype(np.float32), training=False)
    e = rel_err(got, want)
    print("inference logits[:2] rel err", e)
    assert e <= 2e-2
    assert np.array_equal(pred.read()[:2].reshape(-1), ref.catclassifier_fwd(want).reshape(-1))

    train.run(1)
    l = loss.read()
    assert np.isfinite(l).all() and 4.0 < float(l.mean()) < 12.0  # ~ln(1000) = 6.9 for an untrained net
    assert abs(train.loss_scale() - 1024.0 * 1.02) < 1e-2          # no overflow: the scale grows by 2 %
    arena, planned = ctx.memory()
    assert 0 < arena < planned
