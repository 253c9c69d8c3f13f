"""GPU parity: every entry point of the C ABI (include/saga_hip.h) against the CPU oracle on the
same seeded inputs.  fp32 within 1e-4 and fp16 within 2e-2 of the per-tensor max-abs value;
labels, pooling indices and flags bit-exact."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import ref
from saga_amd import kernels as K
from tests.gpu_util import assert_close, dev, host, rnd

pytestmark = pytest.mark.gpu

DT = [torch.float32, torch.float16]
LAYOUTS = [("nchw", 0), ("nhwc", 0), ("nhwc", 8)]


def S():
    return K.stream_ptr()


def T(g, name):
    t = g[name]
    return np.array(t["data"][: int(np.prod(t["dims"]))], np.float32).reshape(t["dims"])


def w_dev(w, dtype, layout):
    return dev(w, dtype, "nhwc" if layout == "nhwc" else "nchw")


CONV_CASES = [
    # N, C, H, W, K, R, pad, stride, group
    (2, 16, 9, 9, 8, 3, 1, 1, 1),
    (2, 8, 11, 10, 16, 3, 1, 2, 1),
    (1, 3, 15, 15, 8, 7, 3, 2, 1),
    (2, 16, 8, 8, 32, 1, 0, 1, 1),
    (2, 32, 8, 8, 16, 1, 0, 2, 1),
    (2, 8, 7, 7, 4, 3, 0, 1, 2),
    (3, 64, 14, 14, 64, 3, 1, 1, 1),
    (2, 16, 13, 13, 24, 3, 0, 2, 1),
    (1, 8, 17, 18, 8, 5, 2, 4, 1),
    (2, 24, 9, 9, 40, 2, 1, 2, 1),
    (2, 4, 12, 12, 16, 5, 2, 2, 1),
    (2, 1, 10, 11, 8, 3, 1, 2, 1),
    (1, 3, 21, 21, 72, 8, 3, 4, 1),
    (2, 32, 12, 11, 72, 5, 2, 2, 1),
    (5, 96, 10, 10, 40, 3, 1, 1, 1),
    # thin inputs under a 7-row filter: whole output rows per block, several tiles per image, a partial last tile
    (2, 3, 56, 56, 64, 7, 3, 2, 1),
    (1, 4, 33, 29, 24, 7, 3, 2, 1),
    # 3x3 on 64 -> 64 channels with enough images for the kernel that keeps whole rows in LDS: four full tiles
    # per image; a partial last tile, a row length that is no multiple of anything and 56 output channels
    (37, 64, 56, 56, 64, 3, 1, 1, 1),
    (130, 64, 30, 27, 56, 3, 1, 1, 1),
    # ... and for the backward filter that does the same (tiles of a whole number of 16-pixel steps): 48 output
    # channels and a last tile of two rows; eight rows of 32 pixels per tile
    (64, 64, 30, 56, 48, 3, 1, 1, 1),
    (128, 64, 32, 32, 64, 3, 1, 1, 1),
    # 1x1 from 64 to 256 channels: enough pixels for the streaming kernel (a partial last strip of 64), and a small
    # ragged tensor that takes it only when SAGA_HIP_C64_WIDE=2 forces it
    (45, 64, 56, 55, 256, 1, 0, 1, 1),
    (3, 64, 30, 31, 256, 1, 0, 1, 1),
    # dilated (a tenth entry: dilation)
    (2, 16, 13, 12, 24, 3, 2, 1, 1, 2),
    (2, 32, 15, 15, 16, 3, 3, 2, 1, 3),
    (1, 8, 17, 17, 8, 5, 4, 1, 1, 2),
    (2, 64, 14, 14, 64, 3, 2, 1, 1, 2),
]


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("layout,padc", LAYOUTS)
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_fwd_bwd(case, layout, padc, dtype):
    N, Cc, H, W, Kk, R, pad, stride, group = case[:9]
    dil = case[9] if len(case) > 9 else 1
    rng = np.random.default_rng(hash(case) % 1000)
    x = rnd(rng, N, Cc, H, W, dtype=dtype)
    w = rnd(rng, Kk, Cc // group, R, R, dtype=dtype, scale=(2.0 / (Cc // group * R * R)) ** 0.5)
    y_ref = ref.conv2d_fwd(x, w, pad, stride, dil, group)
    dy = rnd(rng, *y_ref.shape, dtype=dtype)
    dx_ref = ref.conv2d_bwd_data(dy, w, x.shape, pad, stride, dil, group)
    dw_ref = ref.conv2d_bwd_filter(x, dy, w.shape, pad, stride, dil, group)

    xd, wd = dev(x, dtype, layout, padc), w_dev(w, dtype, layout)
    yd = dev(np.zeros_like(y_ref), dtype, layout, padc)
    K.conv2d(K.CONV_FWD, xd, wd, yd, pad, stride, dil, group)
    assert_close(host(yd), y_ref, dtype, "y")
    # beta = 1 accumulates into the existing output (residual sum folded into the conv)
    K.conv2d(K.CONV_FWD, xd, wd, yd, pad, stride, dil, group, 1.0, 1.0)
    assert_close(host(yd), 2 * y_ref, dtype, "y beta=1")

    dyd = dev(dy, dtype, layout, padc)
    dxd = dev(np.zeros_like(x), dtype, layout, padc)
    K.conv2d(K.CONV_BWD_DATA, dyd, wd, dxd, pad, stride, dil, group)
    assert_close(host(dxd), dx_ref, dtype, "dx")
    dwd = w_dev(np.zeros_like(w), dtype, layout)
    K.conv2d(K.CONV_BWD_FILTER, xd, dyd, dwd, pad, stride, dil, group)
    assert_close(host(dwd), dw_ref, dtype, "dw")
    K.conv2d(K.CONV_BWD_FILTER, xd, dyd, dwd, pad, stride, dil, group, 1.0, 1.0)
    assert_close(host(dwd), 2 * dw_ref, dtype, "dw beta=1")


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
@pytest.mark.parametrize("R,S", [(1, 3), (3, 1), (2, 5)])
def test_conv_nonsquare_filter(R, S, layout, dtype):
    """Filters with R != S (the oracle's pad applies to both axes, as the reference's single `pad` does)."""
    rng = np.random.default_rng(R * 10 + S)
    N, Cc, H, W, Kk, pad, stride = 2, 16, 11, 12, 24, 1, 1
    x = rnd(rng, N, Cc, H, W, dtype=dtype)
    w = rnd(rng, Kk, Cc, R, S, dtype=dtype, scale=(2.0 / (Cc * R * S)) ** 0.5)
    y_ref = ref.conv2d_fwd(x, w, pad, stride)
    dy = rnd(rng, *y_ref.shape, dtype=dtype)
    xd, wd = dev(x, dtype, layout), w_dev(w, dtype, layout)
    yd = dev(np.zeros_like(y_ref), dtype, layout)
    K.conv2d(K.CONV_FWD, xd, wd, yd, pad, stride)
    assert_close(host(yd), y_ref, dtype, "y")
    dyd, dxd = dev(dy, dtype, layout), dev(np.zeros_like(x), dtype, layout)
    K.conv2d(K.CONV_BWD_DATA, dyd, wd, dxd, pad, stride)
    assert_close(host(dxd), ref.conv2d_bwd_data(dy, w, x.shape, pad, stride), dtype, "dx")
    dwd = w_dev(np.zeros_like(w), dtype, layout)
    K.conv2d(K.CONV_BWD_FILTER, xd, dyd, dwd, pad, stride)
    assert_close(host(dwd), ref.conv2d_bwd_filter(x, dy, w.shape, pad, stride), dtype, "dw")


@pytest.mark.parametrize("case", [(2, 64, 14, 64, 3, 1, 1, 3), (3, 32, 9, 160, 1, 0, 1, 1), (2, 128, 13, 24, 3, 1, 2, 0),
                                  (2, 3, 30, 64, 7, 3, 2, 3), (2, 16, 8, 20, 3, 1, 1, 3),
                                  # the stem kernel: partial last tile; more tiles than blocks and a ragged channel tile
                                  (2, 3, 56, 64, 7, 3, 2, 3), (130, 3, 64, 40, 7, 3, 2, 1),
                                  # 3x3 64 -> 64 with whole rows in LDS (see CONV_CASES)
                                  (37, 64, 56, 64, 3, 1, 1, 3), (130, 64, 30, 56, 3, 1, 1, 1), (40, 64, 56, 64, 3, 1, 1, 0),
                                  # 3x3 layers of the last stages: many channels, tiles with dead rows, 7x7 images
                                  (3, 128, 14, 256, 3, 1, 1, 3), (6, 64, 7, 136, 3, 1, 1, 1), (2, 64, 28, 64, 3, 1, 1, 2),
                                  # 1x1 64 -> 256 (see CONV_CASES): norm alone, with relu, with residual and relu
                                  (45, 64, 56, 256, 1, 0, 1, 0), (43, 64, 56, 256, 1, 0, 1, 3), (3, 64, 30, 256, 1, 0, 1, 3),
                                  (3, 64, 31, 256, 1, 0, 1, 1)])
def test_conv_with_folded_bn_inference(case):
    """Convolution with the inference batch norm (+ residual + relu) in its epilogue against the two
    separate operators of the oracle."""
    N, Cc, H, Kk, R, pad, stride, flags = case
    dtype = torch.float16
    rng = np.random.default_rng(Cc * 5 + Kk)
    x = rnd(rng, N, Cc, H, H, dtype=dtype)
    w = rnd(rng, Kk, Cc, R, R, dtype=dtype, scale=(2.0 / (Cc * R * R)) ** 0.5)
    y_conv = ref.round_half(ref.conv2d_fwd(x, w, pad, stride))
    z = rnd(rng, *y_conv.shape, dtype=dtype)
    s, b = (1 + 0.2 * rng.standard_normal(Kk)).astype(np.float32), (0.1 * rng.standard_normal(Kk)).astype(np.float32)
    m, v = (0.3 * rng.standard_normal(Kk)).astype(np.float32), rng.uniform(0.5, 1.5, Kk).astype(np.float32)
    want = ref.bn_infer(y_conv, s, b, m, v, 1e-5)
    if flags & K.BN_ADD:
        want = want + z
    if flags & K.BN_RELU:
        want = ref.act_fwd(want)
    L = K.lib()
    xd, wd, zd = dev(x, dtype, "nhwc"), dev(w, dtype, "nhwc"), dev(z, dtype, "nhwc")
    yd = dev(np.zeros_like(y_conv), dtype, "nhwc")
    sd, bd, md, vd = (dev(t) for t in (s, b, m, v))
    p = K.ConvParams(pad, stride, 1, 1)
    vx, vw, vy = K.view(xd), K.view(wd), K.view(yd)
    ws = torch.zeros(max(1, L.saga_hip_conv2d_workspace_size(K.CONV_FWD, C.byref(vx), C.byref(vw), C.byref(vy),
                                                             C.byref(p))), dtype=torch.uint8, device="cuda")
    K.check(L.saga_hip_conv2d_fwd_bn_infer(C.byref(vx), C.byref(vw), C.byref(vy),
                                           C.byref(K.view(zd)) if flags & K.BN_ADD else None, C.byref(p), K.ptr(sd),
                                           K.ptr(bd), K.ptr(md), K.ptr(vd), 1e-5, flags, K.ptr(ws), ws.numel(), S()))
    assert_close(host(yd), want, dtype, "conv+bn")


BNSTATS_CASES = [
    # N, C, H, K, R, pad, stride, relu+add
    (2, 64, 14, 64, 3, 1, 1, False),
    (3, 32, 9, 160, 1, 0, 1, True),
    (2, 128, 13, 24, 3, 1, 2, True),
    (2, 3, 30, 64, 7, 3, 2, False),
    (2, 3, 56, 64, 7, 3, 2, False),
    (130, 3, 64, 64, 7, 3, 2, True),
    (37, 64, 56, 64, 3, 1, 1, False),
    (130, 64, 30, 56, 3, 1, 1, True),
    # 3x3 layers of the last stages: row counts that are no multiple of the tile, 7x7 images, 56x56 at 64 channels
    (3, 128, 14, 256, 3, 1, 1, True),
    (6, 64, 7, 136, 3, 1, 1, False),
    (2, 64, 56, 64, 3, 1, 1, True),
    # 1x1 64 -> 256 (see CONV_CASES)
    (45, 64, 56, 256, 1, 0, 1, True),
    (3, 64, 31, 256, 1, 0, 1, False),
]


@pytest.mark.parametrize("case", BNSTATS_CASES)
def test_conv_bnstats_then_bn_from_partials(case):
    """Convolution that leaves the batch-norm partial sums, followed by the batch norm that starts
    from them: same results as the separate conv and batch-norm entry points."""
    N, Cc, H, Kk, R, pad, stride, fused = case
    dtype = torch.float16
    rng = np.random.default_rng(Cc * 7 + Kk)
    x = rnd(rng, N, Cc, H, H, dtype=dtype)
    w = rnd(rng, Kk, Cc, R, R, dtype=dtype, scale=(2.0 / (Cc * R * R)) ** 0.5)
    y_ref = ref.round_half(ref.conv2d_fwd(x, w, pad, stride))
    L = K.lib()
    xd, wd = dev(x, dtype, "nhwc"), dev(w, dtype, "nhwc")
    yd = dev(np.zeros_like(y_ref), dtype, "nhwc")
    p = K.ConvParams(pad, stride, 1, 1)
    vx, vw, vy = K.view(xd), K.view(wd), K.view(yd)
    nbytes = L.saga_hip_conv2d_fwd_bnstats_size(C.byref(vx), C.byref(vw), C.byref(vy), C.byref(p))
    assert nbytes > 0
    partial = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    ws = torch.zeros(max(1, L.saga_hip_conv2d_workspace_size(K.CONV_FWD, C.byref(vx), C.byref(vw), C.byref(vy),
                                                             C.byref(p))), dtype=torch.uint8, device="cuda")
    rows = C.c_int(0)
    K.check(L.saga_hip_conv2d_fwd_bnstats(C.byref(vx), C.byref(vw), C.byref(vy), C.byref(p), 1.0, K.ptr(ws), ws.numel(),
                                          K.ptr(partial), nbytes, C.byref(rows), S()))
    assert_close(host(yd), y_ref, dtype, "y")
    # the partial rows add up to the sums over the stored (rounded) output
    yh = host(yd).astype(np.float64)
    got = host(partial)[: rows.value * Kk * 2].reshape(rows.value, Kk, 2).astype(np.float64).sum(0)
    np.testing.assert_allclose(got[:, 0], yh.sum((0, 2, 3)), rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(got[:, 1], (yh * yh).sum((0, 2, 3)), rtol=1e-4, atol=1e-3)

    flags = (K.BN_RELU | K.BN_ADD) if fused else 0
    z = rnd(rng, *y_ref.shape, dtype=dtype)
    s, b = (1 + 0.2 * rng.standard_normal(Kk)).astype(np.float32), (0.1 * rng.standard_normal(Kk)).astype(np.float32)
    m, v = np.zeros(Kk, np.float32), np.ones(Kk, np.float32)
    zd, od = dev(z, dtype, "nhwc"), dev(np.zeros_like(y_ref), dtype, "nhwc")
    sd, bd, md, vd = (dev(t) for t in (s, b, m, v))
    sm, sv = dev(np.zeros(Kk, np.float32)), dev(np.zeros(Kk, np.float32))
    ws2 = torch.zeros(2 * Kk, dtype=torch.float32, device="cuda")
    # the relu mask (one bit per element) exists for fp16 tensors with whole 8-channel vectors
    want_mask = fused and Kk % 8 == 0
    mask = torch.zeros(max(1, int(np.prod(y_ref.shape)) // 8), dtype=torch.uint8, device="cuda")
    K.check(L.saga_hip_bn_train_fwd_partials(C.byref(K.view(yd)), C.byref(K.view(zd)) if fused else None,
                                             C.byref(K.view(od)), K.ptr(sd), K.ptr(bd), K.ptr(md), K.ptr(vd),
                                             K.ptr(sm), K.ptr(sv), 1e-5, 0.1, flags, K.ptr(partial), rows.value,
                                             K.ptr(mask) if want_mask else None, K.ptr(ws2), ws2.numel() * 4, S()))
    o_ref, rsm, rsv, rm, rv = ref.bn_train_fwd(host(yd), s, b, m, v, 1e-5, 0.1)
    if fused:
        o_ref = ref.act_fwd(o_ref + z)
    assert_close(host(od), o_ref, dtype, "bn y")
    assert_close(host(sm), rsm, torch.float32, "saved mean", 1e-3)
    assert_close(host(sv), rsv, torch.float32, "saved invstd", 1e-3)
    assert_close(host(md), rm, torch.float32, "running mean", 1e-3)
    assert_close(host(vd), rv, torch.float32, "running var", 1e-3)
    if want_mask:
        # bit j of byte [pixel][c/8] <-> the stored y[pixel][8*(c/8)+j] > 0, bit-exact
        y_dev = host(od).transpose(0, 2, 3, 1).reshape(-1, Kk // 8, 8)
        bits = np.unpackbits(mask.cpu().numpy().reshape(-1, Kk // 8, 1), axis=2, bitorder="little")
        np.testing.assert_array_equal(bits.astype(bool), y_dev > 0)
        # backward with the mask in place of y: y is passed poisoned, so any read of it would show
        dy = rnd(rng, *y_ref.shape, dtype=dtype)
        dyp = dy * (host(od) > 0)
        dx_ref, ds_ref, db_ref = ref.bn_bwd(host(yd), dyp, s, host(sm), host(sv))
        dyd = dev(dy, dtype, "nhwc")
        dxd, dzd = dev(np.zeros_like(y_ref), dtype, "nhwc"), dev(np.zeros_like(y_ref), dtype, "nhwc")
        poisoned = dev(np.full_like(y_ref, -1.0), dtype, "nhwc")
        dsd, dbd = dev(np.zeros(Kk, np.float32)), dev(np.zeros(Kk, np.float32))
        vx = K.view(yd)
        wsb = torch.zeros(L.saga_hip_bn_workspace_size(C.byref(vx)), dtype=torch.uint8, device="cuda")
        K.check(L.saga_hip_bn_bwd_ex(C.byref(vx), C.byref(K.view(poisoned)), C.byref(K.view(dyd)), C.byref(K.view(dxd)),
                                     C.byref(K.view(dzd)), K.ptr(sd), K.ptr(bd), K.ptr(sm), K.ptr(sv), K.ptr(dsd),
                                     K.ptr(dbd), 0.0, 0.0, 0.0, flags, K.ptr(mask), K.ptr(wsb), wsb.numel(), S()))
        assert_close(host(dzd), dyp, dtype, "bn dz (mask bits)")
        assert_close(host(dxd), dx_ref, dtype, "bn dx (mask bits)")
        assert_close(host(dsd), ds_ref, torch.float32, "bn ds (mask bits)", 5e-3)
        assert_close(host(dbd), db_ref, torch.float32, "bn db (mask bits)", 5e-3)


@pytest.mark.parametrize("dtype", DT)
def test_conv_golden(golden, dtype):
    g = golden["ops"]
    for layout in ("nchw", "nhwc"):
        x, w = dev(T(g, "conv_input_x"), dtype, layout), w_dev(T(g, "conv_input_w"), dtype, layout)
        y = dev(np.zeros((1, 2, 8, 8), np.float32), dtype, layout)
        K.conv2d(K.CONV_FWD, x, w, y, pad=1)
        b = dev(T(g, "conv_input_b").reshape(-1), dtype)
        K.check(K.lib().saga_hip_bias_add(C.byref(K.view(y)), C.byref(K.view(b.view(1, 2, 1, 1))), S()))
        sse = float(((host(y).astype(np.float64) - T(g, "conv_output")) ** 2).sum())
        assert sse <= (1e-4 if dtype == torch.float32 else 1e-3), sse


@pytest.mark.parametrize("dtype", DT)
def test_transposed_conv(dtype):
    # forward of a transposed conv is bwd_data with x in the dy role (src/cuda/cuda_dnn.cpp:545-548)
    rng = np.random.default_rng(3)
    x, w = rnd(rng, 2, 16, 5, 5, dtype=dtype), rnd(rng, 16, 8, 2, 2, dtype=dtype, scale=0.2)
    Ho = ref.tconv_out(5, 2, 0, 2)
    y_ref = ref.conv2d_bwd_data(x, w, (2, 8, Ho, Ho), 0, 2)
    for layout in ("nchw", "nhwc"):
        yd = dev(np.zeros_like(y_ref), dtype, layout)
        K.conv2d(K.CONV_BWD_DATA, dev(x, dtype, layout), w_dev(w, dtype, layout), yd, 0, 2)
        assert_close(host(yd), y_ref, dtype, "tconv y")


def test_backward_data_with_batched_filter_transpose():
    """saga_hip_filter_transpose_batched + saga_hip_conv2d_bwd_data_wt: every filter of a set transposed in one
    launch (bit-exact against numpy, including shapes that are no multiple of the 64x64 tile or of 8), and
    backward data fed with such a copy bit-identical to saga_hip_conv2d_bwd_data."""
    rng = np.random.default_rng(21)
    L = K.lib()
    # N, C, H, W, K, R, pad, stride
    cases = [(2, 64, 14, 14, 64, 3, 1, 1), (2, 32, 9, 10, 160, 1, 0, 1), (3, 128, 13, 13, 24, 3, 1, 2),
             (1, 200, 6, 6, 72, 5, 2, 1), (2, 20, 7, 7, 12, 3, 1, 1)]
    ws_, jobs, keep, first = [], [], [], 0
    for (N, Cc, H, W, Kk, R, pad, stride) in cases:
        w = rnd(rng, Kk, Cc, R, R, dtype=torch.float16, scale=(2.0 / (Cc * R * R)) ** 0.5)
        wd = w_dev(w, torch.float16, "nhwc")
        wt = torch.full((Cc * R * R * Kk,), 7.0, dtype=torch.float16, device="cuda")
        nb = L.saga_hip_filter_transpose_blocks(C.byref(K.view(wd)))
        assert nb == R * R * ((Kk + 63) // 64) * ((Cc + 63) // 64)
        jobs.append(K.FilterTransposeJob(wd.data_ptr(), wt.data_ptr(), Kk, Cc, R * R, first))
        first += nb
        ws_.append((w, wd, wt))
    arr = (K.FilterTransposeJob * len(jobs))(*jobs)
    jd = torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8).cuda()
    K.check(L.saga_hip_filter_transpose_batched(K.ptr(jd), len(jobs), first, S()))
    torch.cuda.synchronize()
    for (N, Cc, H, W, Kk, R, pad, stride), (w, wd, wt) in zip(cases, ws_):
        want = np.ascontiguousarray(w.transpose(1, 2, 3, 0)).astype(np.float16)  # C,R,S,K
        np.testing.assert_array_equal(wt.cpu().numpy().reshape(want.shape), want)
        P, Q = ref.conv_out(H, R, pad, stride), ref.conv_out(W, R, pad, stride)
        dy = rnd(rng, N, Kk, P, Q, dtype=torch.float16)
        dyd = dev(dy, torch.float16, "nhwc")
        dx_a = dev(np.ones((N, Cc, H, W), np.float32), torch.float16, "nhwc")
        dx_b = dev(np.ones((N, Cc, H, W), np.float32), torch.float16, "nhwc")
        p = K.ConvParams(pad, stride, 1, 1)
        vdy, vw, va, vb = K.view(dyd), K.view(wd), K.view(dx_a), K.view(dx_b)
        nbytes = L.saga_hip_conv2d_bwd_data_wt_bytes(C.byref(vdy), C.byref(vw), C.byref(va), C.byref(p))
        wsz = L.saga_hip_conv2d_workspace_size(K.CONV_BWD_DATA, C.byref(va), C.byref(vw), C.byref(vdy), C.byref(p))
        ws = torch.empty(max(wsz, 16), dtype=torch.uint8, device="cuda")
        K.check(L.saga_hip_conv2d_bwd_data(C.byref(vdy), C.byref(vw), C.byref(va), C.byref(p), 1.0, 1.0, K.ptr(ws),
                                           ws.numel(), S()))
        if nbytes == 0:  # not on the path that takes a transposed filter: the call says so, and NULL falls through
            assert L.saga_hip_conv2d_bwd_data_wt(C.byref(vdy), C.byref(vw), K.ptr(wt), C.byref(vb), C.byref(p), 1.0, 1.0,
                                                 K.ptr(ws), ws.numel(), S()) == -3
            K.check(L.saga_hip_conv2d_bwd_data_wt(C.byref(vdy), C.byref(vw), None, C.byref(vb), C.byref(p), 1.0, 1.0,
                                                  K.ptr(ws), ws.numel(), S()))
        else:
            assert nbytes == wt.numel() * 2
            K.check(L.saga_hip_conv2d_bwd_data_wt(C.byref(vdy), C.byref(vw), K.ptr(wt), C.byref(vb), C.byref(p), 1.0, 1.0,
                                                  None, 0, S()))
        np.testing.assert_array_equal(host(dx_a), host(dx_b))
        assert_close(host(dx_a), ref.conv2d_bwd_data(dy, w, (N, Cc, H, W), pad, stride) + 1, torch.float16, "bwd data")


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("layout,padc", LAYOUTS)
def test_bias(layout, padc, dtype):
    rng = np.random.default_rng(5)
    y, b = rnd(rng, 3, 16, 5, 5, dtype=dtype), rnd(rng, 16, dtype=dtype)
    yd = dev(y, dtype, layout, padc)
    bd = dev(b, torch.float32)
    K.check(K.lib().saga_hip_bias_add(C.byref(K.view(yd)), C.byref(K.view(bd.view(1, 16, 1, 1))), S()))
    assert_close(host(yd), ref.bias_add(y, b), dtype, "bias add")
    db = dev(np.ones(16, np.float32), torch.float32)
    dyd = dev(y, dtype, layout, padc)
    K.check(K.lib().saga_hip_bias_bwd(C.byref(K.view(dyd)), C.byref(K.view(db.view(1, 16, 1, 1))), 1.0, None, 0, S()))
    assert_close(host(db), ref.bias_bwd(y) + 1, dtype, "bias bwd")


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("padc", [0, 8, 3])
@pytest.mark.parametrize("shape", [(4, 64, 96, 96), (2, 20, 200, 150), (64, 1000, 5, 5), (1, 4104, 16, 16)])
def test_bias_bwd_large(shape, padc, dtype):
    """Tensors large enough for the two-pass reduction over row blocks (needs the workspace)."""
    rng = np.random.default_rng(6)
    y = rnd(rng, *shape, dtype=dtype)
    c = shape[1]
    dyd = dev(y, dtype, "nhwc", padc)
    vdy = K.view(dyd)
    need = K.lib().saga_hip_bias_bwd_workspace_size(C.byref(vdy))
    assert need > 0
    db = dev(np.ones(c, np.float32), torch.float32)
    vdb = K.view(db.view(1, c, 1, 1))
    assert K.lib().saga_hip_bias_bwd(C.byref(vdy), C.byref(vdb), 1.0, None, 0, S()) == -4
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    K.check(K.lib().saga_hip_bias_bwd(C.byref(vdy), C.byref(vdb), 1.0, K.ptr(ws), need, S()))
    got, want = host(db), ref.bias_bwd(y) + 1
    scale = np.abs(y.astype(np.float64)).sum(axis=(0, 2, 3)).max()
    assert np.abs(got - want).max() <= 2e-6 * scale, "bias bwd large"


BNBWD_LINK_CASES = [
    # N, C (norm channels = dx channels), H, W, K (dy channels), R, pad, stride, relu, beta, channel pad of dx / x
    (2, 64, 14, 14, 64, 3, 1, 1, True, 0.0, 0),     # 3x3 of a bottleneck, 256x64 tile
    (3, 160, 9, 10, 32, 1, 0, 1, True, 0.0, 0),     # 1x1, 160 channels: two block columns, the second ragged
    (2, 128, 13, 13, 24, 3, 1, 2, True, 0.0, 8),    # stride 2: four residue classes, padded rows
    (2, 128, 13, 13, 24, 3, 1, 2, True, 1.0, 0),    # stride 2 accumulating onto an earlier writer
    (2, 64, 12, 12, 64, 1, 0, 2, False, 0.0, 0),    # 1x1 stride 2: three classes get no tap and are zero-filled
    (6, 64, 7, 7, 136, 3, 1, 1, False, 1.0, 0),     # no relu, beta 1, 7x7 images
    (2, 64, 56, 56, 64, 3, 1, 1, True, 0.0, 0),     # many block rows
    (5, 512, 7, 7, 128, 1, 0, 1, True, 0.0, 0),     # at most one block per CU: the kernel with producer wavefronts
    (11, 256, 56, 56, 64, 1, 0, 1, True, 0.0, 0),   # more than 256 blocks of 256x128
    (2, 256, 12, 12, 64, 1, 0, 2, True, 1.0, 0),    # 1x1 stride 2 accumulating: three classes run blocks with no
                                                    # reduction step at all, which mask and sum the old gradient
    (2, 128, 13, 13, 24, 3, 1, 4, True, 1.0, 8),    # stride 4: sixteen residue classes, seven without a tap
]


@pytest.mark.parametrize("case", BNBWD_LINK_CASES)
def test_conv_bwd_data_linked_to_bn_backward(case):
    """saga_hip_conv2d_bwd_data_bnbwd + saga_hip_bn_bwd_linked against the two separate entry points
    (saga_hip_conv2d_bwd_data, saga_hip_bn_bwd_ex) and the oracle: the stored gradient is the unlinked one
    masked by the norm's relu, bit for bit; the partial sums are its per-channel sums; dx, ds, db agree."""
    N, Cc, H, W, Kk, R, pad, stride, relu, beta, padc = case
    dtype = torch.float16
    rng = np.random.default_rng(Cc * 11 + Kk + R)
    L = K.lib()
    # the norm's forward on the device: its own statistics and output define the mask
    x = rnd(rng, N, Cc, H, W, dtype=dtype) * 1.5 + 0.5
    x = x.astype(np.float16).astype(np.float32)
    s, b, m, v = _bn_params(rng, Cc)
    flags = K.BN_RELU if relu else 0
    xd, yd = dev(x, dtype, "nhwc", padc), dev(np.zeros_like(x), dtype, "nhwc")
    sd, bd, md, vd = (dev(t) for t in (s, b, m, v))
    sm, sv = dev(np.zeros(Cc, np.float32)), dev(np.zeros(Cc, np.float32))
    wsb = K.bn_workspace(xd)
    K.check(L.saga_hip_bn_train_fwd(C.byref(K.view(xd)), None, C.byref(K.view(yd)), K.ptr(sd), K.ptr(bd), K.ptr(md),
                                    K.ptr(vd), K.ptr(sm), K.ptr(sv), 1e-5, 0.1, flags, K.ptr(wsb), wsb.numel(), S()))
    keep = host(yd) > 0 if relu else np.ones_like(x, bool)
    # the convolution whose backward data produces the gradient of y
    P, Q = ref.conv_out(H, R, pad, stride), ref.conv_out(W, R, pad, stride)
    w = rnd(rng, Kk, Cc, R, R, dtype=dtype, scale=(2.0 / (Kk * R * R)) ** 0.5)
    dy = rnd(rng, N, Kk, P, Q, dtype=dtype)
    old = rnd(rng, N, Cc, H, W, dtype=dtype)
    wd, dyd = dev(w, dtype, "nhwc"), dev(dy, dtype, "nhwc")
    ga, gb = dev(old, dtype, "nhwc", padc), dev(old, dtype, "nhwc", padc)
    p = K.ConvParams(pad, stride, 1, 1)
    vdy, vw, va, vb, vx = K.view(dyd), K.view(wd), K.view(ga), K.view(gb), K.view(xd)
    wsz = L.saga_hip_conv2d_workspace_size(K.CONV_BWD_DATA, C.byref(va), C.byref(vw), C.byref(vdy), C.byref(p))
    ws = torch.empty(max(wsz, 16), dtype=torch.uint8, device="cuda")
    # unlinked
    K.check(L.saga_hip_conv2d_bwd_data(C.byref(vdy), C.byref(vw), C.byref(va), C.byref(p), 1.0, beta, K.ptr(ws),
                                       ws.numel(), S()))
    g_ref = ref.round_half(ref.conv2d_bwd_data(dy, w, x.shape, pad, stride) + beta * old)
    assert_close(host(ga), g_ref, dtype, "unlinked gradient")
    dxa = dev(np.zeros_like(x), dtype, "nhwc")
    dsa, dba = dev(np.zeros(Cc, np.float32)), dev(np.zeros(Cc, np.float32))
    K.check(L.saga_hip_bn_bwd_ex(C.byref(vx), None, C.byref(va), C.byref(K.view(dxa)), None, K.ptr(sd),
                                 K.ptr(bd), K.ptr(sm), K.ptr(sv), K.ptr(dsa), K.ptr(dba), 0.0, 0.0, 0.0, flags, None,
                                 K.ptr(wsb), wsb.numel(), S()))
    # linked
    nbytes = L.saga_hip_conv2d_bwd_data_bnbwd_size(C.byref(vdy), C.byref(vw), C.byref(vb), C.byref(p))
    assert nbytes > 0
    partial = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    link = K.BnBwdLink(C.pointer(vx), K.ptr(sd), K.ptr(bd), K.ptr(sm), K.ptr(sv), flags, 0, K.ptr(partial), nbytes)
    K.check(L.saga_hip_conv2d_bwd_data_bnbwd(C.byref(vdy), C.byref(vw), None, C.byref(vb), C.byref(p), 1.0, beta,
                                             K.ptr(ws), ws.numel(), C.byref(link), S()))
    rows = link.partial_rows
    assert 0 < rows * Cc * 2 * 4 <= nbytes
    g_masked = np.where(keep, host(ga), 0.0)
    np.testing.assert_array_equal(host(gb), g_masked)
    got = host(partial)[: rows * Cc * 2].reshape(rows, Cc, 2).astype(np.float64)
    assert np.isfinite(got).all(), "a partial row was not written"
    got = got.sum(0)
    mean = host(sm).astype(np.float64).reshape(1, Cc, 1, 1)
    gm = g_masked.astype(np.float64)
    want0, want1 = gm.sum((0, 2, 3)), (gm * (x - mean)).sum((0, 2, 3))
    np.testing.assert_allclose(got[:, 0], want0, rtol=1e-4, atol=1e-3 * max(1.0, np.abs(want0).max()))
    np.testing.assert_allclose(got[:, 1], want1, rtol=1e-4, atol=1e-3 * max(1.0, np.abs(want1).max()))
    dxb = dev(np.ones_like(x), dtype, "nhwc")
    dsb, dbb = dev(np.ones(Cc, np.float32)), dev(np.ones(Cc, np.float32))
    K.check(L.saga_hip_bn_bwd_linked(C.byref(vx), C.byref(vb), C.byref(K.view(dxb)), K.ptr(sd), K.ptr(sm), K.ptr(sv),
                                     K.ptr(dsb), K.ptr(dbb), 0.0, 0.0, K.ptr(partial), rows, K.ptr(wsb), wsb.numel(),
                                     S()))
    dx_ref, ds_ref, db_ref = ref.bn_bwd(x, g_masked, s, host(sm), host(sv))
    for what, got_d, want_d in (("linked", dxb, dx_ref), ("unlinked", dxa, dx_ref)):
        assert_close(host(got_d), want_d, dtype, f"bn dx ({what})")
    assert_close(host(dxb), host(dxa), dtype, "bn dx linked against unlinked", 2e-3)
    assert_close(host(dsb), ds_ref, torch.float32, "bn ds", 5e-3)
    assert_close(host(dbb), db_ref, torch.float32, "bn db", 5e-3)
    assert_close(host(dsb), host(dsa), torch.float32, "bn ds linked against unlinked", 1e-4)
    assert_close(host(dbb), host(dba), torch.float32, "bn db linked against unlinked", 1e-4)
    # accumulation of the parameter gradients and of dx
    K.check(L.saga_hip_bn_bwd_linked(C.byref(vx), C.byref(vb), C.byref(K.view(dxb)), K.ptr(sd), K.ptr(sm), K.ptr(sv),
                                     K.ptr(dsb), K.ptr(dbb), 1.0, 1.0, K.ptr(partial), rows, K.ptr(wsb), wsb.numel(),
                                     S()))
    assert_close(host(dxb), 2 * dx_ref, dtype, "bn dx (beta 1)")
    assert_close(host(dsb), 2 * ds_ref, torch.float32, "bn ds (beta 1)", 5e-3)


def test_conv_bwd_data_bn_link_rejections():
    """Outside the pipelined fp16 channels-last path the linked entry point says so and leaves dx alone."""
    L = K.lib()
    rng = np.random.default_rng(5)
    dtype = torch.float16

    def attempt(Cc, layout, xdtype=torch.float16, dil=1, size=None):
        x = rnd(rng, 2, Cc, 8, 8, dtype=dtype)
        w = rnd(rng, 16, Cc, 3, 3, dtype=dtype)
        Pq = ref.conv_out(8, 3, dil, 1, dil)
        dyd, wd = dev(rnd(rng, 2, 16, Pq, Pq, dtype=dtype), dtype, layout), w_dev(w, dtype, layout)
        xd, gd = dev(x, xdtype, layout), dev(np.full_like(x, 3.0), dtype, layout)
        par = [dev(np.ones(Cc, np.float32)) for _ in range(4)]
        p = K.ConvParams(dil, 1, dil, 1)
        vdy, vw, vg, vx = K.view(dyd), K.view(wd), K.view(gd), K.view(xd)
        nbytes = L.saga_hip_conv2d_bwd_data_bnbwd_size(C.byref(vdy), C.byref(vw), C.byref(vg), C.byref(p))
        partial = torch.zeros(max(1, nbytes if size is None else size) // 4 + 1, dtype=torch.float32, device="cuda")
        link = K.BnBwdLink(C.pointer(vx), *(K.ptr(t) for t in par), K.BN_RELU, 0, K.ptr(partial),
                           nbytes if size is None else size)
        ws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
        rc = L.saga_hip_conv2d_bwd_data_bnbwd(C.byref(vdy), C.byref(vw), None, C.byref(vg), C.byref(p), 1.0, 0.0,
                                              K.ptr(ws), ws.numel(), C.byref(link), S())
        torch.cuda.synchronize()
        return rc, nbytes, host(gd)

    rc, nbytes, g = attempt(20, "nhwc")            # channel count no multiple of 8
    assert (rc, nbytes) == (-3, 0) and (g == 3.0).all()
    rc, nbytes, g = attempt(16, "nchw")            # channels-first
    assert (rc, nbytes) == (-3, 0) and (g == 3.0).all()
    rc, nbytes, g = attempt(16, "nhwc", dil=2)     # dilated
    assert (rc, nbytes) == (-3, 0) and (g == 3.0).all()
    rc, nbytes, g = attempt(16, "nhwc", xdtype=torch.float32)  # the norm's input in another type
    assert rc == -3 and (g == 3.0).all()
    rc, nbytes, g = attempt(16, "nhwc", size=64)   # partial buffer too small
    assert rc == -4 and nbytes > 64 and (g == 3.0).all()
    rc, nbytes, g = attempt(16, "nhwc")
    assert rc == 0 and not (g == 3.0).all()


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm(tA, tB, dtype):
    rng = np.random.default_rng(11)
    M, N, Kd = 37, 70, 129
    A, B = rnd(rng, M, Kd, dtype=dtype, scale=0.3), rnd(rng, Kd, N, dtype=dtype, scale=0.3)
    Cref = A.astype(np.float64) @ B.astype(np.float64)
    Ad = dev(A.T if tA else A, dtype)
    Bd = dev(B.T if tB else B, dtype)
    Cd = dev(np.ones((M, N), np.float32), dtype)
    code = K.HALF if dtype == torch.float16 else K.FLOAT
    K.check(K.lib().saga_hip_gemm(tA, tB, M, N, Kd, 1.0, K.ptr(Ad), Ad.shape[1], K.ptr(Bd), Bd.shape[1], 1.0, K.ptr(Cd),
                                  N, code, S()))
    assert_close(host(Cd), Cref + 1, dtype, "gemm")


def test_fc_golden(golden):
    g = golden["ops"]
    x, w = T(g, "fc2_input_x"), T(g, "fc2_input_w")  # transW: w is [out, in]
    xd, wd = dev(x), dev(w)
    yd = dev(np.zeros((2, 8), np.float32))
    K.check(K.lib().saga_hip_gemm(0, 1, 2, 8, 32, 1.0, K.ptr(xd), 32, K.ptr(wd), 32, 0.0, K.ptr(yd), 8, K.FLOAT, S()))
    assert float(((host(yd) - T(g, "fc2_output_no_bias")) ** 2).sum()) <= 1e-4
    x, w = T(g, "fc1_input_x"), T(g, "fc1_input_w")
    xd, wd, yd = dev(x), dev(w), dev(np.zeros((2, 3), np.float32))
    K.check(K.lib().saga_hip_gemm(0, 0, 2, 3, 2, 1.0, K.ptr(xd), 2, K.ptr(wd), 3, 0.0, K.ptr(yd), 3, K.FLOAT, S()))
    assert float(((host(yd) - T(g, "fc1_output_no_bias")) ** 2).sum()) <= 1e-4


def _bn_params(rng, Cc):
    s = (rng.standard_normal(Cc) * 0.5 + 1).astype(np.float32)
    b = rng.standard_normal(Cc).astype(np.float32)
    m = (rng.standard_normal(Cc) * 0.1).astype(np.float32)
    v = rng.uniform(0.5, 1.5, Cc).astype(np.float32)
    return s, b, m, v


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("layout,padc", LAYOUTS)
@pytest.mark.parametrize("flags", [0, K.BN_RELU, K.BN_RELU | K.BN_ADD])
@pytest.mark.parametrize("shape", [(4, 16, 6, 6), (3, 10, 5, 7), (2, 64, 9, 9)])
def test_batchnorm(shape, flags, layout, padc, dtype):
    rng = np.random.default_rng(sum(shape) + flags)
    Cc = shape[1]
    x = rnd(rng, *shape, dtype=dtype) * 2 + 3  # mean far from zero: exercises the shifted statistics
    if dtype == torch.float16:
        x = x.astype(np.float16).astype(np.float32)
    z = rnd(rng, *shape, dtype=dtype)
    s, b, m, v = _bn_params(rng, Cc)
    L = K.lib()
    xd, zd = dev(x, dtype, layout, padc), dev(z, dtype, layout, padc)
    sd, bd, md, vd = (dev(t) for t in (s, b, m, v))
    zarg = C.byref(K.view(zd)) if flags & K.BN_ADD else None

    def post(y):
        if flags & K.BN_ADD:
            y = y + z
        if flags & K.BN_RELU:
            y = ref.act_fwd(y)
        return y

    # inference
    yd = dev(np.zeros(shape, np.float32), dtype, layout, padc)
    K.check(L.saga_hip_bn_infer(C.byref(K.view(xd)), zarg, C.byref(K.view(yd)), K.ptr(sd), K.ptr(bd), K.ptr(md),
                                K.ptr(vd), 1e-5, flags, S()))
    assert_close(host(yd), post(ref.bn_infer(x, s, b, m, v)), dtype, "bn infer")

    # training forward
    ws = K.bn_workspace(xd)
    sm, sv = dev(np.zeros(Cc, np.float32)), dev(np.zeros(Cc, np.float32))
    K.check(L.saga_hip_bn_train_fwd(C.byref(K.view(xd)), zarg, C.byref(K.view(yd)), K.ptr(sd), K.ptr(bd), K.ptr(md),
                                    K.ptr(vd), K.ptr(sm), K.ptr(sv), 1e-5, 0.1, flags, K.ptr(ws), ws.numel(), S()))
    y_bn, rsm, rsv, rm, rv = ref.bn_train_fwd(x, s, b, m, v, 1e-5, 0.1)
    y_ref = post(y_bn)
    assert_close(host(yd), y_ref, dtype, "bn train y")
    assert_close(host(sm), rsm, torch.float32, "saved mean", 1e-4 if dtype == torch.float32 else 1e-3)
    assert_close(host(sv), rsv, torch.float32, "saved invstd", 1e-4 if dtype == torch.float32 else 1e-3)
    assert_close(host(md), rm, torch.float32, "running mean", 1e-4 if dtype == torch.float32 else 1e-3)
    assert_close(host(vd), rv, torch.float32, "running var", 1e-4 if dtype == torch.float32 else 1e-3)

    # backward (uses the oracle's saved statistics so both sides see identical inputs)
    dy = rnd(rng, *shape, dtype=dtype)
    y_h = ref.round_half(y_ref) if dtype == torch.float16 else y_ref
    dyp = dy * (y_h > 0) if flags & K.BN_RELU else dy
    dx_ref, ds_ref, db_ref = ref.bn_bwd(x, dyp, s, rsm, rsv)
    dxd = dev(np.ones(shape, np.float32), dtype, layout, padc)
    dzd = dev(np.zeros(shape, np.float32), dtype, layout, padc)
    dsd, dbd = dev(np.zeros(Cc, np.float32)), dev(np.zeros(Cc, np.float32))
    y_in = dev(y_h, dtype, layout, padc)
    dyd, rsmd, rsvd = dev(dy, dtype, layout, padc), dev(rsm), dev(rsv)  # named: the kernel reads them after this line
    K.check(L.saga_hip_bn_bwd(C.byref(K.view(xd)), C.byref(K.view(y_in)) if flags & K.BN_RELU else None,
                              C.byref(K.view(dyd)), C.byref(K.view(dxd)),
                              C.byref(K.view(dzd)) if flags & K.BN_ADD else None, K.ptr(sd), K.ptr(rsmd),
                              K.ptr(rsvd), K.ptr(dsd), K.ptr(dbd), 1.0, 0.0, 0.0, flags, K.ptr(ws), ws.numel(), S()))
    assert_close(host(dxd), dx_ref + 1, dtype, "bn dx (beta=1)")
    assert_close(host(dsd), ds_ref, torch.float32, "bn ds", 1e-4 if dtype == torch.float32 else 5e-3)
    assert_close(host(dbd), db_ref, torch.float32, "bn db", 1e-4 if dtype == torch.float32 else 5e-3)
    if flags & K.BN_ADD:
        assert_close(host(dzd), dyp, dtype, "bn dz")
    if flags & K.BN_RELU and not flags & K.BN_ADD:
        # with the bias, the mask comes from x (y = NULL): same gradients.  The mask is rebuilt from
        # the statistics passed in, so the forward's own statistics and output are used here.
        y_own = host(yd)
        dyp2 = dy * (y_own > 0)
        dx2_ref, ds2_ref, db2_ref = ref.bn_bwd(x, dyp2, s, host(sm), host(sv))
        dx2 = dev(np.zeros(shape, np.float32), dtype, layout, padc)
        y_arg = None if layout.startswith("nhwc") else C.byref(K.view(yd))  # only channels-last can do without y
        K.check(L.saga_hip_bn_bwd_ex(C.byref(K.view(xd)), y_arg, C.byref(K.view(dyd)), C.byref(K.view(dx2)), None,
                                     K.ptr(sd), K.ptr(bd), K.ptr(sm), K.ptr(sv), K.ptr(dsd), K.ptr(dbd), 0.0, 0.0,
                                     0.0, flags, None, K.ptr(ws), ws.numel(), S()))
        assert_close(host(dx2), dx2_ref, dtype, "bn dx (mask from x)")
        assert_close(host(dsd), ds2_ref, torch.float32, "bn ds (mask from x)", 1e-4 if dtype == torch.float32 else 5e-3)
        assert_close(host(dbd), db2_ref, torch.float32, "bn db (mask from x)", 1e-4 if dtype == torch.float32 else 5e-3)


def test_batchnorm_golden(golden):
    g = golden["ops"]
    x = T(g, "batchnorm_input_x")
    for layout in ("nchw", "nhwc"):
        xd = dev(x, torch.float32, layout)
        yd = dev(np.zeros_like(x), torch.float32, layout)
        p = [dev(T(g, "batchnorm_input_" + n)) for n in "sbmv"]
        K.check(K.lib().saga_hip_bn_infer(C.byref(K.view(xd)), None, C.byref(K.view(yd)), K.ptr(p[0]), K.ptr(p[1]),
                                          K.ptr(p[2]), K.ptr(p[3]), 1e-5, 0, S()))
        assert float(((host(yd) - T(g, "batchnorm_output")) ** 2).sum()) <= 1e-4


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("layout,padc", LAYOUTS)
@pytest.mark.parametrize("mode", ["relu", "sigmoid", "tanh", "swish", "leakyrelu"])
def test_activation(mode, layout, padc, dtype):
    rng = np.random.default_rng(2)
    shape = (2, 16, 5, 5)
    x, dy = rnd(rng, *shape, dtype=dtype), rnd(rng, *shape, dtype=dtype)
    alpha = 0.01 if mode == "leakyrelu" else 0.0
    code = ["relu", "sigmoid", "tanh", "swish", "leakyrelu"].index(mode)
    xd = dev(x, dtype, layout, padc)
    yd = dev(np.zeros(shape, np.float32), dtype, layout, padc)
    K.check(K.lib().saga_hip_act_fwd(code, alpha, C.byref(K.view(xd)), C.byref(K.view(yd)), 0.0, S()))
    y_ref = ref.act_fwd(x, mode, alpha)
    assert_close(host(yd), y_ref, dtype, "act fwd")
    dxd = dev(np.ones(shape, np.float32), dtype, layout, padc)
    dyd = dev(dy, dtype, layout, padc)
    K.check(K.lib().saga_hip_act_bwd(code, alpha, C.byref(K.view(xd)), C.byref(K.view(yd)), C.byref(K.view(dyd)),
                                     C.byref(K.view(dxd)), 1.0, S()))
    assert_close(host(dxd), ref.act_bwd(x, host(yd), dy, mode, alpha) + 1, dtype, "act bwd")


def test_relu_golden_and_nan(golden):
    g = golden["ops"]
    x = T(g, "relu_input")
    xd, yd = dev(x), dev(np.zeros_like(x))
    K.check(K.lib().saga_hip_act_fwd(0, 0.0, C.byref(K.view(xd)), C.byref(K.view(yd)), 0.0, S()))
    np.testing.assert_array_equal(host(yd), T(g, "relu_output"))
    xd = dev(np.array([[np.nan, -1.0, 2.0]], np.float32))
    yd = dev(np.zeros((1, 3), np.float32))
    K.check(K.lib().saga_hip_act_fwd(0, 0.0, C.byref(K.view(xd)), C.byref(K.view(yd)), 0.0, S()))
    r = host(yd)
    assert np.isnan(r[0, 0]) and r[0, 1] == 0 and r[0, 2] == 2


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("layout,padc", LAYOUTS)
@pytest.mark.parametrize("k,pad,stride,H", [(2, 0, 2, 8), (3, 1, 2, 9), (3, 1, 1, 6), (7, 0, 1, 7), (40, 0, 1, 40),
                                            (32, 2, 4, 44)])
def test_pooling(k, pad, stride, H, layout, padc, dtype):
    rng = np.random.default_rng(k * 10 + H)
    shape = (2, 16, H, H)
    x = rnd(rng, *shape, dtype=dtype)
    x = np.maximum(x, 0)  # post-relu data: many exact ties at 0 stress the first-index rule
    P = ref.pool_out(H, k, pad, stride)
    oshape = (2, 16, P, P)
    dy = rnd(rng, *oshape, dtype=dtype)
    L = K.lib()
    xd = dev(x, dtype, layout, padc)
    for mode, code in (("max", K.POOL_MAX), ("avg", K.POOL_AVG)):
        yd = dev(np.zeros(oshape, np.float32), dtype, layout, padc)
        idx = torch.zeros(oshape, dtype=torch.int32, device="cuda")
        K.check(L.saga_hip_pool_fwd(code, C.byref(K.view(xd)), C.byref(K.view(yd)),
                                    C.byref(K.view(idx)) if mode == "max" else None, k, pad, stride, S()))
        if mode == "max":
            y_ref, idx_ref = ref.maxpool_fwd(x, k, pad, stride, with_idx=True)
            np.testing.assert_array_equal(host(yd), y_ref)  # max is exact in any precision
            np.testing.assert_array_equal(idx.cpu().numpy(), idx_ref)  # pooling indices bit-exact
            dx_ref = ref.maxpool_bwd(x, dy, k, pad, stride)
        else:
            assert_close(host(yd), ref.avgpool_fwd(x, k, pad, stride), dtype, "avgpool")
            dx_ref = ref.avgpool_bwd(dy, shape, k, pad, stride)
        dxd = dev(np.ones(shape, np.float32), dtype, layout, padc)
        dyd = dev(dy, dtype, layout, padc)
        K.check(L.saga_hip_pool_bwd(code, C.byref(K.view(xd)), C.byref(K.view(yd)), C.byref(K.view(dyd)),
                                    C.byref(K.view(dxd)), k, pad, stride, 1.0, S()))
        assert_close(host(dxd), dx_ref + 1, dtype, mode + "pool bwd")


# (k, pad, stride, H, W, C); the last three: image rows in strips of 2, 1 and 7 output rows, the last strip short
POOL_CODE_CASES = [(2, 0, 2, 8, 9, 16), (3, 1, 2, 9, 10, 16), (3, 1, 2, 12, 13, 16), (3, 0, 2, 11, 12, 16), (3, 0, 2, 8, 9, 16),
                   (3, 1, 1, 6, 7, 16), (3, 0, 3, 10, 11, 16), (2, 1, 1, 5, 6, 16),
                   (3, 1, 2, 37, 112, 64), (3, 1, 2, 10, 75, 128), (3, 1, 2, 43, 300, 8)]


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("padc", [0, 8])
@pytest.mark.parametrize("k,pad,stride,H,W,Cc", POOL_CODE_CASES)
def test_maxpool_with_position_codes(k, pad, stride, H, W, Cc, padc, dtype):
    """The training pair saga_hip_maxpool_fwd_codes / _bwd_codes on channels-last tensors (dense and
    with a wider channel pitch): y and the recorded first-maximum positions bit-exact against the
    oracle's indices, dx against the oracle's backward - on post-relu data full of exact ties, with
    a NaN and with rows of -inf."""
    rng = np.random.default_rng(k * 100 + H + pad)
    shape = (3, Cc, H, W)
    x = np.maximum(rnd(rng, *shape, dtype=dtype), 0)
    x[0, 3, 1, 2] = np.nan
    x[1, 5] = -np.inf
    P, Q = ref.pool_out(H, k, pad, stride), ref.pool_out(W, k, pad, stride)
    oshape = (3, Cc, P, Q)
    dy = rnd(rng, *oshape, dtype=dtype)
    y_ref, idx_ref = ref.maxpool_fwd(x, k, pad, stride, with_idx=True)
    L = K.lib()
    xd = dev(x, dtype, "nhwc", padc)
    yd = dev(np.zeros(oshape, np.float32), dtype, "nhwc", padc)
    codes = torch.full((3, P, Q, Cc), 255, dtype=torch.uint8, device="cuda")
    K.check(L.saga_hip_maxpool_fwd_codes(C.byref(K.view(xd)), C.byref(K.view(yd)), K.ptr(codes), k, pad, stride, S()))
    np.testing.assert_array_equal(host(yd), y_ref)
    # code r*k+s -> input position (p*stride-pad+r)*W + (q*stride-pad+s), the oracle's index
    cd = codes.cpu().numpy().astype(np.int64).transpose(0, 3, 1, 2)
    pp, qq = np.meshgrid(np.arange(P), np.arange(Q), indexing="ij")
    pos = (pp * stride - pad + cd // k) * W + (qq * stride - pad + cd % k)
    np.testing.assert_array_equal(pos, idx_ref)
    dx_ref = ref.maxpool_bwd(x, dy, k, pad, stride)
    dyd = dev(dy, dtype, "nhwc", padc)
    for beta in (0.0, 1.0):
        dxd = dev(np.ones(shape, np.float32), dtype, "nhwc", padc)
        K.check(L.saga_hip_maxpool_bwd_codes(K.ptr(codes), C.byref(K.view(dyd)), C.byref(K.view(dxd)), k, pad, stride,
                                             beta, S()))
        assert_close(host(dxd), dx_ref + beta, dtype, "maxpool bwd from codes")
    # what the pair does not take is refused, not computed wrongly
    xn = dev(x, dtype, "nchw")
    yn = dev(np.zeros(oshape, np.float32), dtype, "nchw")
    rc = L.saga_hip_maxpool_fwd_codes(C.byref(K.view(xn)), C.byref(K.view(yn)), K.ptr(codes), k, pad, stride, S())
    assert rc == -3  # SAGA_HIP_EUNSUPPORTED


def test_maxpool_codes_on_zeros_of_both_signs_and_several_nans():
    """The fp16 3x3 / stride 2 pooling compares 16-bit order keys, not floats.  What a float comparison decides
    without being asked has to hold there too: -0 and +0 tie (the first one is the maximum), the first NaN of a
    window wins whatever its sign or payload and whatever follows it (+inf, a 'larger' NaN), a window of -inf
    reports its first position.  Positions bit-exact against the oracle's indices, values equal."""
    H, W, Cc = 7, 9, 8
    bits = np.full((2, Cc, H, W), 0xbc00, np.uint16)  # -1 everywhere
    neg0, pos0, pinf, ninf = 0x8000, 0x0000, 0x7c00, 0xfc00
    bits[0, 0, 2, 2], bits[0, 0, 2, 3] = neg0, pos0      # -0 first, then +0
    bits[0, 1, 2, 2], bits[0, 1, 2, 3] = pos0, neg0      # +0 first, then -0
    bits[0, 2, 2, 2], bits[0, 2, 2, 3] = 0xfe00, 0x7e00  # a negative NaN, then a positive one
    bits[0, 3, 2, 2], bits[0, 3, 2, 3] = 0x7c01, 0x7fff  # a signalling NaN, then the one with every bit set
    bits[0, 4, 2, 2], bits[0, 4, 2, 3] = pinf, 0x7e00    # +inf, then a NaN
    bits[0, 5, 2, 3], bits[0, 5, 3, 2] = 0xfe00, pinf    # a negative NaN, +inf a row below
    bits[0, 6] = ninf                                    # nothing but -inf
    bits[0, 7, 0, 0], bits[0, 7, 6, 8] = neg0, 0xffff    # in the corners, next to the padding
    bits[1] = bits[0][:, ::-1, ::-1]                     # and everything met from the other side
    x16 = bits.view(np.float16)
    x = x16.astype(np.float32)
    P, Q = ref.pool_out(H, 3, 1, 2), ref.pool_out(W, 3, 1, 2)
    y_ref, idx_ref = ref.maxpool_fwd(x, 3, 1, 2, with_idx=True)
    L = K.lib()
    for flags, fn in ((None, "plain"), (0, "norm"), (K.BN_RELU, "norm + relu")):
        xd = dev(x16, torch.float16, "nhwc")
        assert np.array_equal(xd.cpu().numpy().view(np.uint16), bits)
        yd = dev(np.zeros((2, Cc, P, Q), np.float32), torch.float16, "nhwc")
        codes = torch.full((2, P, Q, Cc), 255, dtype=torch.uint8, device="cuda")
        if flags is None:
            K.check(L.saga_hip_maxpool_fwd_codes(C.byref(K.view(xd)), C.byref(K.view(yd)), K.ptr(codes), 3, 1, 2, S()))
            want_y, want_idx = y_ref, idx_ref
        else:  # through the norm's arithmetic with scale 1 and shift 0
            ss = dev(np.concatenate([np.ones(Cc, np.float32), np.zeros(Cc, np.float32)]))
            K.check(L.saga_hip_maxpool_fwd_codes_bn(C.byref(K.view(xd)), C.byref(K.view(yd)), K.ptr(codes), 3, 1, 2,
                                                    K.ptr(ss), flags, S()))
            xr = np.where(np.isnan(x), x, np.maximum(x, 0)) if flags else x
            want_y, want_idx = ref.maxpool_fwd(xr, 3, 1, 2, with_idx=True)
        np.testing.assert_array_equal(host(yd), want_y, err_msg=fn)
        cd = codes.cpu().numpy().astype(np.int64).transpose(0, 3, 1, 2)
        pp, qq = np.meshgrid(np.arange(P), np.arange(Q), indexing="ij")
        pos = (pp * 2 - 1 + cd // 3) * W + (qq * 2 - 1 + cd % 3)
        np.testing.assert_array_equal(pos, want_idx, err_msg=fn)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("k,pad,stride,H,relu,W,Cw", [(3, 1, 2, 12, True, 13, 16), (3, 1, 2, 9, False, 10, 16), (2, 0, 2, 8, True, 9, 16),
                                                     (3, 0, 2, 11, True, 12, 16), (3, 1, 2, 37, True, 112, 64), (3, 1, 2, 10, False, 75, 128),
                                                     (3, 1, 2, 43, True, 300, 8)])
def test_maxpool_on_a_batch_norm_that_is_never_written(k, pad, stride, H, relu, W, Cw, dtype):
    """saga_hip_bn_train_fwd_partials with y NULL (statistics only, scale and shift left for the consumer) followed
    by saga_hip_maxpool_fwd_codes_bn, against the same two operators run one after the other with the normalised
    tensor in between: pooled values and position codes bit for bit, saved and running statistics equal."""
    rng = np.random.default_rng(k * 10 + H)
    Cc = Cw if dtype == torch.float16 else 8
    shape = (3, Cc, H, W)
    x = rnd(rng, *shape, dtype=dtype)
    P, Q = ref.pool_out(H, k, pad, stride), ref.pool_out(W, k, pad, stride)
    s, b = (1 + 0.3 * rng.standard_normal(Cc)).astype(np.float32), (0.2 * rng.standard_normal(Cc)).astype(np.float32)
    s[1] = -s[1]  # a negative scale: the maximum of the normalised values sits at the minimum of x
    L = K.lib()
    xd = dev(x, dtype, "nhwc")
    rows = 3 * H * W
    # partial sums as a producing convolution would leave them: two rows that add up to the sums over x
    xr = host(xd).astype(np.float64).transpose(0, 2, 3, 1).reshape(rows, Cc)
    half_rows = rows // 2
    part = np.stack([np.stack([xr[:half_rows].sum(0), (xr[:half_rows] ** 2).sum(0)], 1),
                     np.stack([xr[half_rows:].sum(0), (xr[half_rows:] ** 2).sum(0)], 1)]).astype(np.float32)
    partial = dev(part.reshape(-1))
    flags = K.BN_RELU if relu else 0

    def run(fused):
        sd, bd = dev(s), dev(b)
        md, vd = dev(np.zeros(Cc, np.float32)), dev(np.ones(Cc, np.float32))
        sm, sv = dev(np.zeros(Cc, np.float32)), dev(np.zeros(Cc, np.float32))
        ws = torch.zeros(2 * Cc, dtype=torch.float32, device="cuda")
        yp = dev(np.zeros((3, Cc, P, Q), np.float32), dtype, "nhwc")
        codes = torch.full((3, P, Q, Cc), 255, dtype=torch.uint8, device="cuda")
        if fused:
            K.check(L.saga_hip_bn_train_fwd_partials(C.byref(K.view(xd)), None, None, K.ptr(sd), K.ptr(bd), K.ptr(md),
                                                     K.ptr(vd), K.ptr(sm), K.ptr(sv), 1e-5, 0.1, flags, K.ptr(partial), 2,
                                                     None, K.ptr(ws), ws.numel() * 4, S()))
            K.check(L.saga_hip_maxpool_fwd_codes_bn(C.byref(K.view(xd)), C.byref(K.view(yp)), K.ptr(codes), k, pad, stride,
                                                    K.ptr(ws), flags, S()))
        else:
            yd = dev(np.zeros(shape, np.float32), dtype, "nhwc")
            K.check(L.saga_hip_bn_train_fwd_partials(C.byref(K.view(xd)), None, C.byref(K.view(yd)), K.ptr(sd), K.ptr(bd),
                                                     K.ptr(md), K.ptr(vd), K.ptr(sm), K.ptr(sv), 1e-5, 0.1, flags,
                                                     K.ptr(partial), 2, None, K.ptr(ws), ws.numel() * 4, S()))
            K.check(L.saga_hip_maxpool_fwd_codes(C.byref(K.view(yd)), C.byref(K.view(yp)), K.ptr(codes), k, pad, stride, S()))
        return host(yp), codes.cpu().numpy(), [host(t) for t in (md, vd, sm, sv)]

    y1, c1, st1 = run(True)
    y0, c0, st0 = run(False)
    np.testing.assert_array_equal(y1, y0)
    np.testing.assert_array_equal(c1, c0)
    for a_, b_ in zip(st1, st0):
        np.testing.assert_array_equal(a_, b_)
    # and against the oracle: batch norm, relu, max pooling
    mean, var = xr.mean(0), xr.var(0)
    yn = (host(xd).astype(np.float64) - mean[None, :, None, None]) / np.sqrt(var + 1e-5)[None, :, None, None]
    yn = yn * s[None, :, None, None] + b[None, :, None, None]
    if relu:
        yn = np.maximum(yn, 0)
    want = ref.maxpool_fwd(ref.round_half(yn.astype(np.float32)) if dtype == torch.float16 else yn.astype(np.float32), k, pad, stride)
    assert_close(y1, want, dtype, "pooled batch norm")


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("pad,H,W,relu,beta", [(1, 12, 14, True, 0.0), (1, 9, 11, True, 1.0), (1, 16, 16, False, 0.0), (0, 11, 13, True, 0.0)])
def test_batch_norm_backward_through_a_max_pooling(pad, H, W, relu, beta, dtype):
    """saga_hip_bn_bwd_pooled - the backward of a max pooling (3x3, stride 2) and of the batch norm (+ relu) in front
    of it without the gradient tensor between them - against saga_hip_maxpool_bwd_codes followed by
    saga_hip_bn_bwd_ex: dx equal to the last bit or two of the type, ds and db to 1e-5."""
    rng = np.random.default_rng(H * 31 + W + pad)
    Cc = 16 if dtype == torch.float16 else 8
    N = 3
    shape = (N, Cc, H, W)
    x = rnd(rng, *shape, dtype=dtype)
    P, Q = ref.pool_out(H, 3, pad, 2), ref.pool_out(W, 3, pad, 2)
    s, b = (1 + 0.3 * rng.standard_normal(Cc)).astype(np.float32), (0.2 * rng.standard_normal(Cc)).astype(np.float32)
    flags = K.BN_RELU if relu else 0
    L = K.lib()
    xd = dev(x, dtype, "nhwc")
    xh = host(xd).astype(np.float64)
    mean, var = xh.mean((0, 2, 3)), xh.var((0, 2, 3))
    sm, sv = dev(mean.astype(np.float32)), dev((1.0 / np.sqrt(var + 1e-5)).astype(np.float32))
    sd, bd = dev(s), dev(b)
    # forward: the norm's output and the pooling's codes, by the unfused operators
    yd = dev(np.zeros(shape, np.float32), dtype, "nhwc")
    md, vd = dev(mean.astype(np.float32)), dev(var.astype(np.float32))
    K.check(L.saga_hip_bn_infer(C.byref(K.view(xd)), None, C.byref(K.view(yd)), K.ptr(sd), K.ptr(bd), K.ptr(md), K.ptr(vd),
                                1e-5, flags, S()))
    yp = dev(np.zeros((N, Cc, P, Q), np.float32), dtype, "nhwc")
    codes = torch.full((N, P, Q, Cc), 255, dtype=torch.uint8, device="cuda")
    K.check(L.saga_hip_maxpool_fwd_codes(C.byref(K.view(yd)), C.byref(K.view(yp)), K.ptr(codes), 3, pad, 2, S()))
    dp = rnd(rng, N, Cc, P, Q, dtype=dtype)
    dpd = dev(dp, dtype, "nhwc")
    init = rnd(rng, *shape, dtype=dtype)

    # unfused: pooling backward into dy, then the norm's backward
    dyd = dev(np.zeros(shape, np.float32), dtype, "nhwc")
    K.check(L.saga_hip_maxpool_bwd_codes(K.ptr(codes), C.byref(K.view(dpd)), C.byref(K.view(dyd)), 3, pad, 2, 0.0, S()))
    dx0 = dev(init, dtype, "nhwc")
    ds0, db0 = dev(np.ones(Cc, np.float32)), dev(np.ones(Cc, np.float32))
    wsb = torch.zeros(L.saga_hip_bn_workspace_size(C.byref(K.view(xd))), dtype=torch.uint8, device="cuda")
    K.check(L.saga_hip_bn_bwd_ex(C.byref(K.view(xd)), None if relu else None, C.byref(K.view(dyd)), C.byref(K.view(dx0)), None,
                                 K.ptr(sd), K.ptr(bd), K.ptr(sm), K.ptr(sv), K.ptr(ds0), K.ptr(db0), beta, 0.0, 0.0, flags,
                                 None, K.ptr(wsb), wsb.numel(), S()))
    # fused
    need = L.saga_hip_bn_bwd_pooled_workspace_size(C.byref(K.view(xd)), C.byref(K.view(dpd)), 3, pad, 2)
    assert need > 0
    ws = torch.full((need,), 0x7f, dtype=torch.uint8, device="cuda")
    dx1 = dev(init, dtype, "nhwc")
    ds1, db1 = dev(np.ones(Cc, np.float32)), dev(np.ones(Cc, np.float32))
    K.check(L.saga_hip_bn_bwd_pooled(C.byref(K.view(xd)), C.byref(K.view(dpd)), K.ptr(codes), C.byref(K.view(dx1)), K.ptr(sd),
                                     K.ptr(bd), K.ptr(sm), K.ptr(sv), K.ptr(ds1), K.ptr(db1), beta, 0.0, flags, 3, pad, 2,
                                     K.ptr(ws), need, S()))
    np.testing.assert_allclose(host(ds1), host(ds0), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(host(db1), host(db0), rtol=1e-5, atol=1e-5)
    assert_close(host(dx1), host(dx0), dtype, "dx", 2e-3 if dtype == torch.float16 else 1e-5)
    # what it does not take is refused by the size query and by the call
    assert L.saga_hip_bn_bwd_pooled_workspace_size(C.byref(K.view(xd)), C.byref(K.view(dpd)), 2, pad, 2) == 0


def test_pooling_golden(golden):
    g = golden["ops"]
    x = T(g, "pooling_input")
    for layout in ("nchw", "nhwc"):
        xd = dev(x, torch.float32, layout)
        for code, k, st, name in ((K.POOL_MAX, 2, 2, "maxpool_output"), (K.POOL_MAX, 8, 1, "maxpool_output_global"),
                                  (K.POOL_AVG, 2, 2, "avgpool_output"), (K.POOL_AVG, 8, 1, "avgpool_output_global")):
            want = T(g, name)
            yd = dev(np.zeros_like(want), torch.float32, layout)
            K.check(K.lib().saga_hip_pool_fwd(code, C.byref(K.view(xd)), C.byref(K.view(yd)), None, k, 0, st, S()))
            assert float(((host(yd) - want) ** 2).sum()) <= 1e-4, name


@pytest.mark.parametrize("dtype", DT)
def test_add_axpby_convert_concat(dtype, golden):
    rng = np.random.default_rng(9)
    shape = (2, 8, 4, 4)
    a, b = rnd(rng, *shape, dtype=dtype), rnd(rng, *shape, dtype=dtype)
    L = K.lib()
    for la, lb, lo in (("nchw", "nchw", "nchw"), ("nhwc", "nhwc", "nhwc"), ("nhwc", "nchw", "nhwc")):
        ad, bd, od = dev(a, dtype, la), dev(b, dtype, lb, 8 if lb == "nhwc" else 0), dev(np.zeros(shape), dtype, lo)
        K.check(L.saga_hip_add(C.byref(K.view(ad)), C.byref(K.view(bd)), C.byref(K.view(od)), S()))
        assert_close(host(od), a + b, dtype, "add")
        K.check(L.saga_hip_axpby(C.byref(K.view(ad)), C.byref(K.view(od)), 1.0, 1.0, S()))
        assert_close(host(od), 2 * a + b, dtype, "axpby")
    # concat realised as strided outputs: two producers write channel slices of one NHWC buffer
    g = golden["ops"]
    x0, x1 = T(g, "concat_input_x0"), T(g, "concat_input_x1")
    wide = torch.zeros((2, 4, 4, 4), dtype=dtype, device="cuda")  # N,H,W,C
    for i, src in enumerate((x0, x1)):
        sl = wide[..., 2 * i:2 * i + 2].permute(0, 3, 1, 2)
        srcd = dev(src, dtype, "nhwc")
        K.check(L.saga_hip_axpby(C.byref(K.view(srcd)), C.byref(K.view(sl)), 1.0, 0.0, S()))
        torch.cuda.synchronize()
    got = host(wide.permute(0, 3, 1, 2))
    assert float(((got - T(g, "concat_output")) ** 2).sum()) <= (1e-4 if dtype == torch.float32 else 1e-3)
    # u8 -> float/half with scale
    u = rng.integers(0, 256, shape).astype(np.uint8)
    ud = torch.from_numpy(u).cuda()
    od = dev(np.zeros(shape), dtype, "nhwc")
    K.check(L.saga_hip_convert(C.byref(K.view(ud)), C.byref(K.view(od)), 1 / 255.0, S()))
    assert_close(host(od), u.astype(np.float32) / 255.0, dtype, "convert")


@pytest.mark.parametrize("dtype", DT)
def test_softmax(dtype):
    rng = np.random.default_rng(4)
    x = rnd(rng, 2, 8, 5, 5, dtype=dtype, scale=3)
    for layout in ("nchw", "nhwc"):
        xd, yd = dev(x, dtype, layout), dev(np.zeros_like(x), dtype, layout)
        K.check(K.lib().saga_hip_softmax(C.byref(K.view(xd)), C.byref(K.view(yd)), S()))
        assert_close(host(yd), ref.softmax(x), dtype, "softmax")


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("shape,out", [((3, 1, 28, 28), (224, 224)), ((2, 3, 32, 32), (32, 32)), ((2, 5, 9, 7), (4, 13))])
def test_spatial_transform(shape, out, dtype):
    """Resize with the identity matrix (what the classifier harness does in front of ResNet-50) and
    random affine maps that reach outside the image."""
    rng = np.random.default_rng(shape[2] + out[0])
    x = rnd(rng, *shape, dtype=dtype)
    ident = np.tile(np.array([[1, 0, 0], [0, 1, 0]], np.float32), (shape[0], 1, 1))
    for theta in (ident, ident + rng.normal(0, 0.3, ident.shape).astype(np.float32)):
        want = ref.spatial_transform(x, theta, *out)
        td = torch.from_numpy(theta).cuda()
        for layout in ("nchw", "nhwc"):
            xd = dev(x, dtype, layout)
            yd = dev(np.zeros((shape[0], shape[1]) + out, np.float32), dtype, layout)
            K.check(K.lib().saga_hip_spatial_transform(C.byref(K.view(xd)), K.ptr(td), C.byref(K.view(yd)), S()))
            assert_close(host(yd), want, dtype, "spatial transform")


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("N,Cc", [(7, 10), (64, 1000), (5, 65)])
def test_catclassifier(N, Cc, dtype):
    rng = np.random.default_rng(N + Cc)
    x = rnd(rng, N, Cc, dtype=dtype, scale=3)
    x[1, 3] = x[1, Cc - 2] = x[1].max() + 1  # tie -> first index
    if N > 2:
        x[2, :] = 0.5  # all equal -> label 0
    labels = rng.integers(0, Cc, N).astype(np.int32)
    xd = dev(x, dtype)
    pred = torch.zeros(N, dtype=torch.int32, device="cuda")
    L = K.lib()
    K.check(L.saga_hip_catclassifier_fwd(C.byref(K.view(xd)), K.ptr(pred), S()))
    pred_ref = ref.catclassifier_fwd(x)
    np.testing.assert_array_equal(pred.cpu().numpy(), pred_ref)  # labels bit-exact
    scale = 1.0 / N if dtype == torch.float32 else 1024.0 / N
    dxd = dev(np.zeros_like(x), dtype)
    loss = torch.zeros(N, dtype=torch.float32, device="cuda")
    labd = torch.from_numpy(labels).cuda()
    K.check(L.saga_hip_catclassifier_bwd(C.byref(K.view(xd)), C.byref(K.view(dxd)), K.ptr(pred), K.ptr(labd),
                                         K.ptr(loss), scale, S()))
    dx_ref, loss_ref = ref.catclassifier_bwd(x, pred_ref, labels, scale)
    assert_close(host(dxd), dx_ref, dtype, "catclassifier dx")
    assert_close(host(loss), loss_ref, torch.float32, "loss", 1e-5)


def test_adam_f32_100_steps():
    rng = np.random.default_rng(1)
    n = 10007
    w = rng.standard_normal(n).astype(np.float32)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    wd, md, vd = dev(w), dev(m), dev(v)
    aux = torch.zeros(4, dtype=torch.int32, device="cuda")
    L = K.lib()
    for t in range(1, 101):
        g = (rng.standard_normal(n) * 0.1).astype(np.float32)
        b1t, b2t = ref.adam_bias_terms(t)
        gd = dev(g)
        K.check(L.saga_hip_adam_f32(n, K.ptr(wd), K.ptr(gd), K.ptr(md), K.ptr(vd), float(b1t), float(b2t), 1e-3, 1e-4,
                                    K.ptr(aux), S()))
        torch.cuda.synchronize()
        ref.adam_f32(w, g, m, v, t, 1e-3, 1e-4)
    assert_close(host(wd), w, torch.float32, "adam weights after 100 steps", 1e-5)
    assert aux.cpu().tolist() == [0, 0, 0, 0]
    g = np.zeros(n, np.float32)
    g[5], g[n - 1] = np.inf, np.nan  # vector body and scalar tail
    before = host(wd).copy()
    gd = dev(g)
    K.check(L.saga_hip_adam_f32(n, K.ptr(wd), K.ptr(gd), K.ptr(md), K.ptr(vd), 1.0, 1.0, 1e-3, 0.0, K.ptr(aux), S()))
    assert aux.cpu().tolist() == [0, 1, 1, 0]
    after = host(wd)
    assert after[5] == before[5] and after[n - 1] == before[n - 1]


def test_adam_mixed_100_steps():
    rng = np.random.default_rng(2)
    n = 4099
    scale = 256.0
    w16 = rng.standard_normal(n).astype(np.float16)
    c = w16.astype(np.float32)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    wbits = w16.view(np.uint16).copy()
    wd = torch.from_numpy(w16.copy()).cuda()
    cd, md, vd = dev(c), dev(m), dev(v)
    aux = torch.zeros(4, dtype=torch.int32, device="cuda")
    L = K.lib()
    for t in range(1, 101):
        g16 = (rng.standard_normal(n) * 0.1 * scale).astype(np.float16)
        b1t, b2t = ref.adam_bias_terms(t)
        gd = torch.from_numpy(g16).cuda()
        K.check(L.saga_hip_adam_mixed(n, float(np.float32(1.0) / np.float32(scale)), K.ptr(wd), K.ptr(gd), K.ptr(md),
                                      K.ptr(vd), K.ptr(cd), float(b1t), float(b2t), 1e-3, 1e-4, K.ptr(aux), S()))
        torch.cuda.synchronize()
        ref.adam_mixed(wbits, g16.view(np.uint16), m, v, c, t, 1e-3, scale, 1e-4)
    assert_close(host(cd), c, torch.float32, "adam master weights after 100 steps", 1e-5)
    got16 = wd.cpu().numpy().view(np.uint16).astype(np.int32)
    assert np.abs(got16 - wbits.astype(np.int32)).max() <= 1  # fp16 copies agree to one ulp
    assert aux.cpu().tolist() == [0, 0, 0, 0]
    gbad = np.zeros(n, np.uint16)
    gbad[0], gbad[1], gbad[n - 1] = 0x7800, 0x7c00, 0x7e00
    gd = torch.from_numpy(gbad.view(np.float16)).cuda()
    K.check(L.saga_hip_adam_mixed(n, 1.0, K.ptr(wd), K.ptr(gd), K.ptr(md), K.ptr(vd), K.ptr(cd), 1.0, 1.0, 1e-3, 0.0,
                                  K.ptr(aux), S()))
    assert aux.cpu().tolist() == [1, 1, 1, 0]


def test_fill():
    t = torch.zeros(1000003, dtype=torch.uint8, device="cuda")
    K.check(K.lib().saga_hip_fill(C.c_void_p(t.data_ptr() + 3), 0xAB, 1000000 - 3, S()))
    h = t.cpu().numpy()
    assert (h[3:1000000] == 0xAB).all() and (h[:3] == 0).all() and (h[1000000:] == 0).all()


def test_rejects_bad_arguments():
    x = dev(np.zeros((1, 4, 4, 4), np.float32))
    y = dev(np.zeros((1, 4, 3, 3), np.float32))
    w = dev(np.zeros((4, 4, 3, 3), np.float32))
    with pytest.raises(K.SagaHipError):
        K.conv2d(K.CONV_FWD, x, w, y, pad=0)  # y should be 2x2
    # an input smaller than the dilated filter has no output position at all: 4 + 0 < (3 - 1) * 3 + 1 with
    # stride 2 would come out as one position if the shape rule's division truncated toward zero
    y1 = dev(np.zeros((1, 4, 1, 1), np.float32))
    p = K.ConvParams(0, 2, 3, 1)
    assert K.lib().saga_hip_conv2d_fwd(C.byref(K.view(x)), C.byref(K.view(w)), C.byref(K.view(y1)), C.byref(p), 1.0, 0.0,
                                       None, 0, S()) == -2
    assert K.lib().saga_hip_act_fwd(99, 0.0, C.byref(K.view(x)), C.byref(K.view(x)), 0.0, S()) == -1


RESNET_SHAPES = [
    # C, H, K, R, stride, pad   (rows of the ResNet-50 v1.5 shape list, batch reduced to 2)
    (64, 56, 64, 3, 1, 1),
    (64, 56, 256, 1, 1, 0),
    (256, 56, 64, 1, 1, 0),
    (128, 56, 128, 3, 2, 1),
    (256, 56, 512, 1, 2, 0),
    (512, 7, 512, 3, 1, 1),
    (1024, 14, 2048, 1, 2, 0),
    (16, 32, 16, 3, 1, 1),
    (24, 9, 40, 3, 1, 1),
]


# N, C, H, W, K: 3x3 / stride 1 / pad 1 problems at the image sizes and channel counts of the residual stages
# (whole small images, ragged batches, output channels beyond / short of whole tiles, non-square images),
# forward and backward data with beta 0 and 1, dense and as channel slices
PATCH_CASES = [
    (3, 64, 56, 56, 64),
    (2, 128, 28, 28, 128),
    (3, 256, 14, 14, 256),
    (6, 512, 7, 7, 512),
    (5, 64, 7, 7, 72),
    (2, 64, 32, 32, 96),
    (2, 128, 16, 16, 264),
    (1, 192, 14, 14, 40),
    (2, 64, 28, 56, 64),
]


@pytest.mark.parametrize("padc", [0, 8])
@pytest.mark.parametrize("case", PATCH_CASES)
def test_conv3x3_stage_shapes(case, padc):
    N, Cc, H, W, Kk = case
    dtype = torch.float16
    rng = np.random.default_rng(N * 1000 + Cc + Kk + H)
    x = rnd(rng, N, Cc, H, W, dtype=dtype)
    w = rnd(rng, Kk, Cc, 3, 3, dtype=dtype, scale=(2.0 / (Cc * 9)) ** 0.5)
    y_ref = ref.conv2d_fwd(x, w, 1, 1)
    xd, wd = dev(x, dtype, "nhwc", padc), dev(w, dtype, "nhwc")
    yd = dev(np.full_like(y_ref, 7.0), dtype, "nhwc", padc)
    K.conv2d(K.CONV_FWD, xd, wd, yd, 1, 1)
    assert_close(host(yd), y_ref, dtype, "y", tol=2e-3)
    K.conv2d(K.CONV_FWD, xd, wd, yd, 1, 1, 1, 1, 1.0, 1.0)
    assert_close(host(yd), 2 * y_ref, dtype, "y beta=1", tol=3e-3)
    dy = rnd(rng, *y_ref.shape, dtype=dtype)
    dyd = dev(dy, dtype, "nhwc", padc)
    dxd = dev(np.full_like(x, 7.0), dtype, "nhwc", padc)
    K.conv2d(K.CONV_BWD_DATA, dyd, wd, dxd, 1, 1)
    dx_ref = ref.conv2d_bwd_data(dy, w, x.shape, 1, 1)
    assert_close(host(dxd), dx_ref, dtype, "dx", tol=2e-3)
    K.conv2d(K.CONV_BWD_DATA, dyd, wd, dxd, 1, 1, 1, 1, 1.0, 1.0)
    assert_close(host(dxd), 2 * dx_ref, dtype, "dx beta=1", tol=3e-3)


@pytest.mark.parametrize("shape", RESNET_SHAPES)
def test_conv_fp16_nhwc_network_shapes(shape):
    """fp16 NHWC at the real spatial sizes of the target networks: the MFMA implicit-GEMM path."""
    Cc, H, Kk, R, stride, pad = shape
    N, dtype = 2, torch.float16
    rng = np.random.default_rng(Cc + Kk + R)
    x = rnd(rng, N, Cc, H, H, dtype=dtype)
    w = rnd(rng, Kk, Cc, R, R, dtype=dtype, scale=(2.0 / (Cc * R * R)) ** 0.5)
    y_ref = ref.conv2d_fwd(x, w, pad, stride)
    dy = rnd(rng, *y_ref.shape, dtype=dtype)
    xd, wd = dev(x, dtype, "nhwc"), dev(w, dtype, "nhwc")
    yd = dev(np.zeros_like(y_ref), dtype, "nhwc")
    K.conv2d(K.CONV_FWD, xd, wd, yd, pad, stride)
    assert_close(host(yd), y_ref, dtype, "y")
    dyd = dev(dy, dtype, "nhwc")
    dxd = dev(np.zeros_like(x), dtype, "nhwc")
    K.conv2d(K.CONV_BWD_DATA, dyd, wd, dxd, pad, stride)
    assert_close(host(dxd), ref.conv2d_bwd_data(dy, w, x.shape, pad, stride), dtype, "dx")
    dwd = dev(np.zeros_like(w), dtype, "nhwc")
    K.conv2d(K.CONV_BWD_FILTER, xd, dyd, dwd, pad, stride)
    assert_close(host(dwd), ref.conv2d_bwd_filter(x, dy, w.shape, pad, stride), dtype, "dw")
