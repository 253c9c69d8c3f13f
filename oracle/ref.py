"""numpy front door of the CPU oracle (oracle/saga_oracle.c).  TEST INFRASTRUCTURE ONLY.

Every function takes and returns contiguous float32 numpy arrays in logical order (N,C,H,W /
N,C) and forwards to the C restatement.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import this module; the product (saga_amd/) never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libsaga_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = C.CDLL(path)
        _LIB.so_half_to_float.restype = C.c_float
        _LIB.so_half_to_float.argtypes = [C.c_uint16]
        _LIB.so_float_to_half.restype = C.c_uint16
        _LIB.so_float_to_half.argtypes = [C.c_float]
    return _LIB


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


_i = C.c_int
_fl = C.c_float
_sz = C.c_size_t


def conv_out(n, k, pad, stride, dil=1):
    return 1 + (n + 2 * pad - ((k - 1) * dil + 1)) // stride


def tconv_out(n, k, pad, stride, opad=0, dil=1):
    # src/node.cpp:65-69
    return stride * (n - 1) + opad + ((k - 1) * dil + 1) - 2 * pad


def pool_out(n, k, pad, stride):
    return 1 + (n + 2 * pad - k) // stride


def conv2d_fwd(x, w, pad=0, stride=1, dil=1, group=1, y=None, beta=0.0):
    x, w = _f(x), _f(w)
    N, Cc, H, W = x.shape
    K, Cg, R, S = w.shape
    assert Cg * group == Cc
    P, Q = conv_out(H, R, pad, stride, dil), conv_out(W, S, pad, stride, dil)
    if y is None:
        y = np.zeros((N, K, P, Q), np.float32)
    else:
        y = _f(y).copy()
    lib().so_conv2d_fwd(_p(x), _p(w), _p(y), _i(N), _i(Cc), _i(H), _i(W), _i(K), _i(R), _i(S), _i(pad),
                        _i(stride), _i(dil), _i(group), _fl(beta))
    return y


def conv2d_bwd_data(dy, w, xshape, pad=0, stride=1, dil=1, group=1, dx=None, beta=0.0):
    dy, w = _f(dy), _f(w)
    N, Cc, H, W = xshape
    K, Cg, R, S = w.shape
    assert dy.shape == (N, K, conv_out(H, R, pad, stride, dil), conv_out(W, S, pad, stride, dil)), \
        (dy.shape, xshape, w.shape)
    dx = np.zeros(xshape, np.float32) if dx is None else _f(dx).copy()
    lib().so_conv2d_bwd_data(_p(dy), _p(w), _p(dx), _i(N), _i(Cc), _i(H), _i(W), _i(K), _i(R), _i(S), _i(pad),
                             _i(stride), _i(dil), _i(group), _fl(beta))
    return dx


def conv2d_bwd_filter(x, dy, wshape, pad=0, stride=1, dil=1, group=1, dw=None, beta=0.0):
    x, dy = _f(x), _f(dy)
    N, Cc, H, W = x.shape
    K, Cg, R, S = wshape
    dw = np.zeros(wshape, np.float32) if dw is None else _f(dw).copy()
    lib().so_conv2d_bwd_filter(_p(x), _p(dy), _p(dw), _i(N), _i(Cc), _i(H), _i(W), _i(K), _i(R), _i(S), _i(pad),
                               _i(stride), _i(dil), _i(group), _fl(beta))
    return dw


def bias_add(y, b):
    y = _f(y).copy()
    b = _f(b).reshape(-1)
    N, K = y.shape[:2]
    lib().so_bias_add(_p(y), _p(b), _i(N), _i(K), _i(int(np.prod(y.shape[2:]))))
    return y


def bias_bwd(dy, db=None, beta=0.0):
    dy = _f(dy)
    N, K = dy.shape[:2]
    db = np.zeros(K, np.float32) if db is None else _f(db).copy()
    lib().so_bias_bwd(_p(dy), _p(db), _i(N), _i(K), _i(int(np.prod(dy.shape[2:]))), _fl(beta))
    return db


def fc_fwd(x, w, transW=False, y=None, beta=0.0):
    x, w = _f(x), _f(w)
    B, In = x.shape
    Out = w.shape[0] if transW else w.shape[1]
    assert (w.shape[1] if transW else w.shape[0]) == In
    y = np.zeros((B, Out), np.float32) if y is None else _f(y).copy()
    lib().so_fc_fwd(_p(x), _p(w), _p(y), _i(B), _i(In), _i(Out), _i(int(transW)), _fl(beta))
    return y


def fc_bwd_w(x, dy, transW=False, dw=None, beta=0.0):
    x, dy = _f(x), _f(dy)
    B, In = x.shape
    Out = dy.shape[1]
    shape = (Out, In) if transW else (In, Out)
    dw = np.zeros(shape, np.float32) if dw is None else _f(dw).copy()
    lib().so_fc_bwd_w(_p(x), _p(dy), _p(dw), _i(B), _i(In), _i(Out), _i(int(transW)), _fl(beta))
    return dw


def fc_bwd_x(dy, w, transW=False, dx=None, beta=0.0):
    dy, w = _f(dy), _f(w)
    B, Out = dy.shape
    In = w.shape[1] if transW else w.shape[0]
    dx = np.zeros((B, In), np.float32) if dx is None else _f(dx).copy()
    lib().so_fc_bwd_x(_p(dy), _p(w), _p(dx), _i(B), _i(In), _i(Out), _i(int(transW)), _fl(beta))
    return dx


def _nchw(x):
    N, Cc = x.shape[:2]
    return N, Cc, int(np.prod(x.shape[2:]))


def bn_infer(x, s, b, m, v, eps=1e-5):
    x = _f(x)
    s, b, m, v = (_f(t).reshape(-1) for t in (s, b, m, v))
    y = np.empty_like(x)
    N, Cc, HW = _nchw(x)
    lib().so_bn_infer(_p(x), _p(s), _p(b), _p(m), _p(v), _p(y), _i(N), _i(Cc), _i(HW), _fl(eps))
    return y


def bn_train_fwd(x, s, b, run_m=None, run_v=None, eps=1e-5, expavg=0.1):
    """returns y, save_mean, save_invstd, new_run_m, new_run_v"""
    x = _f(x)
    s, b = _f(s).reshape(-1), _f(b).reshape(-1)
    N, Cc, HW = _nchw(x)
    y = np.empty_like(x)
    sm = np.empty(Cc, np.float32)
    sv = np.empty(Cc, np.float32)
    rm = _f(run_m).reshape(-1).copy() if run_m is not None else None
    rv = _f(run_v).reshape(-1).copy() if run_v is not None else None
    lib().so_bn_train_fwd(_p(x), _p(s), _p(b), _p(rm), _p(rv), _p(y), _p(sm), _p(sv), _i(N), _i(Cc), _i(HW),
                          _fl(eps), _fl(expavg))
    return y, sm, sv, rm, rv


def bn_bwd(x, dy, s, save_mean, save_invstd, dx=None, beta_dx=0.0, ds=None, db=None, beta_p=0.0):
    x, dy = _f(x), _f(dy)
    s, sm, sv = (_f(t).reshape(-1) for t in (s, save_mean, save_invstd))
    N, Cc, HW = _nchw(x)
    dx = np.zeros_like(x) if dx is None else _f(dx).copy()
    ds = np.zeros(Cc, np.float32) if ds is None else _f(ds).reshape(-1).copy()
    db = np.zeros(Cc, np.float32) if db is None else _f(db).reshape(-1).copy()
    lib().so_bn_bwd(_p(x), _p(dy), _p(s), _p(sm), _p(sv), _p(dx), _p(ds), _p(db), _i(N), _i(Cc), _i(HW),
                    _fl(beta_dx), _fl(beta_p))
    return dx, ds, db


ACT = {"relu": 0, "sigmoid": 1, "tanh": 2, "swish": 3, "leakyrelu": 4, "elu": 0}


def act_fwd(x, mode="relu", alpha=0.0):
    x = _f(x)
    y = np.empty_like(x)
    lib().so_act_fwd(_p(x), _p(y), _sz(x.size), _i(ACT[mode]), _fl(alpha))
    return y


def act_bwd(x, y, dy, mode="relu", alpha=0.0, dx=None, beta=0.0):
    x, y, dy = _f(x), _f(y), _f(dy)
    dx = np.zeros_like(x) if dx is None else _f(dx).copy()
    lib().so_act_bwd(_p(x), _p(y), _p(dy), _p(dx), _sz(x.size), _i(ACT[mode]), _fl(alpha), _fl(beta))
    return dx


def maxpool_fwd(x, k, pad=0, stride=1, with_idx=False):
    x = _f(x)
    N, Cc, H, W = x.shape
    P, Q = pool_out(H, k, pad, stride), pool_out(W, k, pad, stride)
    y = np.empty((N, Cc, P, Q), np.float32)
    idx = np.empty((N, Cc, P, Q), np.int32)
    lib().so_maxpool_fwd(_p(x), _p(y), _p(idx), _i(N), _i(Cc), _i(H), _i(W), _i(k), _i(pad), _i(stride))
    return (y, idx) if with_idx else y


def maxpool_bwd(x, dy, k, pad=0, stride=1, dx=None, beta=0.0):
    x, dy = _f(x), _f(dy)
    N, Cc, H, W = x.shape
    dx = np.zeros_like(x) if dx is None else _f(dx).copy()
    lib().so_maxpool_bwd(_p(x), _p(dy), _p(dx), _i(N), _i(Cc), _i(H), _i(W), _i(k), _i(pad), _i(stride),
                         _fl(beta))
    return dx


def avgpool_fwd(x, k, pad=0, stride=1):
    x = _f(x)
    N, Cc, H, W = x.shape
    P, Q = pool_out(H, k, pad, stride), pool_out(W, k, pad, stride)
    y = np.empty((N, Cc, P, Q), np.float32)
    lib().so_avgpool_fwd(_p(x), _p(y), _i(N), _i(Cc), _i(H), _i(W), _i(k), _i(pad), _i(stride))
    return y


def avgpool_bwd(dy, xshape, k, pad=0, stride=1, dx=None, beta=0.0):
    dy = _f(dy)
    N, Cc, H, W = xshape
    dx = np.zeros(xshape, np.float32) if dx is None else _f(dx).copy()
    lib().so_avgpool_bwd(_p(dy), _p(dx), _i(N), _i(Cc), _i(H), _i(W), _i(k), _i(pad), _i(stride), _fl(beta))
    return dx


def loss_bwd(x, target, scale):
    """L2 loss node backward: returns dx (like x) and mmss [N,4]"""
    x, target = _f(x), _f(target)
    N = x.shape[0]
    c = int(np.prod(x.shape[1:]))
    dx = np.empty_like(x)
    mmss = np.zeros((N, 4), np.float32)
    lib().so_loss_bwd(_p(x), _p(target), _p(dx), _p(mmss), _i(N), _i(c), _fl(scale))
    return dx, mmss


def tensor_stats(x):
    """the stats node: {min(0,min), max(0,max), mean, variance}"""
    x = _f(x)
    out = np.zeros(4, np.float32)
    lib().so_tensor_stats(_p(x), _p(out), C.c_size_t(x.size))
    return out


def softmax(x):
    x = _f(x)
    N, Cc, HW = _nchw(x)
    y = np.empty_like(x)
    lib().so_softmax(_p(x), _p(y), _i(N), _i(Cc), _i(HW))
    return y


def spatial_transform(x, theta, oh, ow):
    """x [N,C,H,W], theta [N,2,3] -> [N,C,oh,ow]"""
    x, theta = _f(x), _f(theta)
    N, Cc, H, W = x.shape
    assert theta.shape == (N, 2, 3)
    y = np.empty((N, Cc, oh, ow), np.float32)
    lib().so_spatial_transform(_p(x), _p(theta), _p(y), _i(N), _i(Cc), _i(H), _i(W), _i(oh), _i(ow))
    return y


def catclassifier_fwd(x):
    x = _f(x)
    N, Cc = x.shape
    y = np.empty(N, np.int32)
    lib().so_catclassifier_fwd(_p(x), _p(y), _i(N), _i(Cc))
    return y


def catclassifier_bwd(x, pred, label, scale):
    """returns dx, loss[N]"""
    x = _f(x)
    N, Cc = x.shape
    pred = np.ascontiguousarray(pred, np.int32).reshape(-1)
    label = np.ascontiguousarray(label, np.int32).reshape(-1)
    dx = np.empty_like(x)
    loss = np.zeros(N, np.float32)
    lib().so_catclassifier_bwd(_p(x), _p(dx), _p(pred), _p(label), _p(loss), _i(N), _i(Cc), _fl(scale))
    return dx, loss


ADAM_B1 = 0.9
ADAM_B2 = 0.999


def adam_bias_terms(t):
    # src/cuda/cuda_optimizer.cpp:79-80, evaluated in double then narrowed to float
    return np.float32(1.0 / (1.0 - ADAM_B1 ** t)), np.float32(1.0 / (1.0 - ADAM_B2 ** t))


def adam_f32(w, g, m, v, t, lr, lam=0.0):
    """in-place on w, m, v (float32 1-D arrays); returns flags [range, inf, nan]"""
    assert w.dtype == np.float32 and m.dtype == np.float32 and v.dtype == np.float32
    g = _f(g)
    b1t, b2t = adam_bias_terms(t)
    flags = np.zeros(3, np.uint32)
    lib().so_adam_f32(_p(w), _p(g), _p(m), _p(v), _sz(w.size), _fl(b1t), _fl(b2t), _fl(lr), _fl(lam), _p(flags))
    return flags


def adam_mixed(w16, g16, m, v, c, t, lr, scale, lam=0.0):
    """in-place on w16 (uint16 bits), m, v, c; g16 uint16 bits; alpha = 1/scale"""
    assert w16.dtype == np.uint16 and g16.dtype == np.uint16
    b1t, b2t = adam_bias_terms(t)
    flags = np.zeros(3, np.uint32)
    lib().so_adam_mixed(_p(w16), _p(g16), _p(m), _p(v), _p(c), _sz(w16.size), _fl(np.float32(1.0) / np.float32(scale)),
                        _fl(b1t), _fl(b2t), _fl(lr), _fl(lam), _p(flags))
    return flags


def loss_scale_update(scale, flags):
    """src/cuda/cuda_program.cpp:295-302 (float arithmetic)."""
    scale = float(np.float32(scale))  # float *= double literal: product in double, stored as float
    if flags[1] or flags[2]:
        return np.float32(scale * 0.5)
    if flags[0] > 1:
        return np.float32(scale * 0.9)
    return np.float32(scale * 1.02)


def round_half(x):
    return np.asarray(x, np.float32).astype(np.float16).astype(np.float32)
