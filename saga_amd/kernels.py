"""ctypes binding of the C-ABI kernel library (include/saga_hip.h).

Loads saga_amd/lib/libsaga_hip.so and fails loudly when it is missing: there is no CPU or
PyTorch fallback for any entry point.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libsaga_hip.so")

U8, HALF, FLOAT, INT64, I32, I16 = range(6)
CONV_FWD, CONV_BWD_DATA, CONV_BWD_FILTER = range(3)
ACT_RELU, ACT_SIGMOID, ACT_TANH, ACT_SWISH, ACT_LEAKYRELU = range(5)
POOL_MAX, POOL_AVG = range(2)
BN_RELU, BN_ADD = 1, 2


class TensorView(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("dims", C.c_int32 * 4), ("strides", C.c_int64 * 4), ("dtype", C.c_int32)]


class ConvParams(C.Structure):
    _fields_ = [("pad", C.c_int32), ("stride", C.c_int32), ("dilation", C.c_int32), ("group", C.c_int32)]


class FilterTransposeJob(C.Structure):
    _fields_ = [("w", C.c_void_p), ("wt", C.c_void_p), ("K", C.c_int32), ("C", C.c_int32), ("RS", C.c_int32),
                ("first_block", C.c_int32)]


class BnBwdLink(C.Structure):
    _fields_ = [("x", C.POINTER(TensorView)), ("s", C.c_void_p), ("b", C.c_void_p), ("save_mean", C.c_void_p),
                ("save_invstd", C.c_void_p), ("flags", C.c_int32), ("partial_rows", C.c_int32), ("partial", C.c_void_p),
                ("partial_bytes", C.c_size_t)]


class SagaHipError(RuntimeError):
    pass


_lib = None

# name -> (restype, argtypes); every symbol include/saga_hip.h declares
_VP, _I, _F, _SZ = C.c_void_p, C.c_int, C.c_float, C.c_size_t
_TV = C.POINTER(TensorView)
SIGNATURES = {
    "saga_hip_error_string": (C.c_char_p, [_I]),
    "saga_hip_init": (_I, [_I, C.POINTER(C.c_int)]),
    "saga_hip_conv2d_workspace_size": (_SZ, [_I, _TV, _TV, _TV, C.POINTER(ConvParams)]),
    "saga_hip_conv2d_fwd": (_I, [_TV, _TV, _TV, C.POINTER(ConvParams), _F, _F, _VP, _SZ, _VP]),
    "saga_hip_conv2d_fwd_bnstats_size": (_SZ, [_TV, _TV, _TV, C.POINTER(ConvParams)]),
    "saga_hip_conv2d_fwd_bnstats": (_I, [_TV, _TV, _TV, C.POINTER(ConvParams), _F, _VP, _SZ, _VP, _SZ,
                                         C.POINTER(C.c_int), _VP]),
    "saga_hip_conv2d_fwd_bn_infer": (_I, [_TV, _TV, _TV, _TV, C.POINTER(ConvParams), _VP, _VP, _VP, _VP, _F, _I, _VP, _SZ,
                                          _VP]),
    "saga_hip_conv2d_bwd_data": (_I, [_TV, _TV, _TV, C.POINTER(ConvParams), _F, _F, _VP, _SZ, _VP]),
    "saga_hip_conv2d_bwd_filter": (_I, [_TV, _TV, _TV, C.POINTER(ConvParams), _F, _F, _VP, _SZ, _VP]),
    "saga_hip_conv2d_bwd_data_wt_bytes": (_SZ, [_TV, _TV, _TV, C.POINTER(ConvParams)]),
    "saga_hip_filter_transpose_blocks": (_I, [_TV]),
    "saga_hip_filter_transpose_batched": (_I, [_VP, _I, _I, _VP]),
    "saga_hip_conv2d_bwd_data_wt": (_I, [_TV, _TV, _VP, _TV, C.POINTER(ConvParams), _F, _F, _VP, _SZ, _VP]),
    "saga_hip_conv2d_bwd_data_bnbwd_size": (_SZ, [_TV, _TV, _TV, C.POINTER(ConvParams)]),
    "saga_hip_conv2d_bwd_data_bnbwd": (_I, [_TV, _TV, _VP, _TV, C.POINTER(ConvParams), _F, _F, _VP, _SZ,
                                            C.POINTER(BnBwdLink), _VP]),
    "saga_hip_bias_add": (_I, [_TV, _TV, _VP]),
    "saga_hip_bias_bwd_workspace_size": (_SZ, [_TV]),
    "saga_hip_bias_bwd": (_I, [_TV, _TV, _F, _VP, _SZ, _VP]),
    "saga_hip_bias_bwd_noalloc": (_I, [_TV, _TV, _F, _VP]),
    "saga_hip_gemm": (_I, [_I, _I, _I, _I, _I, _F, _VP, _I, _VP, _I, _F, _VP, _I, _I, _VP]),
    "saga_hip_bn_infer": (_I, [_TV, _TV, _TV, _VP, _VP, _VP, _VP, _F, _I, _VP]),
    "saga_hip_bn_workspace_size": (_SZ, [_TV]),
    "saga_hip_bn_train_fwd": (_I, [_TV, _TV, _TV, _VP, _VP, _VP, _VP, _VP, _VP, _F, _F, _I, _VP, _SZ, _VP]),
    "saga_hip_bn_train_fwd_partials": (_I, [_TV, _TV, _TV, _VP, _VP, _VP, _VP, _VP, _VP, _F, _F, _I, _VP, _I, _VP, _VP,
                                            _SZ, _VP]),
    "saga_hip_bn_bwd": (_I, [_TV, _TV, _TV, _TV, _TV, _VP, _VP, _VP, _VP, _VP, _F, _F, _F, _I, _VP, _SZ, _VP]),
    "saga_hip_bn_bwd_ex": (_I, [_TV, _TV, _TV, _TV, _TV, _VP, _VP, _VP, _VP, _VP, _VP, _F, _F, _F, _I, _VP, _VP, _SZ,
                                _VP]),
    "saga_hip_bn_bwd_linked": (_I, [_TV, _TV, _TV, _VP, _VP, _VP, _VP, _VP, _F, _F, _VP, _I, _VP, _SZ, _VP]),
    "saga_hip_act_fwd": (_I, [_I, _F, _TV, _TV, _F, _VP]),
    "saga_hip_act_bwd": (_I, [_I, _F, _TV, _TV, _TV, _TV, _F, _VP]),
    "saga_hip_pool_fwd": (_I, [_I, _TV, _TV, _TV, _I, _I, _I, _VP]),
    "saga_hip_pool_bwd": (_I, [_I, _TV, _TV, _TV, _TV, _I, _I, _I, _F, _VP]),
    "saga_hip_add": (_I, [_TV, _TV, _TV, _VP]),
    "saga_hip_axpby": (_I, [_TV, _TV, _F, _F, _VP]),
    "saga_hip_convert": (_I, [_TV, _TV, _F, _VP]),
    "saga_hip_maxpool_fwd_codes": (_I, [_TV, _TV, _VP, _I, _I, _I, _VP]),
    "saga_hip_maxpool_bwd_codes": (_I, [_VP, _TV, _TV, _I, _I, _I, _F, _VP]),
    "saga_hip_maxpool_fwd_codes_bn": (_I, [_TV, _TV, _VP, _I, _I, _I, _VP, _I, _VP]),
    "saga_hip_bn_bwd_pooled_workspace_size": (_SZ, [_TV, _TV, _I, _I, _I]),
    "saga_hip_bn_bwd_pooled": (_I, [_TV, _TV, _VP, _TV, _VP, _VP, _VP, _VP, _VP, _VP, _F, _F, _I, _I, _I, _I, _VP, _SZ, _VP]),
    "saga_hip_softmax": (_I, [_TV, _TV, _VP]),
    "saga_hip_spatial_transform": (_I, [_TV, _VP, _TV, _VP]),
    "saga_hip_dropout_fwd": (_I, [_TV, _TV, _F, C.c_uint64, C.c_uint64, _VP]),
    "saga_hip_dropout_bwd": (_I, [_TV, _TV, _F, C.c_uint64, C.c_uint64, _F, _VP]),
    "saga_hip_catclassifier_fwd": (_I, [_TV, _VP, _VP]),
    "saga_hip_catclassifier_bwd": (_I, [_TV, _TV, _VP, _VP, _VP, _F, _VP]),
    "saga_hip_loss_bwd": (_I, [_TV, _TV, _TV, _VP, _F, _VP]),
    "saga_hip_tensor_stats_workspace_size": (_SZ, []),
    "saga_hip_tensor_stats": (_I, [_TV, _VP, _VP, _SZ, _VP]),
    "saga_hip_adam_f32": (_I, [_SZ, _VP, _VP, _VP, _VP, _F, _F, _F, _F, _VP, _VP]),
    "saga_hip_adam_mixed": (_I, [_SZ, _F, _VP, _VP, _VP, _VP, _VP, _F, _F, _F, _F, _VP, _VP]),
    "saga_hip_fill": (_I, [_VP, _I, _SZ, _VP]),
}


def lib():
    """The loaded library; raises if it was not built (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SagaHipError(
                f"{LIB_PATH} is missing: build it with `make -C saga_amd/csrc` (or __graft_entry__.build())")
        _lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(_lib, name)
            fn.restype = res
            fn.argtypes = args
    return _lib


def check(code):
    if code != 0:
        raise SagaHipError(f"saga_hip error {code}: {lib().saga_hip_error_string(code).decode()}")


_TORCH_DT = None


def _dtype_code(t):
    global _TORCH_DT
    import torch

    if _TORCH_DT is None:
        _TORCH_DT = {torch.uint8: U8, torch.float16: HALF, torch.float32: FLOAT, torch.int64: INT64,
                     torch.int32: I32, torch.int16: I16}
    return _TORCH_DT[t.dtype]


def view(t):
    """SagaTensorView of a torch tensor of rank <= 4 (logical N,C,H,W; strides as they are)."""
    if t is None:
        return None
    dims = list(t.shape) + [1] * (4 - t.dim())
    strides = list(t.stride())
    while len(strides) < 4:
        strides.append(1)
    v = TensorView()
    v.ptr = t.data_ptr()
    v.dims = (C.c_int32 * 4)(*dims)
    v.strides = (C.c_int64 * 4)(*strides)
    v.dtype = _dtype_code(t)
    return v


def _ref(v):
    return C.byref(v) if v is not None else None


def stream_ptr():
    import torch

    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _ws(nbytes, like):
    import torch

    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=like.device)


# ---------------------------------------------------------------- thin call helpers (tests / bench)

def conv2d(kind, a, w, out, pad=0, stride=1, dilation=1, group=1, alpha=1.0, beta=0.0):
    """kind FWD: a=x,out=y ; BWD_DATA: a=dy,out=dx ; BWD_FILTER: a=x, w=dy, out=dw."""
    L = lib()
    p = ConvParams(pad, stride, dilation, group)
    va, vw, vo = view(a), view(w), view(out)
    if kind == CONV_FWD:
        n = L.saga_hip_conv2d_workspace_size(kind, _ref(va), _ref(vw), _ref(vo), C.byref(p))
        ws = _ws(n, a)
        check(L.saga_hip_conv2d_fwd(_ref(va), _ref(vw), _ref(vo), C.byref(p), alpha, beta, ptr(ws), ws.numel(),
                                    stream_ptr()))
    elif kind == CONV_BWD_DATA:
        n = L.saga_hip_conv2d_workspace_size(kind, _ref(vo), _ref(vw), _ref(va), C.byref(p))
        ws = _ws(n, a)
        check(L.saga_hip_conv2d_bwd_data(_ref(va), _ref(vw), _ref(vo), C.byref(p), alpha, beta, ptr(ws), ws.numel(),
                                         stream_ptr()))
    else:
        n = L.saga_hip_conv2d_workspace_size(kind, _ref(va), _ref(vo), _ref(vw), C.byref(p))
        ws = _ws(n, a)
        check(L.saga_hip_conv2d_bwd_filter(_ref(va), _ref(vw), _ref(vo), C.byref(p), alpha, beta, ptr(ws),
                                           ws.numel(), stream_ptr()))
    return out


def bn_workspace(x):
    vx = view(x)
    return _ws(lib().saga_hip_bn_workspace_size(_ref(vx)), x)
