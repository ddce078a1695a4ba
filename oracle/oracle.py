"""TEST INFRASTRUCTURE, NOT PRODUCT CODE: Python access to the CPU oracle and to the reference's own kernels.

Three checkers live here; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this file.

1. `liboracle.so` (oracle/oracle.c): the plain-C restatement of the path, wrapped on numpy arrays.
2. LibTorch CPU (`torch_*` functions): at::addmm / at::matmul / at::lstm in fp16 on the CPU, the ops the reference
   passes through to (runtime/source/executor/op_executor/aten_ops.cpp:47-51, 328-344, 362) and the arbiter
   named for this path's tolerances.  torch is a library of this image, not part of the reference.
3. `oracle/_ref/libref_custom_ops.so`: the reference's own HIP GEMV / add / bmm launchers
   (runtime/include/executor/op_executor/custom_ops.h), compiled from the reference tree by oracle/Makefile.
   GPU only; optional (absent when the reference tree was not available at build time).
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_LIB = os.path.join(_HERE, "liboracle.so")
REF_LIB = os.path.join(_HERE, "_ref", "libref_custom_ops.so")

_u16p = ctypes.POINTER(ctypes.c_uint16)
_i64p = ctypes.POINTER(ctypes.c_int64)
_lib = None
_ref = None


def build(verbose=False):
    """Compiles liboracle.so (and oracle/_ref when the reference tree is present) with oracle/Makefile."""
    res = subprocess.run(["make", "-C", _HERE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building the oracle failed:\n" + res.stdout)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_LIB):
            build()
        l = ctypes.CDLL(ORACLE_LIB)
        l.oracle_half_to_double.restype = ctypes.c_double
        l.oracle_half_to_double.argtypes = [ctypes.c_uint16]
        l.oracle_double_to_half.restype = ctypes.c_uint16
        l.oracle_double_to_half.argtypes = [ctypes.c_double]
        l.oracle_gemm_broadcast.restype = ctypes.c_int
        l.oracle_gemm_broadcast.argtypes = [_i64p, ctypes.POINTER(ctypes.c_int), _i64p, ctypes.POINTER(ctypes.c_int)]
        l.oracle_get_gemm_type.restype = ctypes.c_int
        l.oracle_get_gemm_type.argtypes = [_i64p, _i64p]
        l.oracle_gemv_mv.restype = None
        l.oracle_gemv_mv.argtypes = [_u16p, _u16p, _u16p, _u16p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
        l.oracle_gemv_vm.restype = None
        l.oracle_gemv_vm.argtypes = [_u16p, _u16p, _u16p, _u16p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
        l.oracle_dot.restype = None
        l.oracle_dot.argtypes = [_u16p, _u16p, _u16p, ctypes.c_int64]
        l.oracle_add.restype = None
        l.oracle_add.argtypes = [_u16p, _u16p, _u16p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
        l.oracle_gemv_mv_f32.restype = None
        l.oracle_gemv_mv_f32.argtypes = [ctypes.POINTER(ctypes.c_float)] * 4 + [ctypes.c_int64, ctypes.c_int64]
        l.oracle_lstm.restype = None
        l.oracle_lstm.argtypes = [_u16p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                  ctypes.c_int, ctypes.POINTER(_u16p), _u16p, _u16p, _u16p, _u16p, _u16p]
        l.oracle_lstm_pack_miopen.restype = None
        l.oracle_lstm_pack_miopen.argtypes = [ctypes.POINTER(_u16p), _i64p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                              _u16p, ctypes.c_int]
        _lib = l
    return _lib


def _h(a):
    """Contiguous fp16 array viewed as uint16 + its ctypes pointer."""
    a = np.ascontiguousarray(a, dtype=np.float16)
    u = a.view(np.uint16)
    return u, u.ctypes.data_as(_u16p)


# ---- shape logic -----------------------------------------------------------------------------------------
def gemm_broadcast(shape1, shape2):
    """Returns (status, shape1, shape2): status 0 ok, 1 the reference aborts, 2 the reference reads out of range."""
    a = (ctypes.c_int64 * 8)(*shape1)
    b = (ctypes.c_int64 * 8)(*shape2)
    ra, rb = ctypes.c_int(len(shape1)), ctypes.c_int(len(shape2))
    rc = lib().oracle_gemm_broadcast(a, ctypes.byref(ra), b, ctypes.byref(rb))
    return rc, list(a[:ra.value]), list(b[:rb.value])


def get_gemm_type(self_shape, other_shape):
    """GEMM_TYPE as the reference numbers it: 1 VV, 2 MV, 3 VM, 4 MM."""
    return lib().oracle_get_gemm_type((ctypes.c_int64 * 4)(*self_shape), (ctypes.c_int64 * 4)(*other_shape))


# ---- GEMV family -----------------------------------------------------------------------------------------
def gemv_mv(W, x, bias=None, relu=False):
    """y[N] = act(W[N,K] . x[K] + bias[N]) on fp16 arrays."""
    Wu, Wp = _h(W)
    xu, xp = _h(x)
    N, K = Wu.shape
    y = np.empty(N, dtype=np.uint16)
    bp = None
    if bias is not None:
        bu, bp = _h(bias)
    lib().oracle_gemv_mv(Wp, xp, bp, y.ctypes.data_as(_u16p), N, K, K, int(relu))
    return y.view(np.float16)


def gemv_vm(x, A, bias=None, relu=False):
    """y[N] = act(x[K] . A[K,N] + bias[N]) on fp16 arrays."""
    Au, Ap = _h(A)
    xu, xp = _h(x)
    K, N = Au.shape
    y = np.empty(N, dtype=np.uint16)
    bp = None
    if bias is not None:
        bu, bp = _h(bias)
    lib().oracle_gemv_vm(xp, Ap, bp, y.ctypes.data_as(_u16p), K, N, N, int(relu))
    return y.view(np.float16)


def dot(a, b):
    au, ap = _h(a)
    bu, bp = _h(b)
    y = np.empty(1, dtype=np.uint16)
    lib().oracle_dot(ap, bp, y.ctypes.data_as(_u16p), au.size)
    return y.view(np.float16)


def add(a, b):
    """c = a[m, n] + b with b [m, n] or [n] (fp16, one rounding)."""
    au, ap = _h(a)
    bu, bp = _h(b)
    n = au.shape[-1]
    m = au.size // n
    c = np.empty(au.size, dtype=np.uint16)
    lib().oracle_add(ap, bp, c.ctypes.data_as(_u16p), m, n, int(bu.size != au.size))
    return c.view(np.float16).reshape(au.shape)


def gemv_mv_f32(W, x, bias=None):
    W = np.ascontiguousarray(W, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    N, K = W.shape
    y = np.empty(N, dtype=np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    b = np.ascontiguousarray(bias, dtype=np.float32) if bias is not None else None
    lib().oracle_gemv_mv_f32(W.ctypes.data_as(fp), x.ctypes.data_as(fp), b.ctypes.data_as(fp) if b is not None else None,
                             y.ctypes.data_as(fp), N, K)
    return y


# ---- LSTM ------------------------------------------------------------------------------------------------
def lstm(x, h0, c0, params, has_biases, num_layers, bidirectional):
    """x [T, I]; h0, c0 [L*D, H]; params in LibTorch order.  Returns y [T, D*H], hn, cn [L*D, H] (fp16)."""
    xu, xp = _h(x)
    T, I = xu.shape
    H = np.asarray(params[1]).shape[1]
    D = 2 if bidirectional else 1
    keep = [_h(p) for p in params]
    arr = (_u16p * len(keep))(*[k[1] for k in keep])
    h0u, h0p = _h(np.asarray(h0).reshape(num_layers * D, H))
    c0u, c0p = _h(np.asarray(c0).reshape(num_layers * D, H))
    y = np.empty((T, D * H), dtype=np.uint16)
    hn = np.empty((num_layers * D, H), dtype=np.uint16)
    cn = np.empty((num_layers * D, H), dtype=np.uint16)
    lib().oracle_lstm(xp, T, I, H, num_layers, int(bool(bidirectional)), int(bool(has_biases)), arr, h0p, c0p,
                      y.ctypes.data_as(_u16p), hn.ctypes.data_as(_u16p), cn.ctypes.data_as(_u16p))
    return y.view(np.float16), hn.view(np.float16), cn.view(np.float16)


def lstm_pack_miopen(params, has_biases, num_layers, bidirectional):
    """The packed fp16 weight buffer reArangeLstmWeights builds (model_builder.cpp:226-319)."""
    keep = [np.ascontiguousarray(p, dtype=np.float16).view(np.uint16).copy() for p in params]
    sizes = (ctypes.c_int64 * len(keep))(*[k.size for k in keep])
    arr = (_u16p * len(keep))(*[k.ctypes.data_as(_u16p) for k in keep])
    buf = np.zeros(sum(k.size for k in keep), dtype=np.uint16)
    lib().oracle_lstm_pack_miopen(arr, sizes, num_layers, int(bool(bidirectional)), int(bool(has_biases)),
                                  buf.ctypes.data_as(_u16p), 0)
    return buf.view(np.float16)


def lstm_unpack_miopen(buffer, shapes, has_biases, num_layers, bidirectional):
    """Inverse of lstm_pack_miopen: returns the parameter list with the given shapes."""
    buf = np.ascontiguousarray(buffer, dtype=np.float16).view(np.uint16)
    keep = [np.zeros(int(np.prod(s)), dtype=np.uint16) for s in shapes]
    sizes = (ctypes.c_int64 * len(keep))(*[k.size for k in keep])
    arr = (_u16p * len(keep))(*[k.ctypes.data_as(_u16p) for k in keep])
    lib().oracle_lstm_pack_miopen(arr, sizes, num_layers, int(bool(bidirectional)), int(bool(has_biases)),
                                  buf.ctypes.data_as(_u16p), 1)
    return [k.view(np.float16).reshape(s) for k, s in zip(keep, shapes)]


# ---- LibTorch CPU ----------------------------------------------------------------------------------------
def torch_addmm(bias, x, W):
    """at::addmm(b, x[1,in], W[out,in].t()) on the CPU in fp16: the linear route's product."""
    import torch
    return torch.addmm(bias.cpu(), x.cpu(), W.cpu().t())


def torch_lstm(x, h0, c0, params, has_biases, num_layers, bidirectional, batch_first=False):
    """at::lstm on the CPU in the dtype of its arguments, dropout 0, eval mode."""
    import torch
    return torch.lstm(x.cpu(), (h0.cpu(), c0.cpu()), [p.cpu() for p in params], bool(has_biases), int(num_layers), 0.0,
                      False, bool(bidirectional), bool(batch_first))


# ---- the reference's own HIP kernels ------------------------------------------------------------------------
def ref_lib():
    """oracle/_ref/libref_custom_ops.so or None when it was not built."""
    global _ref
    if _ref is None and os.path.exists(REF_LIB):
        r = ctypes.CDLL(REF_LIB)
        vp, i = ctypes.c_void_p, ctypes.c_int
        r.ref_gemv_xAy.argtypes = [vp, vp, vp, vp, i, i]
        r.ref_gemv_Axy.argtypes = [vp, vp, vp, vp, i, i]
        r.ref_addmv_xAy.argtypes = [vp, vp, vp, vp, vp, i, i, i]
        r.ref_addmv_Axy.argtypes = [vp, vp, vp, vp, vp, i, i, i]
        r.ref_custom_add.argtypes = [vp, vp, vp, vp, i, i, i]
        r.ref_bmm_xAy.argtypes = [vp, vp, vp, vp, i, i]
        for f in (r.ref_gemv_xAy, r.ref_gemv_Axy, r.ref_addmv_xAy, r.ref_addmv_Axy, r.ref_custom_add, r.ref_bmm_xAy):
            f.restype = None
        _ref = r
    return _ref
