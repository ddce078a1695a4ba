"""Host-side mirror of the reference runtime's operator interface for the GEMV / LSTM hot path.

Function names, argument meaning and dispatch rules follow the reference's C++ operators
(paths relative to the reference tree):

    custom_aten_addmm   customAtenAddmm   runtime/source/executor/op_executor/aten_ops.cpp:609-758
    custom_aten_matmul  customAtenMatmul  runtime/source/executor/op_executor/aten_ops.cpp:760-932
    aten_linear         atenLinear        runtime/source/executor/op_executor/aten_ops.cpp:304-307
    aten_lstm1 / 2      atenLstm1 / 2     runtime/source/executor/op_executor/aten_ops.cpp:328-344
    gemm_broadcast      gemmBroadcast     runtime/source/executor/utils/utils.cpp:293-371
    get_gemm_type       getGemmType       runtime/source/executor/utils/utils.cpp:373-396

torch tensors carry device memory and the stream; every product that is a batch-1 GEMV, a dot product or an
LSTM runs in libpimhip.so.  True matrix-matrix products take the same LibTorch passthrough the reference takes
(atenAddmm / atenMatmul, aten_ops.cpp:47-51,362).  Errors are raised as NNRuntimeException
(runtime/include/executor/utils/utils.h:166-176) instead of being ignored.
"""
import collections
import contextlib
import ctypes
import enum
import weakref

import torch

from . import _lib as L


class NNRuntimeException(RuntimeError):
    """Counterpart of nn_compiler::runtime::utils::NNRuntimeException."""


class GemmType(enum.IntEnum):
    """GEMM_TYPE of runtime/include/executor/utils/utils.h:30-36."""
    UNKNOW = L.GEMM_UNKNOWN
    VV = L.GEMM_VV
    VM = L.GEMM_VM
    MV = L.GEMM_MV
    MM = L.GEMM_MM


def _check(rc):
    if rc != L.PIMHIP_OK:
        msg = L.load().pimhip_last_error().decode("utf-8", "replace")
        raise NNRuntimeException(f"pimhip error {rc}: {msg}")


_initialized_devices = set()


def initialize(device=None):
    """PimInitialize counterpart (runtime/source/nn_runtime.cpp:32).  Needs a gfx950 GPU."""
    lib = L.load()
    if not torch.cuda.is_available():
        raise NNRuntimeException("no HIP device is visible; this path has no CPU fallback")
    if device is None:
        device = torch.cuda.current_device()
    device = torch.device("cuda", device).index if not isinstance(device, int) else device
    with torch.cuda.device(device):
        _check(lib.pimhip_initialize(device))
    _initialized_devices.add(device)


def deinitialize():
    """PimDeinitialize counterpart (runtime/source/nn_runtime.cpp:85)."""
    _plan_cache.clear()
    _check(L.load().pimhip_deinitialize())
    _initialized_devices.clear()


def _ensure_init(t):
    dev = t.device.index if t.device.index is not None else torch.cuda.current_device()
    if dev not in _initialized_devices:
        initialize(dev)
    return dev


def _stream_handle(stream):
    """hipStream_t as an integer; None means torch's current stream (the null stream unless changed)."""
    if stream is None:
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, torch.cuda.Stream):
        return stream.cuda_stream
    return int(stream)


def gemv_status(stream=None):
    """After the caller has synchronised `stream`: has a reducing block of a sliced I_X_W product given up waiting for
    partial sums since the workspace was last put in order?  Returns (on_this_stream, static_entry_point).  Such a product
    is completed by the block itself; this is for a caller that wants to know."""
    flags = ctypes.c_int(0)
    _check(L.load().pimhip_gemv_status(_stream_handle(stream), ctypes.byref(flags)))
    return bool(flags.value & 1), bool(flags.value & 2)


def gemv_fallbacks(stream=None):
    """How many times a reducing block of a sliced I_X_W product has given up a wait so far, on `stream` plus through the
    static entry point (pimhip_gemv_fallbacks).  Ask after synchronising the stream."""
    n = ctypes.c_uint64(0)
    _check(L.load().pimhip_gemv_fallbacks(_stream_handle(stream), ctypes.byref(n)))
    return int(n.value)


def synchronize_and_check(stream=None):
    """Synchronises `stream` (torch's current one by default).  Kept for callers of the earlier interface, where a sliced
    I_X_W product that gave up a wait left an undefined result and this raised: nothing is left undefined any more."""
    s = stream if isinstance(stream, torch.cuda.Stream) else (torch.cuda.current_stream() if stream is None else None)
    if s is not None:
        s.synchronize()
    else:
        torch.cuda.synchronize()


def set_gemv_spin_limit(spin_limit):
    """Polls of one record before a reducing block of the sliced I_X_W kernel gives up (default 2**22; 0 gives up at once)."""
    _check(L.load().pimhip_set_gemv_spin_limit(int(spin_limit)))


def _require_half_cuda(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise NNRuntimeException("tensors of this path must live on the GPU (there is no CPU fallback)")
        if t.dtype != torch.float16:
            raise NNRuntimeException(f"fp16 tensors required, got {t.dtype}")


# ---------------------------------------------------------------------------------------------------
# shape logic
# ---------------------------------------------------------------------------------------------------
def gemm_broadcast(shape1, shape2):
    """Returns the two shapes padded as gemmBroadcast pads them.  Raises if they do not end at rank 4."""
    lib = L.load()
    a = (ctypes.c_int64 * 4)(*list(shape1) + [0] * (4 - len(shape1)))
    b = (ctypes.c_int64 * 4)(*list(shape2) + [0] * (4 - len(shape2)))
    ra, rb = ctypes.c_int(len(shape1)), ctypes.c_int(len(shape2))
    _check(lib.pimhip_gemm_broadcast(a, ctypes.byref(ra), b, ctypes.byref(rb)))
    return list(a[:ra.value]), list(b[:rb.value])


def get_gemm_type(self_shape, other_shape):
    lib = L.load()
    if len(self_shape) != 4 or len(other_shape) != 4:
        raise NNRuntimeException("get_gemm_type takes two rank-4 shapes")
    a = (ctypes.c_int64 * 4)(*self_shape)
    b = (ctypes.c_int64 * 4)(*other_shape)
    out = ctypes.c_int(0)
    _check(lib.pimhip_get_gemm_type(a, b, ctypes.byref(out)))
    return GemmType(out.value)


# ---------------------------------------------------------------------------------------------------
# GEMV family
# ---------------------------------------------------------------------------------------------------
def _weight_view(w2d):
    """(tensor, order_is_transposed): a 2-D weight usable without a copy, or a contiguous copy.

    A [rows, cols] view whose memory is column-major with a dense pitch (a `.t()` of a row-major matrix, which
    is what SwapAddmmInputs / SwapMatmulInputs leave behind, compiler/source/frontend/optimizer/
    swap_addmm_inputs.cpp:45-97) is the other operand order on the same bytes, so the reference's
    `.contiguous()` copy (aten_ops.cpp:630-632) is not needed.
    """
    if w2d.is_contiguous():
        return w2d, False
    if w2d.dim() == 2 and w2d.stride(0) == 1 and w2d.stride(1) >= w2d.size(0):
        return w2d.t(), True
    return w2d.contiguous(), False


def _gemv(x, weight2d, bias, in_w, out_w, order, act, stream):
    """Launches one GEMV.  weight2d is [in_w, out_w] for I_X_W and [out_w, in_w] for W_X_I."""
    lib = L.load()
    _ensure_init(weight2d)
    w, flipped = _weight_view(weight2d)
    if flipped:
        order = L.PIMHIP_W_X_I if order == L.PIMHIP_I_X_W else L.PIMHIP_I_X_W
    ld = w.stride(0) if w.size(0) > 1 else w.size(1)
    x = x.contiguous()
    if bias is not None:
        bias = bias.contiguous()
        if bias.numel() != out_w:
            raise NNRuntimeException(f"bias has {bias.numel()} elements, the GEMV produces {out_w}")
    out = torch.empty(out_w, dtype=torch.float16, device=weight2d.device)
    _check(lib.pimhip_execute_gemv(out.data_ptr(), x.data_ptr(), w.data_ptr(),
                                   bias.data_ptr() if bias is not None else None, in_w, out_w, ld, act, order,
                                   _stream_handle(stream)))
    return out


def _act_code(act_type):
    # Only "aten::relu" selects an activation (aten_ops.cpp:622-624); "none" and "aten::max" do not.
    return L.PIMHIP_ACT_RELU if act_type == "aten::relu" else L.PIMHIP_ACT_NONE


def custom_aten_addmm(act_type, self_tensor, mat1_tensor, mat2_tensor, beta=1, alpha=1, stream=None):
    """customAtenAddmm: act(mat1 . mat2 + self) with the reference's shape dispatch.

    VM and MV products ignore beta and alpha exactly as the reference does (aten_ops.cpp:627-628).
    """
    _require_half_cuda(self_tensor, mat1_tensor, mat2_tensor)
    dim_i0, dim_i1, dim_self = mat1_tensor.dim(), mat2_tensor.dim(), self_tensor.dim()
    s1, s2 = gemm_broadcast(list(mat1_tensor.shape), list(mat2_tensor.shape))
    gemm_type = get_gemm_type(s1, s2)
    act = _act_code(act_type)

    if gemm_type == GemmType.VM and dim_i0 > 1:
        out_w, in_w = mat2_tensor.size(dim_i1 - 1), mat2_tensor.size(dim_i1 - 2)
        y = _gemv(mat1_tensor.reshape(-1), mat2_tensor.reshape(in_w, out_w), self_tensor.reshape(-1), in_w, out_w,
                  L.PIMHIP_I_X_W, act, stream)
        shape = list(mat1_tensor.shape)
        shape[dim_i0 - 1], shape[dim_i0 - 2] = out_w, 1
        return y.view(shape)
    if gemm_type == GemmType.MV and dim_i1 > 1:
        out_w, in_w = mat1_tensor.size(dim_i0 - 2), mat1_tensor.size(dim_i0 - 1)
        y = _gemv(mat2_tensor.reshape(-1), mat1_tensor.reshape(out_w, in_w), self_tensor.reshape(-1), in_w, out_w,
                  L.PIMHIP_W_X_I, act, stream)
        shape = list(mat2_tensor.shape)
        shape[dim_i1 - 1], shape[dim_i1 - 2] = 1, out_w
        return y.view(shape)
    if dim_self == 1:
        # True GEMM with a 1-D bias (aten_ops.cpp:695-711): LibTorch passthrough.
        bias = self_tensor.unsqueeze(1).repeat(1, mat2_tensor.size(dim_i1 - 1))
        m2 = mat2_tensor.squeeze(0) if dim_i1 != 2 else mat2_tensor
        out = torch.addmm(bias, mat1_tensor, m2, beta=beta, alpha=alpha)
        if act == L.PIMHIP_ACT_RELU:
            out = torch.relu(out)
        for _ in range(dim_i1 - 2):
            out = out.unsqueeze(0)
        return out
    # Batched case (aten_ops.cpp:712-757).  The reference's ENABLE_PIM branch never stores its result; the
    # LibTorch branch is the defined behaviour and is the one taken here.
    out = torch.addmm(self_tensor, mat1_tensor, mat2_tensor, beta=beta, alpha=alpha)
    if act == L.PIMHIP_ACT_RELU:
        out = torch.relu(out)
    return out


def custom_aten_matmul(self_tensor, other_tensor, stream=None):
    """customAtenMatmul: self . other with the reference's shape dispatch, no bias and no activation."""
    _require_half_cuda(self_tensor, other_tensor)
    dim_i0, dim_i1 = self_tensor.dim(), other_tensor.dim()
    s1, s2 = gemm_broadcast(list(self_tensor.shape), list(other_tensor.shape))
    gemm_type = get_gemm_type(s1, s2)

    if gemm_type == GemmType.VM:
        out_w, in_w = other_tensor.size(dim_i1 - 1), other_tensor.size(dim_i1 - 2)
        y = _gemv(self_tensor.reshape(-1), other_tensor.reshape(in_w, out_w), None, in_w, out_w, L.PIMHIP_I_X_W,
                  L.PIMHIP_ACT_NONE, stream)
        if dim_i1 > dim_i0:
            shape = list(other_tensor.shape)
            shape[dim_i1 - 1], shape[dim_i1 - 2] = out_w, 1
        else:
            shape = list(self_tensor.shape)
            shape[dim_i0 - 1], shape[dim_i0 - 2] = out_w, 1
        return y.view(shape)
    if gemm_type == GemmType.MV:
        out_w, in_w = self_tensor.size(dim_i0 - 2), self_tensor.size(dim_i0 - 1)
        y = _gemv(other_tensor.reshape(-1), self_tensor.reshape(out_w, in_w), None, in_w, out_w, L.PIMHIP_W_X_I,
                  L.PIMHIP_ACT_NONE, stream)
        if dim_i0 > dim_i1:
            shape = list(self_tensor.shape)
            shape[dim_i0 - 2] = out_w
            shape.pop()
        else:
            shape = list(other_tensor.shape)
            shape[dim_i1 - 1], shape[dim_i1 - 2] = 1, out_w
        return y.view(shape)
    if gemm_type == GemmType.VV:
        lib = L.load()
        _ensure_init(self_tensor)
        a, b = self_tensor.contiguous(), other_tensor.contiguous()
        in_w = 0
        for i in range(dim_i0):
            if a.size(i) != 1:
                in_w = a.size(i)
                break
        if b.numel() < in_w or a.numel() < in_w:
            raise NNRuntimeException("VV operands are shorter than the detected vector length")
        if dim_i0 > dim_i1:
            shape = list(self_tensor.shape)
            shape[dim_i0 - 1], shape[dim_i0 - 2] = 1, 1
        else:
            shape = list(other_tensor.shape)
            shape[dim_i1 - 1], shape[dim_i1 - 2] = 1, 1
        numel = 1
        for d in shape:
            numel *= d
        if numel != 1:
            raise NNRuntimeException(f"VV output shape {shape} is not a single element")
        out = torch.empty(shape, dtype=torch.float16, device=a.device)
        _check(lib.pimhip_execute_dot(out.data_ptr(), a.data_ptr(), b.data_ptr(), in_w, _stream_handle(stream)))
        return out
    # MM (aten_ops.cpp:883-931): LibTorch passthrough.
    return torch.matmul(self_tensor, other_tensor)


def aten_linear(input_tensor, weight, bias=None, act_type="none", stream=None):
    """atenLinear for a batch-1 input: y = act(W[out,in] . x + b), the MV order on W's own row-major bytes.

    This is the product that ConvertLinearToAddmm + SwapAddmmInputs (+ FuseActivation) reduce aten::linear to
    (compiler/source/frontend/optimizer/convert_linear_to_addmm.cpp:50-51, swap_addmm_inputs.cpp:45-97),
    without the two transposes those passes insert.  Inputs with more than one row take the LibTorch passthrough.
    """
    _require_half_cuda(input_tensor, weight, bias)
    out_w, in_w = weight.shape
    if input_tensor.numel() != in_w:
        out = torch.nn.functional.linear(input_tensor, weight, bias)
        return torch.relu(out) if act_type == "aten::relu" else out
    y = _gemv(input_tensor.reshape(-1), weight, bias, in_w, out_w, L.PIMHIP_W_X_I, _act_code(act_type), stream)
    return y.view(list(input_tensor.shape[:-1]) + [out_w])


def aten_linear_cat2(input1, input2, weight, bias=None, act_type="none", stream=None):
    """y = act(W[out, in1 + in2] . cat(input1, input2) + b) for two batch-1 inputs that lie apart, without concatenating
    them (pimhip_execute_gemv_cat2): the first layer of the RNNT joint network, which the reference turns into two
    dependent addmm launches (RemoveCatForAddmm, compiler/source/frontend/optimizer/remove_cat_for_addmm.cpp:46-191).
    Operands the launch does not take (widths not multiples of 8, more than one row, an input or weight that is not 16-byte
    aligned) are concatenated and go through aten_linear."""
    _require_half_cuda(input1, input2, weight, bias)
    out_w, in_w = weight.shape
    n1, n2 = input1.numel(), input2.numel()
    w = weight if weight.stride(1) == 1 else weight.contiguous()
    x1, x2 = input1.contiguous(), input2.contiguous()
    # (a view at an offset that is not a multiple of eight halves is not 16-byte aligned: the launch refuses it)
    if (n1 + n2 != in_w or (n1 & 7) or (n2 & 7) or (w.stride(0) & 7) or input1.shape[:-1] != input2.shape[:-1] or
            (x1.data_ptr() & 15) or (x2.data_ptr() & 15) or (w.data_ptr() & 15)):
        return aten_linear(torch.cat([input1, input2], -1), weight, bias, act_type, stream)
    _ensure_init(w)
    if bias is not None:
        bias = bias.contiguous()
        if bias.numel() != out_w:
            raise NNRuntimeException(f"bias has {bias.numel()} elements, the GEMV produces {out_w}")
    out = torch.empty(out_w, dtype=torch.float16, device=w.device)
    _check(L.load().pimhip_execute_gemv_cat2(out.data_ptr(), x1.data_ptr(), n1, x2.data_ptr(), n2, w.data_ptr(),
                                             bias.data_ptr() if bias is not None else None, out_w,
                                             w.stride(0) if out_w > 1 else in_w, _act_code(act_type), _stream_handle(stream)))
    return out.view(list(input1.shape[:-1]) + [out_w])


def execute_gemv_group(inputs, weights, biases=None, act_types=None, stream=None):
    """N sibling MV GEMVs (y_i = act_i(W_i . x_i + b_i)) in one launch.

    Replaces executeMultiStream's one-stream-per-GEMV issue
    (runtime/source/executor/op_executor/stream_ops_executor.cpp:27-50).  Returns the list of outputs.
    """
    lib = L.load()
    n = len(weights)
    if len(inputs) != n:
        raise NNRuntimeException("inputs and weights differ in length")
    biases = biases if biases is not None else [None] * n
    act_types = act_types if act_types is not None else ["none"] * n
    _require_half_cuda(*inputs, *weights, *biases)
    if n == 0:
        return []
    _ensure_init(weights[0])
    xs = [x.contiguous().reshape(-1) for x in inputs]
    ws = [w.contiguous() for w in weights]
    bs = [b.contiguous() if b is not None else None for b in biases]
    outs = [torch.empty(w.size(0), dtype=torch.float16, device=w.device) for w in ws]
    for x, w in zip(xs, ws):
        if w.dim() != 2 or x.numel() != w.size(1):
            raise NNRuntimeException("each weight must be [out, in] and each input must have `in` elements")
    vp = ctypes.c_void_p * n
    rc = lib.pimhip_execute_gemv_group(
        n, vp(*[o.data_ptr() for o in outs]), vp(*[x.data_ptr() for x in xs]), vp(*[w.data_ptr() for w in ws]),
        vp(*[b.data_ptr() if b is not None else None for b in bs]),
        (ctypes.c_int64 * n)(*[w.size(1) for w in ws]), (ctypes.c_int64 * n)(*[w.size(0) for w in ws]),
        (ctypes.c_int * n)(*[_act_code(a) for a in act_types]), _stream_handle(stream))
    _check(rc)
    return outs


def aten_bmm(self_tensor, other_tensor, outs=None, stream=None):
    """executeAtenBmm's custom path (runtime/source/executor/op_executor/aten_ops_executor.cpp:668-747): for a single
    row, y[..., 1, n] = x[..., 1, k] . A[..., k, n] on the VM kernel.  `outs` may list up to four preallocated fp16
    buffers of n elements (views into concatenation buffers, as the GNMT decoder uses them, :694-737): the result is
    stored to each of them by the one launch and the first is returned.  More than one row or batch: LibTorch."""
    _require_half_cuda(self_tensor, other_tensor)
    m, k = self_tensor.size(-2), self_tensor.size(-1)
    n, k2 = other_tensor.size(-1), other_tensor.size(-2)
    if k != k2:
        raise NNRuntimeException(f"bmm operands disagree on the reduction width ({k} vs {k2})")
    if m != 1 or self_tensor.numel() != k or other_tensor.numel() != k * n:
        if outs:
            raise NNRuntimeException("preallocated outputs need the single-row product")
        return torch.bmm(self_tensor, other_tensor) if self_tensor.dim() == 3 else torch.matmul(self_tensor, other_tensor)
    lib = L.load()
    _ensure_init(other_tensor)
    x, A = self_tensor.contiguous(), other_tensor.contiguous()
    shape = list(self_tensor.shape)
    shape[-1], shape[-2] = n, m
    if not outs:
        outs = [torch.empty(shape, dtype=torch.float16, device=A.device)]
    if len(outs) > 4:
        raise NNRuntimeException("at most four destinations")
    for o in outs:
        _require_half_cuda(o)
        if o.numel() != n or not o.is_contiguous():
            raise NNRuntimeException(f"every destination must be a contiguous fp16 buffer of {n} elements")
    arr = (ctypes.c_void_p * len(outs))(*[o.data_ptr() for o in outs])
    _check(lib.pimhip_execute_bmm(arr, len(outs), x.data_ptr(), A.data_ptr(), k, n, _stream_handle(stream)))
    return outs[0]


def aten_add(self_tensor, other_tensor, alpha=1, out=None, stream=None):
    """executeAtenAdd's custom path (aten_ops_executor.cpp:43-179): fp16 tensors of equal rank (element-wise) or
    with `other` one row broadcast over the rows of `self`; the reference's kernel ignores alpha (custom_ops.h:415-433)
    and so does this path.  The reference writes the sum into `self` (or, in the GNMT decoder, into a concatenation
    buffer): pass `out` for that; by default a new tensor is returned.  Anything else goes to LibTorch."""
    if (not isinstance(other_tensor, torch.Tensor) or self_tensor.dtype != torch.float16 or
            other_tensor.dtype != torch.float16 or not self_tensor.is_cuda or not other_tensor.is_cuda or
            not _custom_add_dims_ok(self_tensor, other_tensor)):
        return torch.add(self_tensor, other_tensor, alpha=alpha, out=out)
    lib = L.load()
    _ensure_init(self_tensor)
    a, b = self_tensor.contiguous(), other_tensor.contiguous()
    n = a.size(-1)
    m = a.numel() // n if n else 0
    sym = a.dim() == b.dim()
    if (sym and b.numel() != a.numel()) or (not sym and b.numel() != n):
        return torch.add(self_tensor, other_tensor, alpha=alpha, out=out)
    if out is None:
        out = torch.empty_like(a)
    elif out.dtype != torch.float16 or not out.is_cuda or out.numel() != a.numel() or not out.is_contiguous():
        raise NNRuntimeException("`out` must be a contiguous fp16 GPU buffer with as many elements as `self`")
    _check(lib.pimhip_execute_add(out.data_ptr(), a.data_ptr(), b.data_ptr(), m, n, int(not sym), _stream_handle(stream)))
    return out


def custom_add_applies(self_tensor, other_tensor):
    """True where executeAtenAdd takes its custom kernel and this path can: fp16 GPU tensors that pass
    customAddDimensionsCheck, equal in size or `other` one row of `self`."""
    if not (isinstance(other_tensor, torch.Tensor) and self_tensor.dtype == torch.float16 and
            other_tensor.dtype == torch.float16 and self_tensor.is_cuda and other_tensor.is_cuda and
            self_tensor.dim() >= 1 and _custom_add_dims_ok(self_tensor, other_tensor)):
        return False
    if self_tensor.dim() == other_tensor.dim():
        return other_tensor.numel() == self_tensor.numel()
    return other_tensor.numel() == self_tensor.size(-1)


def _custom_add_dims_ok(t1, t2):
    """customAddDimensionsCheck (aten_ops_executor.cpp:87-109) on the larger-rank operand first."""
    s1, s2 = (t1.shape, t2.shape) if t1.dim() >= t2.dim() else (t2.shape, t1.shape)
    if len(s1) in (1, 2):
        return True
    if len(s1) == 3:
        return not (s1[0] != 1 or (len(s2) == 3 and s2[0] != 1))
    if len(s1) == 4:
        return not ((len(s2) == 4 and s1[0] != s2[0]) or s1[1] != 1 or (len(s2) == 4 and s2[1] != 1) or
                    (len(s2) == 3 and s2[0] != 1))
    return False


def input_projection(x, w, bias=None, stream=None):
    """out[T, N] fp32 = x[T, K] . w[N, K]^T + bias[N] (fp32) on the matrix cores."""
    lib = L.load()
    _require_half_cuda(x, w)
    _ensure_init(w)
    x, w = x.contiguous(), w.contiguous()
    T, K = x.shape
    N = w.size(0)
    if w.size(1) != K:
        raise NNRuntimeException("x and w disagree on the reduction width")
    if bias is not None:
        if bias.dtype != torch.float32 or not bias.is_cuda or bias.numel() != N:
            raise NNRuntimeException("bias must be an fp32 GPU tensor of N elements")
        bias = bias.contiguous()
    out = torch.empty((T, N), dtype=torch.float32, device=x.device)
    _check(lib.pimhip_input_projection(out.data_ptr(), x.data_ptr(), w.data_ptr(),
                                       bias.data_ptr() if bias is not None else None, T, K, N,
                                       _stream_handle(stream)))
    return out


def pack_projection_weight(w, stream=None):
    """w[N, K] in the matrix cores' fragment order (one-time); what an LSTM plan does with its batched layers' w_ih."""
    lib = L.load()
    _require_half_cuda(w)
    _ensure_init(w)
    w = w.contiguous()
    nbytes = ctypes.c_uint64()
    _check(lib.pimhip_projection_packed_bytes(w.size(1), w.size(0), ctypes.byref(nbytes)))
    packed = torch.empty(nbytes.value // 2, dtype=torch.float16, device=w.device)
    _check(lib.pimhip_pack_projection_weight(packed.data_ptr(), w.data_ptr(), w.size(1), w.size(0), _stream_handle(stream)))
    return packed


def input_projection_packed(x, packed, n_out, bias=None, stream=None):
    """input_projection with a weight from pack_projection_weight; the same bits, less LDS traffic."""
    lib = L.load()
    _require_half_cuda(x, packed)
    x = x.contiguous()
    T, K = x.shape
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_cuda or bias.numel() != n_out):
        raise NNRuntimeException("bias must be an fp32 GPU tensor of N elements")
    nbytes = ctypes.c_uint64()
    _check(lib.pimhip_projection_packed_bytes(K, n_out, ctypes.byref(nbytes)))
    if packed.numel() * 2 != nbytes.value:
        raise NNRuntimeException("`packed` does not have the size of a packed [n_out, in_w] weight")
    out = torch.empty((T, n_out), dtype=torch.float32, device=x.device)
    _check(lib.pimhip_input_projection_packed(out.data_ptr(), x.data_ptr(), packed.data_ptr(),
                                              bias.contiguous().data_ptr() if bias is not None else None, T, K, n_out,
                                              _stream_handle(stream)))
    return out


# ---------------------------------------------------------------------------------------------------
# LSTM
# ---------------------------------------------------------------------------------------------------
class LstmPlan:
    """Owns a PimHipLstmPlan: the one-time weight preparation of an aten::lstm layer stack.

    Counterpart of ModelBuilder::buildLstmParameterVector / reArangeLstmWeights
    (runtime/source/builder/model_builder.cpp:158-319): `params` is the LibTorch-ordered list
    (w_ih, w_hh[, b_ih, b_hh]) per layer and direction.
    """

    MODE_AUTO, MODE_STEP, MODE_SEQUENCE = 0, 1, 2

    def __init__(self, params, has_biases, num_layers, bidirectional, max_seq_len, stream=None):
        lib = L.load()
        _require_half_cuda(*params)
        _ensure_init(params[0])
        self.params = [p.contiguous() for p in params]  # keeps the weights alive for the plan's lifetime
        self.has_biases = bool(has_biases)
        self.num_layers = int(num_layers)
        self.num_dirs = 2 if bidirectional else 1
        self.hidden = self.params[1].size(1)
        self.input_size = self.params[0].size(1)
        per_cell = 4 if has_biases else 2
        if len(self.params) != self.num_layers * self.num_dirs * per_cell:
            raise NNRuntimeException(
                f"expected {self.num_layers * self.num_dirs * per_cell} parameter tensors, got {len(self.params)}")
        for ci in range(self.num_layers * self.num_dirs):
            in_w = self.input_size if ci < self.num_dirs else self.num_dirs * self.hidden
            w_ih, w_hh = self.params[ci * per_cell], self.params[ci * per_cell + 1]
            if tuple(w_ih.shape) != (4 * self.hidden, in_w) or tuple(w_hh.shape) != (4 * self.hidden, self.hidden):
                raise NNRuntimeException(f"parameter shapes of cell {ci} do not match an LSTM with H={self.hidden}")
            if has_biases:
                for b in self.params[ci * per_cell + 2:ci * per_cell + 4]:
                    if b.numel() != 4 * self.hidden:
                        raise NNRuntimeException(f"bias of cell {ci} does not have 4H elements")
        self.max_seq_len = int(max_seq_len)
        self.device = self.params[0].device
        n = len(self.params)
        arr = (ctypes.c_void_p * n)(*[p.data_ptr() for p in self.params])
        handle = ctypes.c_void_p()
        _check(lib.pimhip_lstm_plan_create(ctypes.byref(handle), arr, n, int(self.has_biases), self.num_layers,
                                           int(self.num_dirs == 2), self.input_size, self.hidden, self.max_seq_len,
                                           _stream_handle(stream)))
        self._handle = handle
        self._finalizer = weakref.finalize(self, LstmPlan._destroy, handle.value)

    @staticmethod
    def _destroy(handle_value):
        try:
            L.load().pimhip_lstm_plan_destroy(ctypes.c_void_p(handle_value))
        except Exception:  # interpreter shutdown
            pass

    def set_mode(self, mode):
        """0 automatic, 1 one launch per step, 2 / 3 the persistent kernel over all CUs (3: four units per block always),
        4 one recurrence per XCD (pimhip_lstm_plan_set_mode)."""
        _check(L.load().pimhip_lstm_plan_set_mode(self._handle, mode))

    def set_measure(self, enabled):
        """Automatic mode times every kernel family on the first eager call of a range of sequence lengths and keeps the
        fastest (the default); False: thresholds choose (pimhip_lstm_plan_set_measure)."""
        _check(L.load().pimhip_lstm_plan_set_measure(self._handle, int(bool(enabled))))

    def measured_mode(self, seq_len):
        """The mode automatic mode uses for sequences of `seq_len` steps; 0 if not measured yet."""
        m = ctypes.c_int(0)
        _check(L.load().pimhip_lstm_plan_measured_mode(self._handle, int(seq_len), ctypes.byref(m)))
        return int(m.value)

    def set_residual(self, first_residual_layer):
        """Layers from `first_residual_layer` on return and hand up h + their own input (the GNMT wiring: an aten::lstm and an
        aten::add per layer in the reference); None or >= num_layers switches it off (pimhip_lstm_plan_set_residual)."""
        _check(L.load().pimhip_lstm_plan_set_residual(self._handle, self.num_layers if first_residual_layer is None else int(first_residual_layer)))

    def set_spin_limit(self, limit):
        _check(L.load().pimhip_lstm_plan_set_spin_limit(self._handle, limit))

    def status(self):
        """Synchronises.  Raises NNRuntimeException only for the one event that leaves a forward undefined (the per-XCD
        kernel's workgroups not dealt to the XCDs in rotation); a wait that gives up is made good inside the launch and
        counted by fallbacks()."""
        torch.cuda.synchronize(self.device)
        _check(L.load().pimhip_lstm_plan_status(self._handle))

    def fallbacks(self):
        """(events, exchanging): waits of the persistent kernels that have given up in forwards of this plan so far, and
        whether sequence calls still use those kernels (False once the plan runs one launch per step for good).
        Synchronises (pimhip_lstm_plan_fallbacks)."""
        torch.cuda.synchronize(self.device)
        events, exchanging = ctypes.c_uint64(0), ctypes.c_int(0)
        _check(L.load().pimhip_lstm_plan_fallbacks(self._handle, ctypes.byref(events), ctypes.byref(exchanging)))
        return int(events.value), bool(exchanging.value)

    def forward(self, x2d, h0, c0, stream=None, out=None):
        """x2d [T, I]; h0, c0 [L*D, H] (any shape with those elements).  Returns y [T, D*H], hn, cn [L*D, H].

        `out` = (y, hn, cn) preallocated contiguous fp16 buffers lets a decoder step write its results straight into
        the buffers that consume them (the GNMT concatenation buffers, miopen_ops_executor.cpp:170-228)."""
        lib = L.load()
        _require_half_cuda(x2d, h0, c0)
        T = x2d.size(0)
        if x2d.dim() != 2 or x2d.size(1) != self.input_size:
            raise NNRuntimeException(f"input must be [T, {self.input_size}], got {list(x2d.shape)}")
        n_state = self.num_layers * self.num_dirs * self.hidden
        if h0.numel() != n_state or c0.numel() != n_state:
            raise NNRuntimeException(f"h0 / c0 must have {n_state} elements")
        x2d, h0, c0 = x2d.contiguous(), h0.contiguous(), c0.contiguous()
        if out is not None:
            y, hn, cn = out
            _require_half_cuda(y, hn, cn)
            if (y.numel() != T * self.num_dirs * self.hidden or hn.numel() != n_state or cn.numel() != n_state or
                    not (y.is_contiguous() and hn.is_contiguous() and cn.is_contiguous())):
                raise NNRuntimeException("`out` buffers must be contiguous with the sizes of y, hn and cn")
        else:
            y = torch.empty((T, self.num_dirs * self.hidden), dtype=torch.float16, device=self.device)
            hn = torch.empty((self.num_layers * self.num_dirs, self.hidden), dtype=torch.float16, device=self.device)
            cn = torch.empty_like(hn)
        # The kernels read all of h0 while they store hn (and x while they store y): an output that shares memory with
        # an input, as a decoder's state buffer does when it is both, is computed beside it and copied over afterwards.
        dests = [y, hn, cn]
        staged = [t if not any(_overlap(t, i) for i in (x2d, h0, c0)) else torch.empty_like(t) for t in dests]
        _check(lib.pimhip_lstm_forward(self._handle, x2d.data_ptr(), h0.data_ptr(), c0.data_ptr(), staged[0].data_ptr(),
                                       staged[1].data_ptr(), staged[2].data_ptr(), T, _stream_handle(stream)))
        for d, t in zip(dests, staged):
            if d is not t:
                if isinstance(stream, int):
                    stream = torch.cuda.ExternalStream(stream)
                with torch.cuda.stream(stream) if stream is not None else contextlib.nullcontext():
                    d.copy_(t)
        return y, hn, cn


class DecoderPlan:
    """One launch per decoder step of a GNMT-style LSTM stack (pimhip_decoder_step): the seq_len-1 cells of every layer,
    the attention context, the residual sums and the classifier, which the reference's interpreter runs as separate
    operators (executeAtenLSTM1 / executeAtenBmm / executeAtenAdd / executeAtenAddmm, aten_ops_executor.cpp:2135-2307,
    668-747, 43-179, 181-216).

    params: LibTorch order per layer (w_ih, w_hh[, b_ih, b_hh]); layer 0 takes x [input_size], or cat(x, ctx) when
    first_takes_context; every later layer takes cat(in, ctx); layers from first_residual_layer on add their input to
    their output; classifier = (W [vocab, H], b [vocab] or None) or None."""

    def __init__(self, params, has_biases, num_layers, first_takes_context=False, first_residual_layer=2, classifier=None,
                 stream=None):
        lib = L.load()
        _require_half_cuda(*params)
        _ensure_init(params[0])
        self.params = [p.contiguous() for p in params]
        self.has_biases = bool(has_biases)
        self.num_layers = int(num_layers)
        per_cell = 4 if has_biases else 2
        if len(self.params) != self.num_layers * per_cell:
            raise NNRuntimeException(f"expected {self.num_layers * per_cell} parameter tensors, got {len(self.params)}")
        self.hidden = self.params[1].size(1)
        self.first_takes_context = bool(first_takes_context)
        self.input_size = self.params[0].size(1) - (self.hidden if self.first_takes_context else 0)
        for l in range(self.num_layers):
            in_w = self.input_size + (self.hidden if self.first_takes_context else 0) if l == 0 else 2 * self.hidden
            w_ih, w_hh = self.params[l * per_cell], self.params[l * per_cell + 1]
            if tuple(w_ih.shape) != (4 * self.hidden, in_w) or tuple(w_hh.shape) != (4 * self.hidden, self.hidden):
                raise NNRuntimeException(f"parameter shapes of layer {l} do not match this decoder wiring")
        self.device = self.params[0].device
        self.cls_w = self.cls_b = None
        self.vocab = 0
        if classifier is not None:
            w, b = classifier
            _require_half_cuda(w, *([b] if b is not None else []))
            if w.dim() != 2 or w.size(1) != self.hidden or (b is not None and b.numel() != w.size(0)):
                raise NNRuntimeException("classifier must be W [vocab, H] with an optional bias [vocab]")
            self.cls_w, self.cls_b = w.contiguous(), (b.contiguous() if b is not None else None)
            self.vocab = self.cls_w.size(0)
        n = len(self.params)
        arr = (ctypes.c_void_p * n)(*[p.data_ptr() for p in self.params])
        handle = ctypes.c_void_p()
        _check(lib.pimhip_decoder_plan_create(
            ctypes.byref(handle), arr, n, int(self.has_biases), self.num_layers, int(self.first_takes_context),
            int(first_residual_layer), self.input_size, self.hidden, self.cls_w.data_ptr() if self.cls_w is not None else None,
            self.cls_b.data_ptr() if self.cls_b is not None else None, self.vocab, _stream_handle(stream)))
        self._handle = handle
        self._finalizer = weakref.finalize(self, DecoderPlan._destroy, handle.value)
        self._enc = None

    def set_encoder(self, enc, stream=None):
        """Once per sentence: enc [S, H], the encoder outputs the attention weights of the following steps refer to.
        Multiplies the context columns of every layer's W_ih with enc (pimhip_decoder_plan_set_encoder); the plan keeps
        enc alive.  Every call projects again (three launches): a buffer that is refilled for the next sentence has the
        same address, and kernels that write it through raw pointers leave no trace a cache could key on."""
        _require_half_cuda(enc)
        if enc.dim() != 2 or enc.size(1) != self.hidden or not enc.is_contiguous():
            raise NNRuntimeException(f"enc must be a contiguous [S, {self.hidden}] tensor")
        _check(L.load().pimhip_decoder_plan_set_encoder(self._handle, enc.data_ptr(), enc.size(0), _stream_handle(stream)))
        self._enc = enc

    @staticmethod
    def _destroy(handle_value):
        try:
            L.load().pimhip_decoder_plan_destroy(ctypes.c_void_p(handle_value))
        except Exception:  # interpreter shutdown
            pass

    def set_spin_limit(self, limit):
        _check(L.load().pimhip_decoder_plan_set_spin_limit(self._handle, limit))

    def status(self):
        """Synchronises.  No step of this plan leaves an undefined result (a wait that gives up is made good inside the same
        launch), so there is nothing to raise; fallbacks() counts such events."""
        torch.cuda.synchronize(self.device)
        _check(L.load().pimhip_decoder_plan_status(self._handle))

    def fallbacks(self):
        """(events, patient): steps of this plan in which a wait has given up so far, and whether waits still run to the
        plan's poll limit (False once, after the third event, they are kept short).  Synchronises
        (pimhip_decoder_plan_fallbacks)."""
        torch.cuda.synchronize(self.device)
        events, patient = ctypes.c_uint64(0), ctypes.c_int(0)
        _check(L.load().pimhip_decoder_plan_fallbacks(self._handle, ctypes.byref(events), ctypes.byref(patient)))
        return int(events.value), bool(patient.value)

    def bind(self, x, h_prev, c_prev, att=None, enc=None, ctx=None, hn=None, cn=None, outs=None, ctx_outs=(), logits=None):
        """Fixes the buffers of a step (lists of [H] tensors per layer; hn / cn default to h_prev / c_prev, i.e. the state is
        updated in place) and returns a callable step(stream=None) that launches it without touching Python tensors
        again: what a decoder loop or a graph capture calls per step.  The context comes from `att` [S], the attention
        weights over the encoder outputs (`enc`, handed to set_encoder here; leave it out when set_encoder has been called
        for this sentence), or from `ctx` [H], a context computed elsewhere."""
        lib = L.load()
        n, H = self.num_layers, self.hidden
        hn = list(h_prev) if hn is None else list(hn)
        cn = list(c_prev) if cn is None else list(cn)
        outs = [None] * n if outs is None else list(outs)
        vecs = [x] + list(h_prev) + list(c_prev) + hn + cn + [o for o in outs if o is not None] + list(ctx_outs)
        for t in (att, enc, ctx, logits):
            if t is not None:
                vecs.append(t)
        _require_half_cuda(*vecs)
        for t in vecs:
            if not t.is_contiguous():
                raise NNRuntimeException("decoder step buffers must be contiguous")
        if len(h_prev) != n or len(c_prev) != n or len(hn) != n or len(cn) != n or len(outs) != n:
            raise NNRuntimeException(f"state lists must have {n} entries")
        for t in list(h_prev) + list(c_prev) + hn + cn + [o for o in outs if o is not None] + list(ctx_outs) + ([ctx] if ctx is not None else []):
            if t.numel() != H:
                raise NNRuntimeException(f"state, output and context vectors must have {H} elements")
        if x.numel() != self.input_size:
            raise NNRuntimeException(f"x must have {self.input_size} elements")
        if ctx is None and att is not None:
            if enc is not None:
                self.set_encoder(enc.reshape(-1, H))
            if self._enc is None or self._enc.size(0) != att.numel():
                raise NNRuntimeException("att needs encoder outputs [len(att), H]: pass enc or call set_encoder first")
        if self.vocab and (logits is None or logits.numel() != self.vocab):
            raise NNRuntimeException(f"logits must have {self.vocab} elements")
        mk = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() if t is not None else None for t in ts])  # noqa: E731
        a_hp, a_cp, a_hn, a_cn, a_out = mk(h_prev), mk(c_prev), mk(hn), mk(cn), mk(outs)
        a_ctx = mk(list(ctx_outs)) if ctx_outs else None
        keep = (vecs, a_hp, a_cp, a_hn, a_cn, a_out, a_ctx)
        ptr = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
        args = (self._handle, ptr(x), ptr(att), ptr(ctx), a_hp, a_cp, a_hn, a_cn, a_out, a_ctx, len(ctx_outs), ptr(logits))

        def step(stream=None, _keep=keep):
            _check(lib.pimhip_decoder_step(*args, _stream_handle(stream)))
        return step


class MoePlan:
    """One launch per token for a top-1 mixture-of-experts feed-forward block (pimhip_moe_ffn_step): router, choice of the
    expert on the GPU, the chosen expert's two products.  The reference runs three customAtenAddmm / atenLinear calls
    (aten_ops.cpp:609-758, :304-307) with the argmax read back on the host in between.

    router = (W_r [E, d_model], b_r [E] or None); w1[e] [d_ff, d_model], w2[e] [d_model, d_ff]; b1 / b2: lists of E biases
    or None; act_type "none" | "aten::relu" (as customAtenAddmm's); scale_by_router_prob multiplies y by softmax(logits)[e] (the Switch Transformer's
    gating)."""

    def __init__(self, router, w1, w2, b1=None, b2=None, act_type="aten::relu", scale_by_router_prob=False, stream=None):
        lib = L.load()
        wr, br = router
        E = len(w1)
        ts = [wr] + list(w1) + list(w2) + ([br] if br is not None else []) + (list(b1) if b1 is not None else []) + \
            (list(b2) if b2 is not None else [])
        _require_half_cuda(*ts)
        _ensure_init(wr)
        if wr.dim() != 2 or wr.size(0) != E or len(w2) != E or (b1 is not None and len(b1) != E) or (b2 is not None and len(b2) != E):
            raise NNRuntimeException("router_w must be [E, d_model] with E experts in w1, w2 (and b1, b2)")
        self.d_model, self.d_ff, self.num_experts = wr.size(1), w1[0].size(0), E
        for e in range(E):
            if tuple(w1[e].shape) != (self.d_ff, self.d_model) or tuple(w2[e].shape) != (self.d_model, self.d_ff):
                raise NNRuntimeException(f"expert {e}: w1 must be [{self.d_ff}, {self.d_model}] and w2 [{self.d_model}, {self.d_ff}]")
            if (b1 is not None and b1[e].numel() != self.d_ff) or (b2 is not None and b2[e].numel() != self.d_model):
                raise NNRuntimeException(f"expert {e}: b1 must have {self.d_ff} and b2 {self.d_model} elements")
        if br is not None and br.numel() != E:
            raise NNRuntimeException(f"router bias must have {E} elements")
        self.device = wr.device
        self._keep = [t.contiguous() for t in ts]   # the plan reads the weights where they lie: keep them alive
        k = iter(self._keep)
        wr_c = next(k)
        w1_c, w2_c = [next(k) for _ in range(E)], [next(k) for _ in range(E)]
        br_c = next(k) if br is not None else None
        b1_c = [next(k) for _ in range(E)] if b1 is not None else None
        b2_c = [next(k) for _ in range(E)] if b2 is not None else None
        mk = lambda lst: (ctypes.c_void_p * E)(*[t.data_ptr() for t in lst]) if lst is not None else None  # noqa: E731
        handle = ctypes.c_void_p()
        _check(lib.pimhip_moe_plan_create(ctypes.byref(handle), wr_c.data_ptr(), br_c.data_ptr() if br_c is not None else None,
                                          mk(w1_c), mk(b1_c), mk(w2_c), mk(b2_c), E, self.d_model, self.d_ff, _act_code(act_type),
                                          int(bool(scale_by_router_prob)), _stream_handle(stream)))
        self._handle = handle
        self._finalizer = weakref.finalize(self, MoePlan._destroy, handle.value)

    @staticmethod
    def _destroy(handle_value):
        try:
            L.load().pimhip_moe_plan_destroy(ctypes.c_void_p(handle_value))
        except Exception:  # interpreter shutdown
            pass

    def set_spin_limit(self, limit):
        _check(L.load().pimhip_moe_plan_set_spin_limit(self._handle, limit))

    def status(self):
        """Synchronises.  No step of this plan leaves an undefined result (a wait that gives up is made good inside the same
        launch), so there is nothing to raise; fallbacks() counts such events."""
        torch.cuda.synchronize(self.device)
        _check(L.load().pimhip_moe_plan_status(self._handle))

    def fallbacks(self):
        """(events, exchanging): waits that have given up inside steps of this plan so far, and whether steps still exchange
        hidden values between workgroups (False once the plan has gone over to the self-sufficient mode for good).
        Synchronises (pimhip_moe_plan_fallbacks)."""
        torch.cuda.synchronize(self.device)
        events, exchanging = ctypes.c_uint64(0), ctypes.c_int(0)
        _check(L.load().pimhip_moe_plan_fallbacks(self._handle, ctypes.byref(events), ctypes.byref(exchanging)))
        return int(events.value), bool(exchanging.value)

    def bind(self, x, y, router_logits=None, expert=None):
        """Fixes the buffers of a step (x, y [d_model] fp16; router_logits [E] fp16 and expert [1] int32 optional) and returns
        a callable step(stream=None): what a serving loop or a graph capture calls per token."""
        lib = L.load()
        _require_half_cuda(x, y, *([router_logits] if router_logits is not None else []))
        for t in (x, y, router_logits, expert):
            if t is not None and not t.is_contiguous():
                raise NNRuntimeException("step buffers must be contiguous")
        if x.numel() != self.d_model or y.numel() != self.d_model:
            raise NNRuntimeException(f"x and y must have {self.d_model} elements")
        if router_logits is not None and router_logits.numel() != self.num_experts:
            raise NNRuntimeException(f"router_logits must have {self.num_experts} elements")
        if expert is not None and (expert.dtype != torch.int32 or expert.numel() != 1 or expert.device != x.device):
            raise NNRuntimeException("expert must be one int32 on the device")
        ptr = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
        args = (self._handle, ptr(x), ptr(y), ptr(router_logits), ptr(expert))

        def step(stream=None, _keep=(x, y, router_logits, expert)):
            _check(lib.pimhip_moe_ffn_step(*args, _stream_handle(stream)))
        return step

    def forward(self, x, stream=None):
        """y, router_logits, expert (device tensors; nothing is read back) for one token x [.., d_model]."""
        y = torch.empty(self.d_model, dtype=torch.float16, device=self.device)
        logits = torch.empty(self.num_experts, dtype=torch.float16, device=self.device)
        expert = torch.empty(1, dtype=torch.int32, device=self.device)
        self.bind(x.contiguous(), y, logits, expert)(stream)
        return y.view(x.shape), logits, expert


def _overlap(a, b):
    """True if the two tensors' storage ranges intersect (both are dense here)."""
    a0, b0 = a.data_ptr(), b.data_ptr()
    return a.numel() > 0 and b.numel() > 0 and a0 < b0 + b.numel() * b.element_size() and b0 < a0 + a.numel() * a.element_size()


# Plans of aten_lstm1/2 calls, found again by their weights.  An entry keeps the caller's own tensors (so their
# addresses cannot be reused by other weights while it lives) and their version counters: a plan holds values derived
# from the weights (b_ih + b_hh, w_ih in matrix-core order, contiguous copies), so an in-place update of a weight makes
# it stale, and the next call builds a new one.  Updates torch does not count (writes through data_ptr from other
# libraries) need invalidate_lstm_plans.  At most PLAN_CACHE_MAX plans are kept; the least recently used one goes first.
PLAN_CACHE_MAX = 64
_plan_cache = collections.OrderedDict()


def _plan_for(params, has_biases, num_layers, bidirectional, seq_len):
    key = (tuple(p.data_ptr() for p in params), bool(has_biases), int(num_layers), bool(bidirectional))
    versions = tuple(p._version for p in params)
    entry = _plan_cache.get(key)
    if entry is not None and entry[2] != versions:
        del _plan_cache[key]
        entry = None
    plan = entry[0] if entry is not None else None
    if plan is None or plan.max_seq_len < seq_len:
        cap = max(int(seq_len), 2 * plan.max_seq_len if plan is not None else 0, 16)
        plan = LstmPlan(params, has_biases, num_layers, bidirectional, cap)
        _plan_cache[key] = (plan, list(params), versions)
    _plan_cache.move_to_end(key)
    while len(_plan_cache) > PLAN_CACHE_MAX:
        _plan_cache.popitem(last=False)
    return plan


def invalidate_lstm_plans(params=None):
    """Drops the cached plans that were built from any of the tensors in `params` (all plans when None): call it after
    changing LSTM weights in a way torch's version counters do not see.  Returns the number of plans dropped.  A plan
    still referenced elsewhere (prepare_lstm's return value) lives on; the cache just stops handing it out."""
    if params is None:
        n = len(_plan_cache)
        _plan_cache.clear()
        return n
    ptrs = {p.data_ptr() for p in params}
    stale = [k for k in _plan_cache if ptrs.intersection(k[0])]
    for k in stale:
        del _plan_cache[k]
    return len(stale)


def prepare_lstm(params, has_biases, num_layers, bidirectional, max_seq_len=64):
    """One-time weight preparation for an LSTM layer stack, done where the reference packs its MIOpen weight buffer
    (ModelBuilder::reArangeLstmWeights, runtime/source/builder/model_builder.cpp:226-319): later aten_lstm1/2 calls
    with the same parameter tensors and at most `max_seq_len` steps allocate no plan."""
    return _plan_for(list(params), has_biases, num_layers, bidirectional, max_seq_len)


def aten_lstm1(input, hx, params, has_biases, num_layers, dropout, train, bidirectional, batch_first, stream=None,
               out=None, first_residual_layer=None):
    """atenLstm1: padded-sequence aten::lstm, batch 1 (the reference's GPU LSTM hard-codes batch 1,
    miopen_ops_executor.cpp:117).  dropout is ignored as in the reference (aten_ops.cpp:333); train must be false.
    Returns (output, hy, cy) shaped like at::lstm's results.  `first_residual_layer` (not part of aten::lstm): layers from
    that one on return and hand up h + their own input (LstmPlan.set_residual), the wiring a fused stack of GNMT's
    lstm + add layers has."""
    del dropout
    if train:
        raise NNRuntimeException("training mode is not part of this inference path")
    if input.dim() != 3:
        raise NNRuntimeException("input must be [T, 1, I] or, with batch_first, [1, T, I]")
    batch = input.size(0) if batch_first else input.size(1)
    if batch != 1:
        raise NNRuntimeException(f"batch size {batch} is not supported (batch 1 only)")
    T = input.size(1) if batch_first else input.size(0)
    h0, c0 = hx[0], hx[1]
    plan = _plan_for(list(params), has_biases, num_layers, bidirectional, T)
    plan.set_residual(first_residual_layer)  # (a cached plan serves calls with and without: set on every call)
    y, hn, cn = plan.forward(input.reshape(T, input.size(2)), h0, c0, stream, out=out)
    D, H = plan.num_dirs, plan.hidden
    seq = y.view(1, T, D * H) if batch_first else y.view(T, 1, D * H)
    return seq, hn.view(num_layers * D, 1, H), cn.view(num_layers * D, 1, H)


def aten_lstm2(data, batch_sizes, hx, params, has_biases, num_layers, dropout, train, bidirectional, stream=None):
    """atenLstm2: packed-sequence aten::lstm.  With batch 1 the packed data [T, I] is the padded sequence and
    batch_sizes must be all ones."""
    del dropout
    if train:
        raise NNRuntimeException("training mode is not part of this inference path")
    if data.dim() != 2:
        raise NNRuntimeException("packed data must be [sum(batch_sizes), I]")
    bs = batch_sizes.cpu() if isinstance(batch_sizes, torch.Tensor) else torch.as_tensor(batch_sizes)
    if bs.numel() != data.size(0) or not bool((bs == 1).all()):
        raise NNRuntimeException("only batch 1 packed sequences (batch_sizes all ones) are supported")
    T = data.size(0)
    plan = _plan_for(list(params), has_biases, num_layers, bidirectional, T)
    y, hn, cn = plan.forward(data, hx[0], hx[1], stream)
    D, H = plan.num_dirs, plan.hidden
    return y, hn.view(num_layers * D, 1, H), cn.view(num_layers * D, 1, H)


RNNT_GREEDY_MAX_VOCAB = 512  # symbols the one-launch greedy loop keeps logits for (kRnntGreedyMaxVocab in csrc/rnnt_greedy_kernels.h)


class RnntPlan:
    """One launch per (t, u) step of an RNN-transducer's greedy decoding loop (pimhip_rnnt_step): the prediction network's
    LSTM cells at seq_len 1 and the joint network relu(W1 . cat(f, g) + b1) -> W2 . + b2.  The reference runs
    executeAtenLSTM1 (aten_ops_executor.cpp:2135-2307) and three executeAtenAddmm per iteration, the joint network's first
    layer split in two by RemoveCatForAddmm (remove_cat_for_addmm.cpp:46-191).

    params: the prediction network's LSTM parameters in LibTorch order; joint = (W1 [J, F + H], b1 [J] or None,
    W2 [V, J], b2 [V] or None)."""

    def __init__(self, params, has_biases, num_layers, joint, stream=None):
        lib = L.load()
        w1, b1, w2, b2 = joint
        ts = list(params) + [w1, w2] + [t for t in (b1, b2) if t is not None]
        _require_half_cuda(*ts)
        _ensure_init(w1)
        per_layer = 4 if has_biases else 2
        if len(params) != per_layer * num_layers:
            raise NNRuntimeException(f"{len(params)} parameters for {num_layers} layers (expected {per_layer * num_layers})")
        self.hidden, self.input_size = params[1].size(1), params[0].size(1)
        self.num_layers = num_layers
        self.joint_size, self.vocab = w1.size(0), w2.size(0)
        self.enc_size = w1.size(1) - self.hidden
        for l in range(num_layers):
            in_w = self.input_size if l == 0 else self.hidden
            if tuple(params[l * per_layer].shape) != (4 * self.hidden, in_w) or tuple(params[l * per_layer + 1].shape) != (4 * self.hidden, self.hidden):
                raise NNRuntimeException(f"layer {l}: w_ih must be [{4 * self.hidden}, {in_w}] and w_hh [{4 * self.hidden}, {self.hidden}]")
        if self.enc_size < 8 or tuple(w2.shape) != (self.vocab, self.joint_size):
            raise NNRuntimeException("joint: W1 must be [J, F + H] and W2 [V, J]")
        if (b1 is not None and b1.numel() != self.joint_size) or (b2 is not None and b2.numel() != self.vocab):
            raise NNRuntimeException("joint: b1 must have J and b2 V elements")
        self.device = w1.device
        self._keep = [t.contiguous() for t in ts]   # the plan reads the weights where they lie: keep them alive
        k = iter(self._keep)
        prm = [next(k) for _ in range(len(params))]
        w1_c, w2_c = next(k), next(k)
        b1_c = next(k) if b1 is not None else None
        b2_c = next(k) if b2 is not None else None
        arr = (ctypes.c_void_p * len(prm))(*[t.data_ptr() for t in prm])
        ptr = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
        handle = ctypes.c_void_p()
        _check(lib.pimhip_rnnt_plan_create(ctypes.byref(handle), arr, len(prm), int(bool(has_biases)), num_layers, self.input_size,
                                           self.hidden, w1_c.data_ptr(), ptr(b1_c), self.joint_size, self.enc_size, w2_c.data_ptr(),
                                           ptr(b2_c), self.vocab, _stream_handle(stream)))
        self._handle = handle
        self._finalizer = weakref.finalize(self, RnntPlan._destroy, handle.value)

    @staticmethod
    def _destroy(handle_value):
        try:
            L.load().pimhip_rnnt_plan_destroy(ctypes.c_void_p(handle_value))
        except Exception:  # interpreter shutdown
            pass

    def set_spin_limit(self, limit):
        _check(L.load().pimhip_rnnt_plan_set_spin_limit(self._handle, limit))

    def fallbacks(self):
        """(events, exchanging): waits that have given up inside steps of this plan so far, and whether steps still exchange
        vectors between workgroups.  Synchronises (pimhip_rnnt_plan_fallbacks)."""
        torch.cuda.synchronize(self.device)
        events, exchanging = ctypes.c_uint64(0), ctypes.c_int(0)
        _check(L.load().pimhip_rnnt_plan_fallbacks(self._handle, ctypes.byref(events), ctypes.byref(exchanging)))
        return int(events.value), bool(exchanging.value)

    def bind(self, x, h_prev, c_prev, f, hn, cn, logits, joint_hidden=None, run_prediction=True):
        """Fixes the buffers of a step and returns a callable step(stream=None): what a decoding loop or a graph capture calls.
        x [I], h_prev / c_prev / hn / cn [L, H], f [F], logits [V], joint_hidden [J] or None; with run_prediction False (the
        step after a blank) x, c_prev, hn, cn may be None."""
        lib = L.load()
        given = [t for t in (x, h_prev, c_prev, f, hn, cn, logits, joint_hidden) if t is not None]
        _require_half_cuda(*given)
        for t in given:
            if not t.is_contiguous():
                raise NNRuntimeException("step buffers must be contiguous")
        n_state = self.num_layers * self.hidden
        sizes = ((x, self.input_size, "x"), (h_prev, n_state, "h_prev"), (c_prev, n_state, "c_prev"), (f, self.enc_size, "f"),
                 (hn, n_state, "hn"), (cn, n_state, "cn"), (logits, self.vocab, "logits"), (joint_hidden, self.joint_size, "joint_hidden"))
        for t, n, name in sizes:
            if t is not None and t.numel() != n:
                raise NNRuntimeException(f"{name} must have {n} elements")
        ptr = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
        args = (self._handle, ptr(x), ptr(h_prev), ptr(c_prev), ptr(f), ptr(hn), ptr(cn), ptr(logits), ptr(joint_hidden),
                int(bool(run_prediction)))

        def step(stream=None, _keep=tuple(given)):
            _check(lib.pimhip_rnnt_step(*args, _stream_handle(stream)))
        return step

    def greedy_decode(self, enc, embedding, x0, blank, max_symbols_per_frame=30, max_symbols=None, h0=None, c0=None,
                      run_prediction_first=True, stream=None):
        """The greedy decoding loop over the frames enc [T, F] in one launch (pimhip_rnnt_greedy_decode): returns
        (symbols int32 [max_symbols], result int32 [8], hn, cn [L, H]), all on the device and not synchronised; result[0] is
        the number of symbols.  embedding [rows >= V, I]: row k is the prediction network's input after symbol k; x0 [I] its
        input before any symbol.  A vocabulary of more than RNNT_GREEDY_MAX_VOCAB symbols runs the same loop driven from the
        host (one step launch and one read of the argmax per iteration): the same outputs, several times slower."""
        lib = L.load()
        enc, embedding = enc.contiguous(), embedding.contiguous()
        given = [t for t in (enc, embedding, x0, h0, c0) if t is not None]
        _require_half_cuda(*given)
        if enc.dim() != 2 or enc.size(1) != self.enc_size:
            raise NNRuntimeException(f"enc must be [T, {self.enc_size}]")
        if embedding.dim() != 2 or embedding.size(1) != self.input_size:
            raise NNRuntimeException(f"embedding must be [rows, {self.input_size}]")
        n_state = self.num_layers * self.hidden
        for t, n, name in ((x0, self.input_size, "x0"), (h0, n_state, "h0"), (c0, n_state, "c0")):
            if t is not None and (t.numel() != n or not t.is_contiguous()):
                raise NNRuntimeException(f"{name} must be contiguous with {n} elements")
        n_frames = enc.size(0)
        if max_symbols is None:
            max_symbols = n_frames * max_symbols_per_frame
        symbols = torch.empty(max(int(max_symbols), 1), dtype=torch.int32, device=self.device)
        result = torch.zeros(8, dtype=torch.int32, device=self.device)
        if self.vocab > RNNT_GREEDY_MAX_VOCAB:
            return self._greedy_decode_from_the_host(enc, embedding, x0, int(blank), int(max_symbols_per_frame), int(max_symbols), h0, c0,
                                                     bool(run_prediction_first), stream, symbols, result)
        hn = torch.empty(self.num_layers, self.hidden, dtype=torch.float16, device=self.device)
        cn = torch.empty_like(hn)
        ptr = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
        _check(lib.pimhip_rnnt_greedy_decode(self._handle, enc.data_ptr(), n_frames, embedding.data_ptr(), embedding.size(0), ptr(x0),
                                             ptr(h0), ptr(c0), int(bool(run_prediction_first)), int(blank), int(max_symbols_per_frame),
                                             int(max_symbols), symbols.data_ptr(), result.data_ptr(), hn.data_ptr(), cn.data_ptr(),
                                             _stream_handle(stream)))
        return symbols[:int(max_symbols)], result, hn, cn

    def _greedy_decode_from_the_host(self, enc, embedding, x0, blank, per_frame, max_symbols, h0, c0, run_prediction, stream, symbols,
                                     result):
        """The same loop for a vocabulary the loop kernel does not take (more than RNNT_GREEDY_MAX_VOCAB symbols): one
        pimhip_rnnt_step and one argmax read back per iteration, as the reference's interpreter drives it
        (examples/runtime/source/pipeline_manager.cpp:105).  Same outputs; synchronises every step."""
        if not 0 <= blank < self.vocab:
            raise NNRuntimeException(f"blank={blank} is not a symbol of the vocabulary of {self.vocab}")
        if embedding.size(0) < self.vocab:
            raise NNRuntimeException(f"embedding has {embedding.size(0)} rows for {self.vocab} symbols")
        if per_frame < 1:
            raise NNRuntimeException("max_symbols_per_frame must be at least 1")
        if x0 is None and run_prediction:
            raise NNRuntimeException("x0 (the prediction network's input before any symbol) is missing")
        shape = (self.num_layers, self.hidden)
        h = torch.zeros(shape, dtype=torch.float16, device=self.device) if h0 is None else h0.reshape(shape).clone()
        c = torch.zeros(shape, dtype=torch.float16, device=self.device) if c0 is None else c0.reshape(shape).clone()
        t, emitted, in_frame, label, steps = 0, [], 0, -1, 0
        while t < enc.size(0) and len(emitted) < max_symbols:
            if run_prediction:
                logits, h, c = self.forward(x0 if label < 0 else embedding[label], h, c, enc[t], True, stream)
            else:
                logits, _, _ = self.forward(None, h, None, enc[t], False, stream)
            # torch.argmax's choice: the first maximum, a NaN counting as the largest
            nan = torch.isnan(logits)
            k = int(nan.float().argmax()) if bool(nan.any()) else int(torch.argmax(logits.float()))
            steps += 1
            if k == blank:
                t, in_frame, run_prediction = t + 1, 0, False
            else:
                emitted.append(k)
                label, in_frame, run_prediction = k, in_frame + 1, True
                if in_frame >= per_frame:
                    t, in_frame = t + 1, 0
        if emitted:
            symbols[:len(emitted)] = torch.tensor(emitted, dtype=torch.int32, device=self.device)
        result.copy_(torch.tensor([len(emitted), t, steps, 0, int(run_prediction), label, 0, 0], dtype=torch.int32))
        return symbols[:max_symbols], result, h, c

    def forward(self, x, h_prev, c_prev, f, run_prediction=True, stream=None):
        """logits [V], hn, cn [L, H] for one step (new tensors; with run_prediction False hn, cn are h_prev, c_prev)."""
        logits = torch.empty(self.vocab, dtype=torch.float16, device=self.device)
        if run_prediction:
            hn, cn = torch.empty_like(h_prev.contiguous()), torch.empty_like(c_prev.contiguous())
            self.bind(x.contiguous(), h_prev.contiguous(), c_prev.contiguous(), f.contiguous(), hn, cn, logits)(stream)
            return logits, hn, cn
        self.bind(None, h_prev.contiguous(), None, f.contiguous(), None, None, logits, run_prediction=False)(stream)
        return logits, h_prev, c_prev
