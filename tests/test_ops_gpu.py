"""The operator layer's dispatch (customAtenAddmm / customAtenMatmul shape rules, weight views, fallbacks), on the
GPU through the C ABI.  Output shapes follow runtime/source/executor/op_executor/aten_ops.cpp:626-694, 770-882."""
import numpy as np
import pytest
import torch

from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3


def maxabs(a, b):
    return float((a.detach().float().cpu().reshape(-1) - b.detach().float().cpu().reshape(-1)).abs().max())


def rnd(g, *shape, scale=0.1):
    return (scale * torch.randn(*shape, generator=g)).half()


def test_addmm_vm_and_mv_output_shapes_and_values(ops):
    g = torch.Generator().manual_seed(1)
    b, x, A = rnd(g, 96), rnd(g, 1, 64, scale=1.0), rnd(g, 64, 96)
    want = torch.addmm(b.float(), x.float(), A.float())
    y = ops.custom_aten_addmm("none", b.to(DEV), x.to(DEV), A.to(DEV))
    assert list(y.shape) == [1, 96] and maxabs(y, want) <= TOL
    # 4-D input as in the reference's unit test: [1,1,1,K] x [K,N]
    y = ops.custom_aten_addmm("aten::relu", b.to(DEV), x.reshape(1, 1, 1, 64).to(DEV), A.to(DEV))
    assert list(y.shape) == [1, 1, 1, 96] and maxabs(y, torch.relu(want)) <= TOL
    # MV: W[out,in] x x[in,1]
    W = A.t().contiguous()
    y = ops.custom_aten_addmm("none", b.to(DEV), W.to(DEV), x.t().to(DEV))
    assert list(y.shape) == [96, 1] and maxabs(y, want) <= TOL
    y = ops.custom_aten_addmm("aten::max", b.to(DEV), W.to(DEV), x.reshape(1, 1, 64, 1).to(DEV))   # not an activation
    assert list(y.shape) == [1, 1, 96, 1] and maxabs(y, want) <= TOL


def test_addmm_ignores_alpha_beta_on_gemv_shapes_like_the_reference(ops):
    """aten_ops.cpp:627-628: local alpha = 1, beta = 0 shadow the IR's scalars on the VM / MV branches."""
    g = torch.Generator().manual_seed(2)
    b, x, A = rnd(g, 40), rnd(g, 1, 24, scale=1.0), rnd(g, 24, 40)
    y1 = ops.custom_aten_addmm("none", b.to(DEV), x.to(DEV), A.to(DEV), beta=1, alpha=1)
    y2 = ops.custom_aten_addmm("none", b.to(DEV), x.to(DEV), A.to(DEV), beta=3, alpha=7)
    assert torch.equal(y1, y2)


def test_transposed_weight_views_need_no_copy_and_give_the_same_result(ops):
    """SwapAddmmInputs hands over transpose views; a `.t()` of a row-major matrix is the other operand order on
    the same bytes."""
    g = torch.Generator().manual_seed(3)
    W, x, b = rnd(g, 520, 264), rnd(g, 1, 264, scale=1.0), rnd(g, 520)
    Wd = W.to(DEV)
    want = oracle.gemv_mv(W.numpy(), x.numpy().reshape(-1), b.numpy())
    y_view = ops.custom_aten_addmm("none", b.to(DEV), x.to(DEV), Wd.t())            # VM on a column-major view
    y_copy = ops.custom_aten_addmm("none", b.to(DEV), x.to(DEV), Wd.t().contiguous())
    assert maxabs(y_view, torch.as_tensor(want)) <= TOL and maxabs(y_copy, torch.as_tensor(want)) <= TOL
    y_mv = ops.custom_aten_addmm("none", b.to(DEV), Wd.t().contiguous().t(), x.to(DEV).t())   # MV on a view
    assert list(y_mv.shape) == [520, 1] and maxabs(y_mv, torch.as_tensor(want)) <= TOL


def test_matmul_shape_rules(ops):
    g = torch.Generator().manual_seed(4)
    x, A = rnd(g, 1, 32, scale=1.0), rnd(g, 32, 48)
    want = x.float() @ A.float()
    for xs, As, out_shape in [((1, 32), (32, 48), [1, 48]), ((1, 1, 1, 32), (32, 48), [1, 1, 1, 48]),
                              ((1, 32), (1, 1, 32, 48), [1, 1, 1, 48]), ((32,), (32, 48), None)]:
        if out_shape is None:
            # rank-1 x rank-2: gemmBroadcast pads to [1,1,1,32] only when shape1[0] != shape2[0]; 32 == 32 here, so
            # the reference pads to [32,1] -> an MM; the passthrough result is still the product
            y = ops.custom_aten_matmul(x.reshape(xs).to(DEV), A.reshape(As).to(DEV))
            assert maxabs(y, want) <= TOL
            continue
        y = ops.custom_aten_matmul(x.reshape(xs).to(DEV), A.reshape(As).to(DEV))
        assert list(y.shape) == out_shape and maxabs(y, want) <= TOL
    W = A.t().contiguous()
    for Ws, xs, out_shape in [((48, 32), (32, 1), [48, 1]), ((48, 32), (1, 1, 32, 1), [1, 1, 48, 1]),
                              ((1, 1, 48, 32), (32, 1), [1, 1, 48])]:
        y = ops.custom_aten_matmul(W.reshape(Ws).to(DEV), x.reshape(xs).to(DEV))
        assert list(y.shape) == out_shape and maxabs(y, want) <= TOL
    # VV: [1,K] x [K,1]
    v = rnd(g, 32, 1, scale=1.0)
    y = ops.custom_aten_matmul(x.to(DEV), v.to(DEV))
    assert list(y.shape) == [1, 1] and maxabs(y, x.float() @ v.float()) <= 1e-2


def test_true_matrix_products_take_the_libtorch_passthrough(ops):
    """aten_ops.cpp:695-711: with a 1-D bias the fallback is written for the swapped operand order the optimiser
    leaves (W[out,in] x X^T[in,M], bias repeated along the M columns)."""
    g = torch.Generator().manual_seed(5)
    b, X, W = rnd(g, 48), rnd(g, 13, 32, scale=1.0), rnd(g, 48, 32)
    want = torch.relu(W.float() @ X.float().t() + b.float()[:, None])
    y = ops.custom_aten_addmm("aten::relu", b.to(DEV), W.to(DEV), X.to(DEV).t())
    assert list(y.shape) == [48, 13] and maxabs(y, want) <= 1e-2
    y = ops.custom_aten_addmm("none", b.to(DEV), W.to(DEV), X.to(DEV).t().unsqueeze(0))   # 3-D mat2 is squeezed, result unsqueezed
    assert list(y.shape) == [1, 48, 13] and maxabs(y, W.float() @ X.float().t() + b.float()[:, None]) <= 1e-2
    y = ops.custom_aten_matmul(X.to(DEV), W.to(DEV).t())
    assert list(y.shape) == [13, 48] and maxabs(y, X.float() @ W.float().t()) <= 1e-2
    y = ops.aten_linear(X.to(DEV), W.to(DEV), b.to(DEV))
    assert list(y.shape) == [13, 48] and maxabs(y, X.float() @ W.float().t() + b.float()) <= 1e-2


def test_wrong_dtype_or_device_is_an_error_not_a_fallback(ops):
    x, A = torch.randn(1, 8), torch.randn(8, 8)
    with pytest.raises(ops.NNRuntimeException):
        ops.custom_aten_matmul(x.half(), A.half())                  # CPU tensors
    with pytest.raises(ops.NNRuntimeException):
        ops.custom_aten_matmul(x.to(DEV), A.to(DEV))                # fp32
    with pytest.raises(ops.NNRuntimeException):
        ops.aten_linear(x.half().to(DEV), A.half().to(DEV), torch.zeros(7).half().to(DEV))   # bias length


def test_rnnt_joint_split_gemvs(ops):
    """RemoveCatForAddmm splits the joint net's addmm over cat([f[1,1024], g[1,320]]) into two GEMVs on the two
    column blocks of the [512, 1344] weight (remove_cat_for_addmm.h:77-79): row-pitch views, summed."""
    g = torch.Generator().manual_seed(6)
    W, f, gg, b = rnd(g, 512, 1344, scale=0.05), rnd(g, 1, 1024, scale=1.0), rnd(g, 1, 320, scale=1.0), rnd(g, 512)
    want = torch.addmm(b.float(), torch.cat([f, gg], 1).float(), W.float().t())
    Wd = W.to(DEV)
    from pimaicompiler_amd import _lib as L
    lib = L.load()
    s = torch.cuda.current_stream().cuda_stream
    y1 = torch.empty(512, dtype=torch.float16, device=DEV)
    y2 = torch.empty(512, dtype=torch.float16, device=DEV)
    fd, gd, bd = f.to(DEV), gg.to(DEV), b.to(DEV)
    assert lib.pimhip_execute_gemv(y1.data_ptr(), fd.data_ptr(), Wd.data_ptr(), bd.data_ptr(), 1024, 512, 1344, 0, 1, s) == 0
    assert lib.pimhip_execute_gemv(y2.data_ptr(), gd.data_ptr(), Wd.data_ptr() + 2 * 1024, None, 320, 512, 1344, 0, 1, s) == 0
    assert maxabs(y1.float() + y2.float(), want) <= 2 * TOL
