"""GPU parity of the fp16 GEMV family, called through the C ABI (pimaicompiler_amd.ops -> libpimhip.so).

Checkers: the CPU oracle (oracle/oracle.c) at sizes it finishes in seconds, LibTorch CPU at::addmm live on the
same seeded inputs at the benchmark sizes, the committed LibTorch golden vectors, and size-independent properties
(zero / one-hot inputs, linearity in x, VM/MV symmetry) at full size.
Tolerance: max abs error <= 2e-3 on GEMV outputs (fp32 accumulation, one rounding to fp16)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import oracle
from pimaicompiler_amd import workloads

pytestmark = pytest.mark.gpu
GEMV_TOL = 2e-3
DEV = "cuda:0"


def maxabs(a, b):
    return float((a.detach().float().cpu().reshape(-1) - torch.as_tensor(np.asarray(b, dtype=np.float32)).reshape(-1)).abs().max())


def ulp_f16(v):
    v = np.abs(np.asarray(v, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(v, 2.0 ** -14)))
    return 2.0 ** (e - 10)


def raw_gemv(P, weight, x, bias, in_w, out_w, ld, act, order, stream=None):
    """Direct call of pimhip_execute_gemv on torch device buffers."""
    from pimaicompiler_amd import _lib as L
    out = torch.full((out_w,), float("nan"), dtype=torch.float16, device=DEV)
    rc = L.load().pimhip_execute_gemv(out.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                      bias.data_ptr() if bias is not None else None, in_w, out_w, ld, act, order,
                                      stream if stream is not None else torch.cuda.current_stream().cuda_stream)
    return rc, out


# ---- against the CPU oracle, both weight orders, ragged sizes -------------------------------------------------
SHAPES = [(1, 8), (1, 1), (3, 5), (7, 17), (16, 8), (64, 64), (100, 264), (255, 1000), (512, 1344), (1000, 24),
          (1024, 1024), (1023, 2056), (2049, 520), (8, 768), (768, 3072), (3072, 768), (33, 8200), (4, 16384)]


@pytest.mark.parametrize("n,k", SHAPES)
@pytest.mark.parametrize("bias,relu", [(True, False), (True, True), (False, False)])
def test_gemv_both_orders_match_oracle(ops, n, k, bias, relu):
    W, x, b = workloads.gemv_inputs(100 + n + k, n, k, bias=True)
    W = (W * 5).half()
    want = oracle.gemv_mv(W.numpy(), x.numpy().reshape(-1), b.numpy() if bias else None, relu=relu)
    from pimaicompiler_amd import _lib as L
    act = L.PIMHIP_ACT_RELU if relu else L.PIMHIP_ACT_NONE
    Wd, xd, bd = W.to(DEV), x.to(DEV).reshape(-1), (b.to(DEV) if bias else None)
    rc, y = raw_gemv(ops, Wd, xd, bd, k, n, 0, act, L.PIMHIP_W_X_I)
    assert rc == 0
    assert maxabs(y, want) <= GEMV_TOL
    Wt = W.t().contiguous().to(DEV)
    rc, y = raw_gemv(ops, Wt, xd, bd, k, n, 0, act, L.PIMHIP_I_X_W)
    assert rc == 0
    assert maxabs(y, want) <= GEMV_TOL


@pytest.mark.parametrize("n,k", [(7, 17), (512, 1344), (1024, 1024), (33, 8200), (4096, 4096)])
def test_relu_keeps_a_nan_as_at_relu_does(ops, n, k):
    """The reference applies at::relu to its GEMV's result (aten_ops.cpp:466, 704-705): a NaN stays a NaN, it does not
    become 0.  One NaN weight poisons one row, one NaN bias another; the oracle and both weight orders agree on which."""
    from pimaicompiler_amd import _lib as L
    W, x, b = workloads.gemv_inputs(300 + n + k, n, k, bias=True)
    W, b = W.clone(), b.clone()
    W[n // 2, k // 3] = float("nan")
    b[n - 1] = float("nan")
    want = oracle.gemv_mv(W.numpy(), x.numpy().reshape(-1), b.numpy(), relu=True)
    assert np.isnan(want[n // 2]) and np.isnan(want[n - 1]) and np.isnan(want).sum() == (1 if n // 2 == n - 1 else 2)
    xd, bd = x.to(DEV).reshape(-1), b.to(DEV)
    for weight, order in ((W.to(DEV), L.PIMHIP_W_X_I), (W.t().contiguous().to(DEV), L.PIMHIP_I_X_W)):
        rc, y = raw_gemv(ops, weight, xd, bd, k, n, 0, L.PIMHIP_ACT_RELU, order)
        assert rc == 0
        y = y.cpu().numpy()
        assert np.array_equal(np.isnan(y), np.isnan(want))
        assert np.nanmax(np.abs(y.astype(np.float32) - want.astype(np.float32))) <= GEMV_TOL and np.nanmin(y) >= 0.0


@pytest.mark.parametrize("n,k", [(7, 17), (1024, 1024), (4096, 4096)])
@pytest.mark.parametrize("x_scale", [256.0, 2.0 ** -6])
def test_subnormal_operands_and_results_are_not_flushed(ops, n, k, x_scale):
    """Weights and bias below the smallest normal fp16 (6.1e-5) are values like any other (LibTorch CPU does not flush
    them either); with the small x the results are subnormal too.  Within one ulp of the oracle's exactly rounded value."""
    torch.manual_seed(3)
    W = (torch.randn(n, k) * 2.0 ** -18).half()
    x = (torch.randn(k) * x_scale).half()
    b = (torch.randn(n) * 2.0 ** -16).half()
    assert float((W.abs() < 6.1e-5).float().mean()) > 0.99
    want = oracle.gemv_mv(W.numpy(), x.numpy(), b.numpy())
    assert np.abs(want.astype(np.float64)).max() > 0.0
    if x_scale < 1.0:
        assert np.mean(np.abs(want.astype(np.float64)) < 6.1e-5) > 0.9
    for weight, order_is_vm in ((W.to(DEV), False), (W.t().contiguous().to(DEV), True)):
        from pimaicompiler_amd import _lib as L
        rc, y = raw_gemv(ops, weight, x.to(DEV), b.to(DEV), k, n, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W if order_is_vm else L.PIMHIP_W_X_I)
        assert rc == 0
        y = y.cpu().numpy()
        assert np.all(np.abs(y.astype(np.float64) - want.astype(np.float64)) <= ulp_f16(want))
        assert np.mean(y.view(np.uint16) == want.view(np.uint16)) > 0.95


def test_gemv_result_is_correctly_rounded_almost_everywhere(ops):
    """fp32 accumulation then one rounding: the result is within one fp16 ulp of the exactly rounded value and
    equal to it for all but near-tie elements."""
    W, x, b = workloads.gemv_inputs(77, 2048, 2048)
    want = oracle.gemv_mv(W.numpy(), x.numpy().reshape(-1), b.numpy())
    y = ops.aten_linear(x.to(DEV), W.to(DEV), b.to(DEV)).cpu().numpy().reshape(-1)
    assert np.all(np.abs(y.astype(np.float64) - want.astype(np.float64)) <= ulp_f16(want))
    assert np.mean(y.view(np.uint16) == want.view(np.uint16)) > 0.97


def test_gemv_row_pitch_and_unaligned_pointers(ops):
    from pimaicompiler_amd import _lib as L
    g = torch.Generator().manual_seed(5)
    big = (0.1 * torch.randn(300, 1040, generator=g)).half()
    x = torch.randn(1024, generator=g).half()
    # MV on a [300, 1024] window of a wider matrix (pitch 1040), vector path (pitch % 8 == 0)
    want = oracle.gemv_mv(big[:, :1024].contiguous().numpy(), x.numpy())
    rc, y = raw_gemv(ops, big.to(DEV), x.to(DEV), None, 1024, 300, 1040, 0, L.PIMHIP_W_X_I)
    assert rc == 0 and maxabs(y, want) <= GEMV_TOL
    # window starting at column 3: 2-byte aligned only -> generic path
    bd = big.to(DEV)
    want = oracle.gemv_mv(big[:, 3:1027].contiguous().numpy(), x.numpy())
    out = torch.empty(300, dtype=torch.float16, device=DEV)
    rc = L.load().pimhip_execute_gemv(out.data_ptr(), x.to(DEV).data_ptr(), bd.data_ptr() + 6, None, 1024, 300, 1040,
                                      0, L.PIMHIP_W_X_I, torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and maxabs(out, want) <= GEMV_TOL
    # VM on a [1024, 296] window of a [1024, 300] matrix (pitch 300: not a multiple of 8 -> generic path)
    A = (0.1 * torch.randn(1024, 300, generator=g)).half()
    want = oracle.gemv_vm(x.numpy(), A[:, :296].contiguous().numpy())
    rc, y = raw_gemv(ops, A.to(DEV), x.to(DEV), None, 1024, 296, 300, 0, L.PIMHIP_I_X_W)
    assert rc == 0 and maxabs(y, want) <= GEMV_TOL


def test_gemv_argument_errors(ops):
    from pimaicompiler_amd import _lib as L
    lib = L.load()
    t = torch.zeros(64, dtype=torch.float16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.pimhip_execute_gemv(None, t.data_ptr(), t.data_ptr(), None, 8, 8, 0, 0, 1, s) == L.PIMHIP_ERR_INVALID_ARGUMENT
    assert lib.pimhip_execute_gemv(t.data_ptr(), t.data_ptr(), t.data_ptr(), None, 8, 8, 0, 7, 1, s) == L.PIMHIP_ERR_INVALID_ARGUMENT
    assert lib.pimhip_execute_gemv(t.data_ptr(), t.data_ptr(), t.data_ptr(), None, 8, 8, 0, 0, 5, s) == L.PIMHIP_ERR_INVALID_ARGUMENT
    assert lib.pimhip_execute_gemv(t.data_ptr(), t.data_ptr(), t.data_ptr(), None, 8, 8, 4, 0, 1, s) == L.PIMHIP_ERR_INVALID_ARGUMENT
    assert lib.pimhip_execute_gemv(t.data_ptr(), t.data_ptr(), t.data_ptr(), None, -1, 8, 0, 0, 1, s) == L.PIMHIP_ERR_INVALID_ARGUMENT
    assert b"in_w" in lib.pimhip_last_error()
    # empty products are legal: no output rows, or an empty reduction (y = bias)
    assert lib.pimhip_execute_gemv(t.data_ptr(), t.data_ptr(), t.data_ptr(), None, 8, 0, 0, 0, 1, s) == 0
    b = torch.arange(8, dtype=torch.float16, device=DEV)
    out = torch.full((8,), -1.0, dtype=torch.float16, device=DEV)
    for order in (0, 1):
        assert lib.pimhip_execute_gemv(out.data_ptr(), t.data_ptr(), t.data_ptr(), b.data_ptr(), 0, 8, 8, 0, order, s) == 0
        assert torch.equal(out, b)


# ---- benchmark configurations against LibTorch CPU, live and golden --------------------------------------------
CONFIGS = [("c1_1024x1024", 1001, 1024, 1024), ("c2_4096x4096", 2001, 4096, 4096), ("c2_16384x4096", 2002, 16384, 4096),
           ("c2_4096x16384", 2003, 4096, 16384), ("c2_32000x1024", 2004, 32000, 1024)]


@pytest.mark.parametrize("name,seed,n,k", CONFIGS)
def test_gemv_configs_match_libtorch_cpu_addmm(ops, golden, name, seed, n, k):
    W, x, b = workloads.gemv_inputs(seed, n, k)
    want = oracle.torch_addmm(b, x, W).reshape(-1)            # at::addmm(b, x, W^T), CPU, fp16
    # the op as the runtime issues it after its rewrite passes: addmm(b, W[out,in], x^T[in,1])
    y = ops.custom_aten_addmm("none", b.to(DEV), W.to(DEV), x.to(DEV).t())
    assert list(y.shape) == [n, 1]
    assert maxabs(y, want.numpy()) <= GEMV_TOL
    # and as aten::linear
    y2 = ops.aten_linear(x.to(DEV), W.to(DEV), b.to(DEV))
    assert list(y2.shape) == [1, n] and torch.equal(y2.reshape(-1), y.reshape(-1))
    g = golden["gemv"]
    if n <= 1024:
        assert maxabs(y, g[name + "_y"]) <= GEMV_TOL
    else:
        idx = g[name + "_idx"]
        assert maxabs(y.reshape(-1)[torch.as_tensor(idx)], g[name + "_y_samples"]) <= GEMV_TOL
        assert abs(float(y.double().sum()) - float(g[name + "_y_sum"][0])) <= GEMV_TOL * n ** 0.5


@pytest.mark.parametrize("n,k", [(16384, 4096), (4096, 16384), (32000, 1024)])
def test_gemv_full_size_properties(ops, n, k):
    g = torch.Generator().manual_seed(n + k)
    W = (0.02 * torch.randn(n, k, generator=g)).half().to(DEV)
    b = (0.01 * torch.randn(n, generator=g)).half().to(DEV)
    # zero input: y == bias exactly
    y = ops.aten_linear(torch.zeros(1, k, dtype=torch.float16, device=DEV), W, b)
    assert torch.equal(y.reshape(-1), b)
    # one-hot input: y == W[:, j] + b with one fp16 rounding, exactly
    for j in (0, k // 2 + 3, k - 1):
        e = torch.zeros(1, k, dtype=torch.float16, device=DEV)
        e[0, j] = 1.0
        y = ops.aten_linear(e, W, b).reshape(-1)
        assert torch.equal(y, (W[:, j].float() + b.float()).half())
    # linearity: W.(2x) == 2 (W.x): scaling by 2 commutes with every rounding above the subnormal range
    x = (2 * torch.rand(1, k, generator=g) - 1).half().to(DEV)
    y1 = ops.aten_linear(x, W).reshape(-1)
    y2 = ops.aten_linear((2 * x).half(), W).reshape(-1)
    assert float((2 * y1.float() - y2.float()).abs().max()) <= 2.0 ** -23  # exact except in the fp16 subnormal range
    # VM on the transposed bytes agrees with MV within fp32 reassociation
    yv = ops.custom_aten_matmul(x, W.t().contiguous())
    assert maxabs(yv, y1.cpu().numpy()) <= GEMV_TOL
    # the sum over all outputs against float64 on the host
    want = (W.cpu().double() @ x.cpu().double().reshape(-1)).sum().item()
    assert abs(float(y1.double().sum()) - want) <= GEMV_TOL * n ** 0.5


@pytest.mark.parametrize("n,k", [(4096, 4096), (32000, 1024), (1024, 1024), (520, 4104)])
def test_gemv_vm_order_full_size_properties(ops, n, k):
    """The VM order splits K over blocks; its cross-block sum has a fixed order, so repeated launches agree to the bit."""
    from pimaicompiler_amd import _lib as L
    g = torch.Generator().manual_seed(n * 3 + k)
    A = (0.02 * torch.randn(k, n, generator=g)).half().to(DEV)
    b = (0.01 * torch.randn(n, generator=g)).half().to(DEV)
    x = (2 * torch.rand(k, generator=g) - 1).half().to(DEV)
    rc, y0 = raw_gemv(ops, A, x, b, k, n, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W)
    assert rc == 0
    for _ in range(10):
        rc, y = raw_gemv(ops, A, x, b, k, n, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W)
        assert rc == 0 and torch.equal(y, y0)
    want = (x.cpu().double() @ A.cpu().double() + b.cpu().double()).numpy()
    assert maxabs(y0, want) <= GEMV_TOL
    # zero input: y == bias exactly; one-hot input: y == A[j, :] + b with one rounding, exactly
    rc, y = raw_gemv(ops, A, torch.zeros_like(x), b, k, n, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W)
    assert torch.equal(y, b)
    for j in (0, k // 3 + 1, k - 1):
        e = torch.zeros_like(x)
        e[j] = 1.0
        rc, y = raw_gemv(ops, A, e, b, k, n, 0, L.PIMHIP_ACT_RELU, L.PIMHIP_I_X_W)
        assert torch.equal(y, torch.relu((A[j].float() + b.float()).half()))
    # several destinations receive the same bits
    outs = [torch.empty(n, dtype=torch.float16, device=DEV) for _ in range(3)]
    ops.aten_bmm(x.reshape(1, 1, k), A.reshape(1, k, n), outs=outs)
    rc, ynb = raw_gemv(ops, A, x, None, k, n, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W)
    assert all(torch.equal(o, ynb) for o in outs)


def test_sliced_vm_product_whose_reducers_give_up_has_the_bits_it_would_have_had(ops):
    """A reducing block that gives up its wait (forced from the host: with a spin limit of 0 it does not poll at all, and
    every kernel still ends by itself) computes the missing partial sums itself, in the order their own block makes them:
    the product that timed out equals the undisturbed one bit for bit.  So do the products after it on the stream, which
    ignore the records until one issued outside a capture has put the workspace back in order; the events are counted."""
    from pimaicompiler_amd import _lib as L
    n, k = 4096, 4096
    g = torch.Generator().manual_seed(77)
    A = (0.02 * torch.randn(k, n, generator=g)).half().to(DEV)
    x = (2 * torch.rand(k, generator=g) - 1).half().to(DEV)
    b = (0.1 * torch.randn(n, generator=g)).half().to(DEV)
    rc, y0 = raw_gemv(ops, A, x, b, k, n, 0, L.PIMHIP_ACT_RELU, L.PIMHIP_I_X_W)
    assert rc == 0
    torch.cuda.synchronize()
    assert ops.gemv_status() == (False, False)
    before = ops.gemv_fallbacks()
    ops.set_gemv_spin_limit(0)
    try:
        for i in range(3):
            rc, y = raw_gemv(ops, A, x, b, k, n, 0, L.PIMHIP_ACT_RELU, L.PIMHIP_I_X_W)
            assert rc == 0
            torch.cuda.synchronize()
            assert torch.equal(y, y0), i
            assert ops.gemv_status() == (True, False) and ops.gemv_fallbacks() == before + i + 1
    finally:
        ops.set_gemv_spin_limit(1 << 22)
    rc, y = raw_gemv(ops, A, x, b, k, n, 0, L.PIMHIP_ACT_RELU, L.PIMHIP_I_X_W)     # puts the workspace back in order on its way
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(y, y0) and ops.gemv_status() == (False, False) and ops.gemv_fallbacks() == before + 3
    # a record that arrives after its reducer has given up must not pass for the next product's: another matrix, same stream
    A2 = (0.02 * torch.randn(k, n, generator=g)).half().to(DEV)
    rc, want2 = raw_gemv(ops, A2, x, None, k, n, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W)
    torch.cuda.synchronize()
    ops.set_gemv_spin_limit(0)
    try:
        raw_gemv(ops, A, x, None, k, n, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W)
        rc, y2 = raw_gemv(ops, A2, x, None, k, n, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W)
    finally:
        ops.set_gemv_spin_limit(1 << 22)
    torch.cuda.synchronize()
    assert rc == 0 and torch.equal(y2, want2)
    ops.synchronize_and_check()


@pytest.mark.parametrize("n1,n2,out_w,bias,act", [(1024, 320, 512, True, "aten::relu"), (8, 8, 1, False, "none"), (4096, 64, 2000, True, "none"),
                                                  (136, 4104, 77, True, "aten::relu"), (512, 512, 4096, False, "none")])
def test_gemv_over_two_separate_inputs_matches_libtorch_on_their_concatenation(ops, n1, n2, out_w, bias, act):
    g = torch.Generator().manual_seed(n1 + n2)
    W = (torch.randn(out_w, n1 + n2, generator=g) / (n1 + n2) ** 0.5).half()
    b = (0.1 * torch.randn(out_w, generator=g)).half() if bias else None
    x1, x2 = torch.randn(1, n1, generator=g).half(), torch.randn(1, n2, generator=g).half()
    want = torch.nn.functional.linear(torch.cat([x1, x2], -1), W, b)
    want = torch.relu(want) if act == "aten::relu" else want
    y = ops.aten_linear_cat2(x1.to(DEV), x2.to(DEV), W.to(DEV), b.to(DEV) if bias else None, act_type=act)
    assert list(y.shape) == [1, out_w] and maxabs(y, want.numpy()) <= GEMV_TOL
    # the same bits as the one-input launch on the concatenation (same kernel shape, same order of sums)
    y1 = ops.aten_linear(torch.cat([x1, x2], -1).to(DEV), W.to(DEV), b.to(DEV) if bias else None, act_type=act)
    assert torch.equal(y, y1)
    # a weight that is a column block of a wider matrix (row pitch larger than the two widths together)
    wide = torch.zeros(out_w, n1 + n2 + 24, dtype=torch.float16)
    wide[:, :n1 + n2] = W
    yv = ops.aten_linear_cat2(x1.to(DEV), x2.to(DEV), wide.to(DEV)[:, :n1 + n2], b.to(DEV) if bias else None, act_type=act)
    assert torch.equal(yv, y)


def test_gemv_over_two_inputs_with_widths_the_launch_does_not_take(ops):
    g = torch.Generator().manual_seed(3)
    W = (0.05 * torch.randn(40, 12 + 20, generator=g)).half()
    x1, x2 = torch.randn(1, 12, generator=g).half(), torch.randn(1, 20, generator=g).half()
    y = ops.aten_linear_cat2(x1.to(DEV), x2.to(DEV), W.to(DEV))          # 12 is no multiple of 8: concatenated, then one GEMV
    assert maxabs(y, torch.nn.functional.linear(torch.cat([x1, x2], -1), W).numpy()) <= GEMV_TOL
    from pimaicompiler_amd import _lib as L
    lib = L.load()
    out = torch.empty(40, dtype=torch.float16, device=DEV)
    rc = lib.pimhip_execute_gemv_cat2(out.data_ptr(), x1.to(DEV).data_ptr(), 12, x2.to(DEV).data_ptr(), 20, W.to(DEV).data_ptr(), None, 40, 0,
                                      L.PIMHIP_ACT_NONE, None)
    assert rc == L.PIMHIP_ERR_UNSUPPORTED


def test_moe_ffn_decode_step_matches_libtorch(ops, golden):
    import importlib.util, os
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(__file__), "golden", "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    Wr, W1, W2, x = mg.moe_inputs()
    g = golden["moe"]
    xd = x.to(DEV)
    logits = ops.aten_linear(xd, Wr.to(DEV))
    assert maxabs(logits, g["logits"]) <= GEMV_TOL
    e = int(torch.argmax(logits.float()))
    assert e == int(g["expert"][0])
    hidden = ops.aten_linear(xd, W1[e].to(DEV), act_type="aten::relu")
    y = ops.aten_linear(hidden, W2[e].to(DEV))
    assert maxabs(hidden, g["hidden"]) <= GEMV_TOL
    assert maxabs(y, g["y"]) <= GEMV_TOL
    # live LibTorch CPU on the same tensors
    want = torch.matmul(torch.relu(torch.matmul(x, W1[e].t())), W2[e].t())
    assert maxabs(y, want.numpy()) <= GEMV_TOL


# ---- the reference's own unit test and kernels -----------------------------------------------------------------
def test_reference_custom_gemv_unit_test_pattern(ops):
    """runtime/unit-tests/custom_op_ut.cpp:20-69: x[1,1,1,1024] . A[1024,4096] and A[4096,1024] . x[1,1,1024,1]
    with U[0,1) fp16 inputs against at::matmul, allclose(atol 1e-3, rtol 1e-5).  Outputs are around 256 where one
    fp16 ulp is 0.25, so the comparison is made where it is meaningful: our fp16 result must be the rounding of a
    value that lies within the reference's tolerance of the exact product."""
    g = torch.Generator().manual_seed(1)
    for order in ("xAy", "Axy"):
        if order == "xAy":
            a, b = torch.rand(1, 1, 1, 1024, generator=g).half(), torch.rand(1024, 4096, generator=g).half()
        else:
            a, b = torch.rand(4096, 1024, generator=g).half(), torch.rand(1, 1, 1024, 1, generator=g).half()
        y = ops.custom_aten_matmul(a.to(DEV), b.to(DEV))
        exact = torch.matmul(a.double(), b.double())
        assert list(y.shape) == list(exact.shape)
        err = (y.double().cpu() - exact).abs().numpy()
        assert np.all(err <= 0.5 * ulp_f16(exact.numpy()) + 1e-3 + 1e-5 * np.abs(exact.numpy()))


def test_against_the_references_own_hip_kernels(ops):
    """The reference's gemvt / addmv kernels (custom_ops.h), compiled from its tree, on the same device buffers.
    They round every product to fp16 before accumulating, so agreement is to tolerance, not to the bit."""
    ref = oracle.ref_lib()
    if ref is None:
        pytest.skip("oracle/_ref was not built (reference tree absent at build time)")
    W, x, b = workloads.gemv_inputs(31, 4096, 1024)
    Wd, xd, bd = W.to(DEV), x.to(DEV).reshape(-1), b.to(DEV)
    s = torch.cuda.current_stream().cuda_stream
    out = torch.zeros(4096, dtype=torch.float16, device=DEV)
    ref.ref_addmv_Axy(s, bd.data_ptr(), Wd.data_ptr(), xd.data_ptr(), out.data_ptr(), 4096, 1024, 1)
    y = ops.aten_linear(xd.reshape(1, -1), Wd, bd, act_type="aten::relu").reshape(-1)
    assert maxabs(y, out.cpu().numpy()) <= GEMV_TOL
    Wt = W.t().contiguous().to(DEV)
    out2 = torch.zeros(4096, dtype=torch.float16, device=DEV)
    ref.ref_gemv_xAy(s, xd.data_ptr(), Wt.data_ptr(), out2.data_ptr(), 4096, 1024)
    y2 = ops.custom_aten_matmul(xd.reshape(1, -1), Wt).reshape(-1)
    assert maxabs(y2, out2.cpu().numpy()) <= GEMV_TOL


# ---- dot, grouped launch, streams ------------------------------------------------------------------------------
@pytest.mark.parametrize("k", [1, 7, 64, 1024, 5000, 70001])
def test_dot_matches_oracle(ops, k):
    g = torch.Generator().manual_seed(k)
    a, b = (0.3 * torch.randn(1, k, generator=g)).half(), (0.3 * torch.randn(k, 1, generator=g)).half()
    y = ops.custom_aten_matmul(a.to(DEV), b.to(DEV)) if k > 1 else None
    want = oracle.dot(a.numpy().reshape(-1), b.numpy().reshape(-1))
    if k == 1:  # [1,1] x [1,1] is not a vector product for getGemmType; call the entry point directly
        from pimaicompiler_amd import _lib as L
        out = torch.empty(1, dtype=torch.float16, device=DEV)
        assert L.load().pimhip_execute_dot(out.data_ptr(), a.to(DEV).data_ptr(), b.to(DEV).data_ptr(), 1,
                                           torch.cuda.current_stream().cuda_stream) == 0
        y = out
    assert abs(float(y.reshape(-1)[0]) - float(want[0])) <= max(GEMV_TOL, float(ulp_f16(float(want[0]))))


def test_gemv_group_equals_separate_launches(ops):
    g = torch.Generator().manual_seed(9)
    shapes = [(768, 768)] * 4 + [(3072, 768), (8, 768), (768, 3072), (1000, 1024)] + [(64, 64)] * 40
    ws = [(0.05 * torch.randn(n, k, generator=g)).half().to(DEV) for n, k in shapes]
    xs = [torch.randn(1, k, generator=g).half().to(DEV) for n, k in shapes]
    bs = [(0.1 * torch.randn(n, generator=g)).half().to(DEV) if i % 2 == 0 else None for i, (n, k) in enumerate(shapes)]
    acts = ["aten::relu" if i % 3 == 0 else "none" for i in range(len(shapes))]
    outs = ops.execute_gemv_group(xs, ws, bs, acts)
    for i, (w, x, b, a, o) in enumerate(zip(ws, xs, bs, acts, outs)):
        single = ops.aten_linear(x, w, b, act_type=a).reshape(-1)
        assert maxabs(o, single.cpu().numpy()) <= 1e-3, i
        want = oracle.gemv_mv(w.cpu().numpy(), x.cpu().numpy().reshape(-1), b.cpu().numpy() if b is not None else None, relu=a == "aten::relu")
        assert maxabs(o, want) <= GEMV_TOL, i


def test_sibling_gemvs_on_separate_streams(ops):
    """executeMultiStream's pattern (stream_ops_executor.cpp:36-47): N GEMVs on N streams, VM order so that the
    split-K workspaces are exercised concurrently; every branch honours its stream."""
    g = torch.Generator().manual_seed(10)
    n_streams = 4
    streams = [torch.cuda.Stream() for _ in range(n_streams)]
    A = [(0.05 * torch.randn(2048, 1024, generator=g)).half().to(DEV) for _ in range(n_streams)]
    x = [torch.randn(1, 2048, generator=g).half().to(DEV) for _ in range(n_streams)]
    torch.cuda.synchronize()
    outs = []
    for rep in range(3):
        outs = []
        for i, s in enumerate(streams):
            with torch.cuda.stream(s):
                outs.append(ops.custom_aten_matmul(x[i], A[i], stream=s))
    torch.cuda.synchronize()
    for i in range(n_streams):
        want = oracle.gemv_vm(x[i].cpu().numpy().reshape(-1), A[i].cpu().numpy())
        assert maxabs(outs[i], want) <= GEMV_TOL
