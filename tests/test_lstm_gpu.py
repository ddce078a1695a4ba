"""GPU parity of the LSTM path (fused step kernel, persistent sequence kernel, MFMA input projection), called
through the C ABI.  Checkers: LibTorch CPU at::lstm live on the same seeded inputs (fp16, the arbiter, and fp32 on
the same fp16-valued weights), the committed LibTorch golden vectors, the CPU oracle, and structural properties.
Tolerance: max abs error <= 5e-3 on y / h / c after the full sequence."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle
from pimaicompiler_amd import workloads

pytestmark = pytest.mark.gpu
LSTM_TOL = 5e-3
DEV = "cuda:0"
# 1: one fused launch per step, 2: persistent sequence kernel over all CUs, 3: the same, four units per block always,
# 4: every recurrence on one XCD (hidden sizes up to 1024)
MODES = [1, 2, 3, 4]


def maxabs(a, b):
    b = b if isinstance(b, torch.Tensor) else torch.as_tensor(np.asarray(b, dtype=np.float32))
    return float((a.detach().float().cpu().reshape(-1) - b.float().reshape(-1)).abs().max())


def run_plan(ops, params, x, h0, c0, has_b, L, bidir, mode, T=None, measure=True):
    T = x.shape[0] if T is None else T
    plan = ops.LstmPlan([p.to(DEV) for p in params], has_b, L, bidir, max(T, 1))
    if mode:
        plan.set_mode(mode)
    plan.set_measure(measure)
    y, hn, cn = plan.forward(x.reshape(x.shape[0], -1).to(DEV), h0.to(DEV), c0.to(DEV))
    plan.status()
    return y, hn, cn


# ---- tiny golden cases (LibTorch CPU, committed) --------------------------------------------------------------
TINY = [f"L{L}_D{D}_b{b}" for L in (1, 2) for D in (1, 2) for b in (1, 0)]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("key", TINY)
def test_lstm_tiny_golden(ops, golden, key, mode):
    g = golden["lstm_tiny"]
    L, D, has_b = int(key[1]), int(key[4]), int(key[7])
    n = L * D * (4 if has_b else 2)
    params = [torch.as_tensor(g[f"{key}_p{i}"]) for i in range(n)]
    x, h0, c0 = (torch.as_tensor(g[key + s]) for s in ("_x", "_h0", "_c0"))
    y, hn, cn = run_plan(ops, params, x, h0, c0, has_b, L, D == 2, mode)
    assert maxabs(y, g[key + "_y"]) <= 2e-3
    assert maxabs(hn, g[key + "_hn"]) <= 2e-3
    assert maxabs(cn, g[key + "_cn"]) <= 2e-3


# ---- against the CPU oracle over ragged shapes ---------------------------------------------------------------
CASES = [  # I, H, L, bidirectional, T, biases
    (8, 8, 1, False, 1, True), (8, 8, 1, False, 2, True), (24, 40, 1, False, 9, True), (64, 320, 1, False, 13, True),
    (16, 72, 2, True, 6, True), (32, 128, 3, False, 5, False), (32, 128, 3, True, 4, True), (240, 512, 2, False, 17, True),
    (8, 1024, 1, False, 3, True), (40, 1032, 1, False, 3, True), (16, 2048, 1, True, 2, False),
    (16, 64, 4, False, 7, True), (16, 64, 5, False, 6, True), (24, 136, 7, False, 3, False), (16, 64, 4, False, 1, True),
    (16, 64, 2, False, 2, True), (32, 1024, 4, False, 5, True),
    # 1024 < H <= 2048: the persistent kernel with 32 columns per lane, one layer (or two directions) per launch
    (32, 2048, 1, False, 5, True), (16, 1536, 2, False, 4, True), (24, 2048, 2, True, 3, True), (8, 1040, 3, False, 6, False),
    (8, 2056, 1, False, 3, True),
    # layer 1 of a bidirectional stack at 65 <= T <= 256 with a 2048-wide input: the packed projection with
    # eight wavefronts per block and 32-column tiles
    (64, 1024, 2, True, 70, True),
    # unidirectional stacks long enough for the pipeline over the XCDs to fill and for its LDS rings to wrap (mode 4 and,
    # from 32 / 16 steps, automatic mode): two, four (one launch), five and nine layers (two and three launches)
    (40, 264, 2, False, 45, True), (24, 520, 4, False, 37, False), (16, 72, 5, False, 35, True), (8, 136, 9, False, 18, True),
]


@pytest.mark.parametrize("mode", [0] + MODES)
@pytest.mark.parametrize("I,H,L,bidir,T,has_b", CASES)
def test_lstm_matches_oracle(ops, I, H, L, bidir, T, has_b, mode):
    if mode >= 2 and H > 2048:
        pytest.skip("the persistent kernel takes hidden sizes up to 2048; larger ones run step by step")
    if mode == 4 and H > 1024:
        pytest.skip("one XCD's registers hold the recurrent weights of hidden sizes up to 1024")
    params, x, h0, c0 = workloads.lstm_inputs(900 + I + H + T, I, H, L, bidir, T, has_b)
    g = torch.Generator().manual_seed(T)
    h0 = (0.3 * torch.randn(h0.shape, generator=g)).half()
    c0 = (0.3 * torch.randn(c0.shape, generator=g)).half()
    D = 2 if bidir else 1
    wy, whn, wcn = oracle.lstm(x.numpy().reshape(T, I), h0.numpy().reshape(L * D, H), c0.numpy().reshape(L * D, H),
                               [p.numpy() for p in params], has_b, L, bidir)
    y, hn, cn = run_plan(ops, params, x, h0, c0, has_b, L, bidir, mode)
    assert maxabs(y, wy) <= 2e-3 and maxabs(hn, whn) <= 2e-3 and maxabs(cn, wcn) <= 2e-3


# ---- stacks with residual sums (the GNMT wiring): layer by layer on LibTorch CPU ----------------------------------
RESIDUAL_CASES = [  # I, H, L, first residual layer, T, biases
    (2048, 1024, 3, 1, 50, True),    # the GNMT encoder above its bidirectional layer
    (64, 64, 4, 2, 20, True),
    (128, 128, 2, 0, 9, False),      # the first layer too (its input is the call's)
    (40, 40, 5, 1, 33, True),        # a last pipeline launch of one layer
    (1024, 1024, 1, 0, 70, True),    # a single layer
    (72, 72, 3, 2, 1, True),         # one step
    (24, 136, 6, 3, 5, True),
]


def libtorch_residual_stack(params, x, h0, c0, has_b, L, first_res):
    """One at::lstm and one at::add per layer, fp16 on the CPU: what the reference's interpreter runs."""
    per = 4 if has_b else 2
    cur, hs, cs = x, [], []
    for l in range(L):
        y, hn, cn = torch.lstm(cur, (h0[l:l + 1], c0[l:l + 1]), params[l * per:(l + 1) * per], has_b, 1, 0.0, False, False, False)
        hs.append(hn)
        cs.append(cn)
        cur = y + cur if l >= first_res else y
    return cur, torch.cat(hs, 0), torch.cat(cs, 0)


@pytest.mark.parametrize("mode", [0, 1, 2, 4])
@pytest.mark.parametrize("I,H,L,first_res,T,has_b", RESIDUAL_CASES)
def test_residual_stack_matches_libtorch_layer_by_layer(ops, I, H, L, first_res, T, has_b, mode):
    params, x, h0, c0 = workloads.lstm_inputs(700 + H + T, I, H, L, False, T, has_b)
    g = torch.Generator().manual_seed(T)
    h0 = (0.3 * torch.randn(h0.shape, generator=g)).half()
    c0 = (0.3 * torch.randn(c0.shape, generator=g)).half()
    want_y, want_hn, want_cn = libtorch_residual_stack(params, x, h0, c0, has_b, L, first_res)
    plan = ops.LstmPlan([p.to(DEV) for p in params], has_b, L, False, T)
    if mode:
        plan.set_mode(mode)
    plan.set_residual(first_res)
    for rep in range(2):                              # a second call finds the hand-over slots of the first
        y, hn, cn = plan.forward(x.reshape(T, I).to(DEV), h0.to(DEV), c0.to(DEV))
        plan.status()
        assert maxabs(y, want_y) <= LSTM_TOL and maxabs(hn, want_hn) <= LSTM_TOL and maxabs(cn, want_cn) <= LSTM_TOL
    # switched off again, the plan is a plain stack
    plan.set_residual(None)
    y, hn, cn = plan.forward(x.reshape(T, I).to(DEV), h0.to(DEV), c0.to(DEV))
    plan.status()
    wy, whn, wcn = torch.lstm(x, (h0, c0), params, has_b, L, 0.0, False, False, False)
    assert maxabs(y, wy) <= LSTM_TOL and maxabs(hn, whn) <= LSTM_TOL


def test_residual_needs_equal_widths_and_one_direction(ops):
    params, x, h0, c0 = workloads.lstm_inputs(1, 64, 32, 2, False, 4)
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 2, False, 4)
    with pytest.raises(ops.NNRuntimeException):
        plan.set_residual(0)                          # layer 0 is 64 wide, its output 32
    plan.set_residual(1)
    params, x, h0, c0 = workloads.lstm_inputs(1, 32, 32, 2, True, 4)
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 2, True, 4)
    with pytest.raises(ops.NNRuntimeException):
        plan.set_residual(1)


def test_persistent_kernel_refuses_what_it_cannot_hold(ops):
    params, x, h0, c0 = workloads.lstm_inputs(1, 16, 2056, 1, False, 2)
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 1, False, 2)
    with pytest.raises(ops.NNRuntimeException):
        plan.set_mode(2)
    params, x, h0, c0 = workloads.lstm_inputs(1, 16, 1032, 1, False, 2)
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 1, False, 2)
    plan.set_mode(2)
    with pytest.raises(ops.NNRuntimeException, match="XCD"):
        plan.set_mode(4)


# ---- benchmark configurations -----------------------------------------------------------------------------------
@pytest.mark.parametrize("mode", MODES)
def test_lstm_c3_rnnt_matches_libtorch_cpu(ops, golden, mode):
    """2 layers unidirectional, I=240, H=1024, T=200."""
    params, x, h0, c0 = workloads.lstm_inputs(3001, 240, 1024, 2, False, 200)
    wy, whn, wcn = oracle.torch_lstm(x, h0, c0, params, True, 2, False)                      # fp16 CPU (arbiter)
    fy, fhn, fcn = oracle.torch_lstm(x.float(), h0.float(), c0.float(), [p.float() for p in params], True, 2, False)
    y, hn, cn = run_plan(ops, params, x, h0, c0, True, 2, False, mode)
    for got, w16, w32 in ((y, wy, fy), (hn, whn, fhn), (cn, wcn, fcn)):
        assert maxabs(got, w16) <= LSTM_TOL
        assert maxabs(got, w32) <= LSTM_TOL
    g = golden["lstm_large"]
    assert maxabs(hn, g["c3_hn"]) <= LSTM_TOL and maxabs(cn, g["c3_cn"]) <= LSTM_TOL
    assert maxabs(y.reshape(200, 1024)[::25, ::16], g["c3_y_samples"]) <= LSTM_TOL


def test_lstm_c4_gnmt_stack_matches_libtorch_cpu(ops, golden):
    """Four at::lstm calls as GNMT composes them (L0 bidirectional I=1024 -> 2048, L1 I=2048, L2, L3 I=1024), T=50,
    then the 1024 -> 32000 classifier GEMV on the last step's output."""
    g = golden["lstm_large"]
    seq_dev, seq_cpu = None, None
    for li, (in_w, bidir) in enumerate([(1024, True), (2048, False), (1024, False), (1024, False)]):
        params, x0, h0, c0 = workloads.lstm_inputs(4001 + li, in_w, 1024, 1, bidir, 50)
        if seq_dev is None:
            seq_dev, seq_cpu = x0.to(DEV), x0
        wy, whn, wcn = oracle.torch_lstm(seq_cpu, h0, c0, params, True, 1, bidir)
        y, hn, cn = ops.aten_lstm1(seq_dev, (h0.to(DEV), c0.to(DEV)), [p.to(DEV) for p in params], True, 1, 0.0, False,
                                   bidir, False)
        D = 2 if bidir else 1
        assert list(y.shape) == [50, 1, D * 1024] and list(hn.shape) == [D, 1, 1024] and list(cn.shape) == [D, 1, 1024]
        assert maxabs(y, wy) <= LSTM_TOL and maxabs(hn, whn) <= LSTM_TOL and maxabs(cn, wcn) <= LSTM_TOL
        assert maxabs(hn, g[f"c4_l{li}_hn"]) <= LSTM_TOL and maxabs(cn, g[f"c4_l{li}_cn"]) <= LSTM_TOL
        assert maxabs(y.reshape(50, -1)[::7, ::32], g[f"c4_l{li}_y_samples"]) <= LSTM_TOL
        seq_dev, seq_cpu = y, wy
    W, _, b = workloads.gemv_inputs(4010, 32000, 1024)
    logits = ops.aten_linear(seq_dev[-1].reshape(1, 1024), W.to(DEV), b.to(DEV)).reshape(-1)
    want = oracle.torch_addmm(b, seq_cpu[-1].reshape(1, 1024), W).reshape(-1)
    # the GEMV input differs by the LSTM's own error (<= 5e-3 per element) times |W| summed: allow for it
    assert maxabs(logits, want) <= 2e-3 + LSTM_TOL * 0.02 * math.sqrt(1024) * 0.5
    assert maxabs(logits[torch.as_tensor(g["c4_logits_idx"])], g["c4_logits_samples"]) <= 2e-3 + LSTM_TOL * 0.02 * math.sqrt(1024) * 0.5


# ---- interface forms --------------------------------------------------------------------------------------------
def test_lstm1_batch_first_and_lstm2_packed_agree(ops):
    params, x, h0, c0 = workloads.lstm_inputs(55, 32, 64, 2, True, 6)
    pd = [p.to(DEV) for p in params]
    hx = (h0.to(DEV), c0.to(DEV))
    y, hn, cn = ops.aten_lstm1(x.to(DEV), hx, pd, True, 2, 0.5, False, True, False)       # dropout is ignored
    yb, hnb, cnb = ops.aten_lstm1(x.to(DEV).transpose(0, 1), hx, pd, True, 2, 0.0, False, True, True)
    assert list(y.shape) == [6, 1, 128] and list(yb.shape) == [1, 6, 128]
    assert torch.equal(y.reshape(-1), yb.reshape(-1)) and torch.equal(hn, hnb) and torch.equal(cn, cnb)
    yp, hnp, cnp = ops.aten_lstm2(x.to(DEV).reshape(6, 32), torch.ones(6, dtype=torch.int64), hx, pd, True, 2, 0.0, False, True)
    assert list(yp.shape) == [6, 128]
    assert torch.equal(y.reshape(-1), yp.reshape(-1)) and torch.equal(hn, hnp) and torch.equal(cn, cnp)
    wy, whn, wcn = oracle.torch_lstm(x, h0, c0, params, True, 2, True)
    assert maxabs(y, wy) <= 2e-3 and maxabs(hn, whn) <= 2e-3 and maxabs(cn, wcn) <= 2e-3
    with pytest.raises(ops.NNRuntimeException):
        ops.aten_lstm1(x.to(DEV).repeat(1, 2, 1), hx, pd, True, 2, 0.0, False, True, False)   # batch 2
    with pytest.raises(ops.NNRuntimeException):
        ops.aten_lstm2(x.to(DEV).reshape(6, 32), torch.tensor([2, 1, 1, 1, 1, 0]), hx, pd, True, 2, 0.0, False, True)


def test_lstm_decode_loop_step_by_step_equals_one_sequence_call(ops):
    """The decoders call aten::lstm with seq_len == 1 inside prim::Loop, feeding (hy, cy) back: T such calls must
    reproduce one call over the whole sequence (same rounding points: h fp16 every step; c passes through fp16
    between calls, so c is compared to tolerance)."""
    params, x, h0, c0 = workloads.lstm_inputs(66, 64, 256, 2, False, 12)
    pd = [p.to(DEV) for p in params]
    y_all, hn_all, cn_all = ops.aten_lstm1(x.to(DEV), (h0.to(DEV), c0.to(DEV)), pd, True, 2, 0.0, False, False, False)
    h, c = h0.to(DEV), c0.to(DEV)
    ys = []
    for t in range(12):
        y, h, c = ops.aten_lstm1(x[t:t + 1].to(DEV), (h, c), pd, True, 2, 0.0, False, False, False)
        ys.append(y)
    assert maxabs(torch.cat(ys), y_all.cpu()) <= 2e-3
    assert maxabs(h, hn_all.cpu()) <= 2e-3 and maxabs(c, cn_all.cpu()) <= 2e-3


def test_lstm_zero_length_sequence_passes_state_through(ops):
    params, x, h0, c0 = workloads.lstm_inputs(77, 16, 32, 1, False, 4)
    g = torch.Generator().manual_seed(1)
    h0 = torch.randn(h0.shape, generator=g).half()
    c0 = torch.randn(c0.shape, generator=g).half()
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 1, False, 4)
    y, hn, cn = plan.forward(x[:0].reshape(0, 16).to(DEV), h0.to(DEV), c0.to(DEV))
    assert y.shape[0] == 0 and torch.equal(hn.cpu().reshape(-1), h0.reshape(-1)) and torch.equal(cn.cpu().reshape(-1), c0.reshape(-1))


def test_lstm_plan_reuse_and_sequence_longer_than_plan(ops):
    params, x, h0, c0 = workloads.lstm_inputs(88, 16, 64, 1, False, 20)
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 1, False, 10)
    with pytest.raises(ops.NNRuntimeException):
        plan.forward(x.reshape(20, 16).to(DEV), h0.to(DEV), c0.to(DEV))
    want = oracle.torch_lstm(x[:10], h0, c0, params, True, 1, False)
    for _ in range(3):  # exchange tags keep advancing across launches of one plan
        y, hn, cn = plan.forward(x[:10].reshape(10, 16).to(DEV), h0.to(DEV), c0.to(DEV))
        plan.status()
        assert maxabs(y, want[0]) <= 2e-3 and maxabs(cn, want[2]) <= 2e-3


# ---- structure at full size -------------------------------------------------------------------------------------
def test_lstm_full_size_zero_weights_closed_form(ops):
    H, I, T = 1024, 240, 40
    b_ih = torch.cat([torch.full((H,), 0.5), torch.full((H,), -1.0), torch.full((H,), 2.0), torch.full((H,), 0.25)]).half()
    b_hh = torch.cat([torch.full((H,), 0.25), torch.full((H,), 0.5), torch.full((H,), -0.5), torch.full((H,), 1.0)]).half()
    params = [torch.zeros(4 * H, I).half(), torch.zeros(4 * H, H).half(), b_ih, b_hh]
    x = torch.randn(T, 1, I).half()
    h0, c0 = torch.zeros(1, 1, H).half(), torch.full((1, 1, H), 0.75).half()
    sig = lambda v: 1 / (1 + math.exp(-v))
    i, f, g, o = sig(0.75), sig(-0.5), math.tanh(1.5), sig(1.25)
    for mode in MODES:
        y, hn, cn = run_plan(ops, params, x, h0, c0, True, 1, False, mode)
        c = 0.75
        for t in range(T):
            c = f * c + i * g
            assert float((y[t].float() - o * math.tanh(c)).abs().max()) <= 6e-4
        assert float((cn.float() - c).abs().max()) <= 1e-3


def test_lstm_bidirectional_equals_forward_on_reversed_input(ops):
    params, x, h0, c0 = workloads.lstm_inputs(99, 128, 1024, 1, True, 24)
    y, hn, cn = run_plan(ops, params, x, h0, c0, True, 1, True, 2)
    yf, hf, cf = run_plan(ops, params[:4], x, h0[:1], c0[:1], True, 1, False, 2)
    yb, hb, cb = run_plan(ops, params[4:], x.flip(0), h0[1:], c0[1:], True, 1, False, 2)
    # The fused two-direction launch and the single-chain launch are different instantiations of the kernel: the
    # compiler may contract multiply-adds differently, so agreement is to a rounding of h, not to the bit.
    assert maxabs(y[:, :1024], yf.cpu()) <= 1e-3 and maxabs(y[:, 1024:], yb.flip(0).cpu()) <= 1e-3
    assert maxabs(hn[0], hf[0].cpu()) <= 1e-3 and maxabs(hn[1], hb[0].cpu()) <= 1e-3 and maxabs(cn[1], cb[0].cpu()) <= 1e-3
    assert torch.equal(hn[1], y[0, 1024:]) and torch.equal(hn[0], y[-1, :1024])


def test_step_and_sequence_kernels_agree(ops):
    params, x, h0, c0 = workloads.lstm_inputs(111, 1024, 1024, 1, False, 50)
    y1, h1, c1 = run_plan(ops, params, x, h0, c0, True, 1, False, 1)
    y2, h2, c2 = run_plan(ops, params, x, h0, c0, True, 1, False, 2)
    assert maxabs(y1, y2.cpu()) <= 1e-3 and maxabs(c1, c2.cpu()) <= 1e-3


def test_switching_the_block_shape_on_one_plan_restarts_the_exchange(ops):
    """Modes 2 and 3 lay out a single layer's exchange entries differently; a plan that switches must not read what
    the other layout left behind."""
    params, x, h0, c0 = workloads.lstm_inputs(77, 64, 1024, 1, False, 23)
    want = oracle.torch_lstm(x, h0, c0, params, True, 1, False)
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 1, False, 23)
    outs = []
    for mode in (2, 3, 3, 2, 4, 0, 3, 4, 1, 2):
        plan.set_mode(mode)
        y, hn, cn = plan.forward(x.reshape(23, 64).to(DEV), h0.to(DEV), c0.to(DEV))
        plan.status()
        assert maxabs(y, want[0]) <= 2e-3 and maxabs(cn, want[2]) <= 2e-3
        outs.append((mode, y.cpu()))
    first = {}
    for mode, y in outs:          # one mode, one instruction stream: repeated runs agree to the bit
        assert torch.equal(first.setdefault(mode, y), y)


def test_sequence_kernels_issued_on_two_streams_do_not_starve_each_other(ops):
    """Each persistent launch needs the whole GPU's worth of resident blocks; launches on different streams are ordered
    one after the other by the library.  (Bounded all the same: a short spin limit turns a mistake into a time-out.)"""
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    cases = []
    for i, st in enumerate(streams):
        params, x, h0, c0 = workloads.lstm_inputs(200 + i, 64, 1024, 2, False, 40)
        plan = ops.LstmPlan([p.to(DEV) for p in params], True, 2, False, 40)
        plan.set_mode(2)
        plan.set_spin_limit(1 << 16)
        cases.append((plan, st, x.reshape(40, 64).to(DEV), h0.to(DEV), c0.to(DEV), oracle.torch_lstm(x, h0, c0, params, True, 2, False)))
    torch.cuda.synchronize()
    outs = []
    for _ in range(4):                       # alternate the streams without synchronising in between
        for plan, st, x, h0, c0, _want in cases:
            outs.append(plan.forward(x, h0, c0, stream=st))
    torch.cuda.synchronize()
    for plan, *_ in cases:
        plan.status()
    for k, (y, hn, cn) in enumerate(outs):
        want = cases[k % 2][5]
        assert maxabs(y, want[0]) <= 2e-3 and maxabs(cn, want[2]) <= 2e-3


def test_automatic_mode_without_measurement_follows_the_thresholds(ops):
    """What automatic mode does where it cannot measure (inside a graph capture, or with measuring switched off): bidirectional
    layers from 16 steps on, single unidirectional layers from 64 (16 at H <= 512) and unidirectional stacks from 32 (16 with
    three layers and more) run one recurrence per XCD: the same bits as mode 4, which sums in another order than mode 2."""
    for I, H, L, bidir, T, same_as in [(32, 256, 2, True, 40, 4), (32, 1024, 1, False, 70, 4), (32, 1024, 1, False, 20, 2),
                                        (32, 256, 1, False, 20, 4), (32, 256, 3, False, 40, 4), (32, 256, 1, True, 9, 2),
                                        (32, 256, 2, False, 20, 2), (32, 256, 2, False, 33, 4), (32, 256, 3, False, 12, 2)]:
        params, x, h0, c0 = workloads.lstm_inputs(800 + T, I, H, L, bidir, T)
        y0, _, c0n = run_plan(ops, params, x, h0, c0, True, L, bidir, 0, measure=False)
        ym, _, cmn = run_plan(ops, params, x, h0, c0, True, L, bidir, same_as)
        assert torch.equal(y0, ym) and torch.equal(c0n, cmn), (I, H, L, bidir, T)
        want = oracle.torch_lstm(x, h0, c0, params, True, L, bidir)
        assert maxabs(y0, want[0]) <= 2e-3 and maxabs(c0n, want[2]) <= 2e-3


def _call_us(plan, xd, hd, cd, reps=12):
    """Shortest of `reps` forwards, each timed with events on torch's current stream, in microseconds."""
    stream = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = None
    for _ in range(reps):
        e0.record(stream)
        plan.forward(xd, hd, cd)
        e1.record(stream)
        e1.synchronize()
        us = e0.elapsed_time(e1) * 1e3
        best = us if best is None else min(best, us)
    return best


@pytest.mark.parametrize("name,I,H,L,bidir,T", [
    ("rnnt_encoder", 240, 1024, 2, False, 200),                      # C3
    ("gnmt_l0", 1024, 1024, 1, True, 50), ("gnmt_l1", 2048, 1024, 1, False, 50), ("gnmt_l2", 1024, 1024, 1, False, 50),   # C4's calls
    ("prediction_net_T2", 320, 320, 2, False, 2), ("prediction_net_T5", 320, 320, 2, False, 5),
    ("prediction_net_T16", 320, 320, 2, False, 16), ("prediction_net_T64", 320, 320, 2, False, 64),
    ("wide", 256, 1536, 1, False, 40),
])
def test_automatic_mode_is_the_fastest_mode_the_plan_has(ops, name, I, H, L, bidir, T):
    """Automatic mode measures: the first eager forward of a plan in a range of sequence lengths runs the call under every
    kernel family that takes it and keeps the fastest (as the reference keeps the faster of its two libraries per layer on the
    first inference).  Afterwards a call in automatic mode is not slower than the same call under any forced mode by more than
    5 % (+ 4 us: two plans in the same mode differ by that much on the shortest calls, where the host's launches show in the
    events), and its result is the oracle's."""
    params, x, h0, c0 = workloads.lstm_inputs(900 + T, I, H, L, bidir, T)
    pd = [p.to(DEV) for p in params]
    xd, hd, cd = x.reshape(T, I).to(DEV), h0.to(DEV), c0.to(DEV)
    auto = ops.LstmPlan(pd, True, L, bidir, T)
    assert auto.measured_mode(T) == 0
    y, hn, cn = auto.forward(xd, hd, cd)            # measures
    auto.status()
    chosen = auto.measured_mode(T)
    assert chosen in (1, 2, 4)
    want = oracle.torch_lstm(x, h0, c0, params, True, L, bidir)
    assert maxabs(y, want[0]) <= LSTM_TOL and maxabs(hn, want[1]) <= LSTM_TOL and maxabs(cn, want[2]) <= LSTM_TOL
    y2, _, _ = auto.forward(xd, hd, cd)             # the same mode from now on: the same bits
    assert torch.equal(y, y2)
    forced = {}
    for mode in (1, 2, 4):
        plan = ops.LstmPlan(pd, True, L, bidir, T)
        try:
            plan.set_mode(mode)
        except ops.NNRuntimeException:
            continue                                 # this hidden size does not fit that kernel
        plan.forward(xd, hd, cd)
        forced[mode] = plan
    # (the plans take turns, three rounds: what the GPU ran just before shifts a call's time by several per cent)
    times, t_auto = {m: float("inf") for m in forced}, float("inf")
    for _ in range(3):
        t_auto = min(t_auto, _call_us(auto, xd, hd, cd, reps=6))
        for m, plan in forced.items():
            times[m] = min(times[m], _call_us(plan, xd, hd, cd, reps=6))
    print(f"{name}: automatic took mode {chosen}: {t_auto:.1f} us; forced {({m: round(t, 1) for m, t in times.items()})}", flush=True)
    assert t_auto <= 1.05 * min(times.values()) + 4.0, (name, chosen, t_auto, times)
    assert auto.fallbacks() == (0, True)


def test_per_xcd_kernel_finds_its_groups_on_any_queue(ops):
    """Workgroup b of a launch runs on XCD (b + o) % 8, with a start o that belongs to the hardware queue and moves over a
    process's life (this test is placed after ones that use several streams for that reason): the kernel takes its
    groups from the hardware's XCC_ID, so it is right on every stream, whatever o is there."""
    from pimaicompiler_amd import _lib as L
    lib = L.load()
    params, x, h0, c0 = workloads.lstm_inputs(611, 48, 512, 1, True, 24)
    want = oracle.torch_lstm(x, h0, c0, params, True, 1, True)
    pd = [p.to(DEV) for p in params]
    xd, hd, cd = x.reshape(24, 48).to(DEV), h0.to(DEV), c0.to(DEV)
    starts = []
    for st in [torch.cuda.current_stream()] + [torch.cuda.Stream() for _ in range(5)]:
        where = torch.full((64,), -1, dtype=torch.int32, device=DEV)
        torch.cuda.synchronize()
        assert lib.pimhip_probe_xcc_map(where.data_ptr(), 64, 512, st.cuda_stream) == 0
        st.synchronize()
        m = where.cpu().tolist()
        assert all(0 <= v < 8 for v in m) and all(m[b] == (m[0] + b) % 8 for b in range(64)), m     # a rotation
        starts.append(m[0])
        plan = ops.LstmPlan(pd, True, 1, True, 24)
        plan.set_mode(4)
        with torch.cuda.stream(st):
            y, hn, cn = plan.forward(xd, hd, cd, stream=st)
        st.synchronize()
        plan.status()
        assert maxabs(y, want[0]) <= 2e-3 and maxabs(cn, want[2]) <= 2e-3
    print("first workgroup's XCD per stream:", starts, flush=True)


# ---- the bounded wait ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("mode,layers,bidir,res", [(2, 1, False, None), (2, 3, False, None), (2, 1, True, None), (3, 1, False, None),
                                                   (4, 1, False, None), (4, 1, True, None), (4, 3, False, None), (4, 3, False, 1)])
def test_a_forward_whose_waits_give_up_still_gives_the_right_result(ops, mode, layers, bidir, res):
    """A wait that gives up costs time, not the result.  Forced from the host: with a spin limit of 0 every wait whose first
    look fails gives up at once (every kernel still ends by itself); the workgroups then compute their units of the
    recurrence by themselves, inside the same launch, and y, hn, cn of THAT forward are right.  So are the forwards after it
    (self-sufficient from their start until a forward outside a capture has re-initialised the exchange), the events are
    counted, and after the third the plan runs one launch per step.  Covers the all-CU kernel (one layer, a wavefront of
    three, the two directions of a layer, four units per block) and the per-XCD kernel (one layer, two directions, a
    pipeline of three layers whose recurrence and projection groups all give up, the same with residual sums)."""
    H, T = 256, 12
    params, x, h0, c0 = workloads.lstm_inputs(123, H if res is not None else 64, H, layers, bidir, T)
    g = torch.Generator().manual_seed(5)
    h0, c0 = (0.3 * torch.randn(h0.shape, generator=g)).half(), (0.3 * torch.randn(c0.shape, generator=g)).half()
    pd = [p.to(DEV) for p in params]
    plan = ops.LstmPlan(pd, True, layers, bidir, T)
    plan.set_mode(mode)
    plan.set_residual(res)
    if res is None:
        want = oracle.torch_lstm(x, h0, c0, params, True, layers, bidir)
    else:
        want = libtorch_residual_stack(params, x, h0, c0, True, layers, res)
    xd, hd, cd = x.reshape(T, -1).to(DEV), h0.to(DEV), c0.to(DEV)

    def check():
        y, hn, cn = plan.forward(xd, hd, cd)
        plan.status()
        assert maxabs(y, want[0]) <= 5e-3 and maxabs(hn, want[1]) <= 5e-3 and maxabs(cn, want[2]) <= 5e-3

    check()
    assert plan.fallbacks() == (0, True)
    plan.set_spin_limit(0)
    events = 0
    for _ in range(5):
        check()                               # right whether or not a wait gave up in it
        now, exchanging = plan.fallbacks()
        assert now >= events and exchanging == (now < 3)
        events = now
    assert events >= 3                        # some first look fails in every such forward
    plan.set_spin_limit(1 << 22)
    check()
    assert plan.fallbacks() == (events, False)   # one launch per step: nothing waits any more


def test_a_wait_that_gave_up_and_nobody_asked_about_costs_the_caller_nothing(ops):
    """aten_lstm1 never asks for the status: the forward whose wait gave up (forced from the host with a spin limit of 0)
    returns the right tensors all the same, and so does the next call, which re-initialises the exchange on its way."""
    params, x, h0, c0 = workloads.lstm_inputs(124, 64, 512, 2, False, 30)
    pd = [p.to(DEV) for p in params]
    xd, hx = x.to(DEV), (h0.to(DEV), c0.to(DEV))
    want = oracle.torch_lstm(x, h0, c0, params, True, 2, False)
    plan = ops.prepare_lstm(pd, True, 2, False, 30)
    plan.set_mode(2)
    plan.set_spin_limit(0)
    y, hn, cn = ops.aten_lstm1(xd, hx, pd, True, 2, 0.0, False, False, False)     # gives up inside the kernel, returns normally
    torch.cuda.synchronize()
    assert maxabs(y, want[0]) <= 5e-3 and maxabs(cn, want[2]) <= 5e-3
    plan.set_spin_limit(1 << 22)
    y, hn, cn = ops.aten_lstm1(xd, hx, pd, True, 2, 0.0, False, False, False)
    torch.cuda.synchronize()
    assert maxabs(y, want[0]) <= 5e-3 and maxabs(cn, want[2]) <= 5e-3
    assert plan.fallbacks() == (1, True)
    ops.invalidate_lstm_plans(pd)


def test_plan_cache_follows_weight_updates_and_is_bounded(ops):
    """A cached plan holds values derived from the weights (the summed biases, w_ih in matrix-core order): an in-place
    update seen by torch's version counter gives a new plan, invalidate_lstm_plans drops plans on request, and the cache
    never holds more than PLAN_CACHE_MAX plans."""
    from pimaicompiler_amd import ops as O
    params, x, h0, c0 = workloads.lstm_inputs(125, 64, 128, 1, False, 20)
    pd = [p.to(DEV) for p in params]
    xd, hx = x.to(DEV), (h0.to(DEV), c0.to(DEV))
    y0 = ops.aten_lstm1(xd, hx, pd, True, 1, 0.0, False, False, False)[0]
    assert maxabs(y0, oracle.torch_lstm(x, h0, c0, params, True, 1, False)[0]) <= 2e-3
    plan0 = O._plan_for(pd, True, 1, False, 20)
    # in-place update of w_ih (packed copy) and b_ih (summed bias): both live in the plan, not in the caller's tensors
    params2 = [p.clone() for p in params]
    params2[0] = (params2[0] * 0.5).half()
    params2[2] = (params2[2] + 0.25).half()
    pd[0].copy_(params2[0].to(DEV))
    pd[2].copy_(params2[2].to(DEV))
    y1 = ops.aten_lstm1(xd, hx, pd, True, 1, 0.0, False, False, False)[0]
    assert O._plan_for(pd, True, 1, False, 20) is not plan0
    assert maxabs(y1, oracle.torch_lstm(x, h0, c0, params2, True, 1, False)[0]) <= 2e-3
    assert ops.invalidate_lstm_plans(pd) == 1 and ops.invalidate_lstm_plans(pd) == 0
    # bound
    keep = []
    for i in range(O.PLAN_CACHE_MAX + 3):
        prm, *_ = workloads.lstm_inputs(300 + i, 8, 8, 1, False, 2)
        keep.append([p.to(DEV) for p in prm])
        O._plan_for(keep[-1], True, 1, False, 2)
    assert len(O._plan_cache) == O.PLAN_CACHE_MAX
    assert ops.invalidate_lstm_plans() == O.PLAN_CACHE_MAX


@pytest.mark.parametrize("mode", [2, 3, 4])
def test_persistent_kernel_survives_a_nan_input(ops, mode):
    """A NaN cannot carry the exchange's flag bit, so it is exchanged as 0; the cell state keeps it, and y is NaN from
    that step on exactly as in LibTorch.  No wait times out."""
    params, x, h0, c0 = workloads.lstm_inputs(5, 64, 512, 1, False, 12)
    x = x.clone()
    x[7, 0, 3] = float("nan")
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 1, False, 12)
    plan.set_mode(mode)
    y, hn, cn = plan.forward(x.reshape(12, 64).to(DEV), h0.to(DEV), c0.to(DEV))
    plan.status()
    want = oracle.torch_lstm(x, h0, c0, params, True, 1, False)[0]
    assert maxabs(y[:7], want[:7]) <= 2e-3
    assert bool(torch.isnan(want[7:]).all()) and bool(torch.isnan(y[7:]).all()) and bool(torch.isnan(cn).all())


@pytest.mark.parametrize("mode", [1, 2, 3, 4])
def test_saturated_gates_reach_their_limits_exactly(ops, mode):
    """Weights forty times the usual size drive the gates far into saturation (pre-activations of tens to hundreds): the
    sigmoid and tanh built on the hardware exp2 and reciprocal must give exactly 0, 1 and -1 there, as LibTorch's do, and
    nothing may turn into a NaN (exp2 overflows to inf, whose reciprocal is 0).  Two steps only: with such a gain a
    longer recurrence amplifies any last-bit difference into another trajectory, in LibTorch's own builds too."""
    T = 2
    params, x, h0, c0 = workloads.lstm_inputs(9, 64, 256, 2, False, T)
    params = [(p.float() * 40).half() for p in params]
    x = (x.float() * 8).half()
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 2, False, T)
    plan.set_mode(mode)
    y, hn, cn = plan.forward(x.reshape(T, 64).to(DEV), h0.to(DEV), c0.to(DEV))
    plan.status()
    want_y, want_hn, want_cn = oracle.torch_lstm(x, h0, c0, params, True, 2, False)
    assert not bool(torch.isnan(y).any()) and not bool(torch.isnan(cn).any())
    # it does saturate: most gates of the last step are 0 or 1 to within fp16, so c moved by a whole unit or stayed
    moved = (want_cn.float() - c0.float()).abs().reshape(-1)
    assert float(((moved - moved.round()).abs() < 2e-3).float().mean()) > 0.3 and float(moved.max()) > 0.9
    assert maxabs(y, want_y) <= 5e-3 and maxabs(hn, want_hn) <= 5e-3 and maxabs(cn, want_cn) <= 1e-2


def test_a_nan_travels_through_the_pipeline_of_layers(ops):
    """Mode 4 hands h from layer to layer through slots whose "not written yet" mark is the all-ones pattern, itself a NaN:
    a NaN h is stored there in its canonical form, so it arrives, and nobody waits for a slot that looks empty."""
    params, x, h0, c0 = workloads.lstm_inputs(6, 64, 256, 3, False, 20)
    x = x.clone()
    x[11, 0, 5] = float("nan")
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 3, False, 20)
    plan.set_mode(4)
    y, hn, cn = plan.forward(x.reshape(20, 64).to(DEV), h0.to(DEV), c0.to(DEV))
    plan.status()
    want = oracle.torch_lstm(x, h0, c0, params, True, 3, False)
    assert maxabs(y[:11], want[0][:11]) <= 2e-3
    assert bool(torch.isnan(want[0][11:]).all()) and bool(torch.isnan(y[11:]).all()) and bool(torch.isnan(cn).all())


# ---- input projection (the MFMA kernel) against fp32 torch on the host ---------------------------------------------
@pytest.mark.parametrize("T,K,N", [(1, 8, 16), (5, 24, 40), (16, 32, 16), (17, 40, 100), (50, 1024, 4096), (50, 2048, 4096),
                                   (200, 240, 4096), (200, 1024, 4096), (341, 240, 4096), (700, 64, 256),
                                   (200, 2048, 4096), (130, 4096, 256), (70, 2048, 520)])
def test_input_projection_matches_fp32_matmul(ops, T, K, N):
    g = torch.Generator().manual_seed(T + K + N)
    x = torch.randn(T, K, generator=g).half()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).half()
    b = torch.randn(N, generator=g)
    want = x.float() @ w.float().t() + b
    out = ops.input_projection(x.to(DEV), w.to(DEV), b.to(DEV))
    assert out.dtype == torch.float32 and list(out.shape) == [T, N]
    assert maxabs(out, want) <= 1e-4 * max(1.0, float(want.abs().max()))   # fp32 accumulation of exact fp16 products
    out = ops.input_projection(x.to(DEV), w.to(DEV))
    assert maxabs(out, want - b) <= 1e-4 * max(1.0, float(want.abs().max()))
    # the weight in fragment order (what a plan keeps for its batched layers): the same products, summed in the same
    # or (with eight wavefronts per block) another fixed order
    packed = ops.pack_projection_weight(w.to(DEV))
    tol = 1e-5 * max(1.0, float(want.abs().max()))
    assert maxabs(ops.input_projection_packed(x.to(DEV), packed, N), out.cpu()) <= tol
    got = ops.input_projection_packed(x.to(DEV), packed, N, b.to(DEV))
    assert maxabs(got, want) <= 1e-4 * max(1.0, float(want.abs().max()))
    assert torch.equal(got, ops.input_projection_packed(x.to(DEV), packed, N, b.to(DEV)))
