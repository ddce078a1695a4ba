"""Pins the CPU oracle (oracle/oracle.c) before anything is checked against it: LibTorch-CPU golden vectors,
closed forms, brute force in float64, and structural invariants chosen so that a dropped term, a wrong gate
order, a transposed operand or a wrong rounding fails at least one of them."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle
from pimaicompiler_amd import workloads

GEMV_TOL = 2e-3   # max abs error allowed on GEMV outputs
LSTM_TOL = 5e-3   # max abs error allowed on y / h / c


def maxabs(a, b):
    return float(np.max(np.abs(np.asarray(a, dtype=np.float64) - np.asarray(b, dtype=np.float64))))


# ---- fp16 conversion ---------------------------------------------------------------------------------------
def test_half_to_double_is_exact_for_every_bit_pattern():
    lib = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float64)
    for b in range(0, 65536, 7):
        got = lib.oracle_half_to_double(int(b))
        assert (math.isnan(got) and math.isnan(want[b])) or got == want[b], b


def test_double_to_half_rounds_to_nearest_even():
    lib = oracle.lib()
    rng = np.random.default_rng(1)
    vals = np.concatenate([rng.normal(size=2000), rng.normal(size=500) * 1e-5, rng.normal(size=500) * 3e4,
                           [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                            2.0 ** -14, 2.0 ** -14 - 2.0 ** -25]])
    # exact ties between neighbouring halves
    h = rng.integers(0, 0x7bff, size=500).astype(np.uint16)
    lo, hi = h.view(np.float16).astype(np.float64), (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    vals = np.concatenate([vals, (lo + hi) / 2])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    for v, w in zip(vals, want):
        assert lib.oracle_double_to_half(float(v)) == int(w), v


# ---- GEMV: LibTorch golden vectors ---------------------------------------------------------------------------
def test_gemv_mv_c1_matches_libtorch_addmm(golden):
    W, x, b = workloads.gemv_inputs(1001, 1024, 1024)
    y = oracle.gemv_mv(W.numpy(), x.numpy().reshape(-1), b.numpy())
    g = golden["gemv"]["c1_1024x1024_y"]
    assert maxabs(y, g) <= GEMV_TOL
    # both round an fp32-or-better sum once: all but a few near-tie elements agree to the bit
    assert np.mean(y.view(np.uint16) == g.view(np.uint16)) > 0.97


@pytest.mark.parametrize("name,seed,n,k", [("c2_4096x4096", 2001, 4096, 4096), ("c2_16384x4096", 2002, 16384, 4096),
                                          ("c2_4096x16384", 2003, 4096, 16384), ("c2_32000x1024", 2004, 32000, 1024)])
def test_gemv_mv_sweep_samples_match_libtorch(golden, name, seed, n, k):
    W, x, b = workloads.gemv_inputs(seed, n, k)
    idx = golden["gemv"][name + "_idx"]
    y = oracle.gemv_mv(W.numpy()[idx], x.numpy().reshape(-1), b.numpy()[idx])
    assert maxabs(y, golden["gemv"][name + "_y_samples"]) <= GEMV_TOL


def test_moe_step_matches_libtorch(golden):
    import importlib.util, os
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(__file__), "golden", "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    Wr, W1, W2, x = mg.moe_inputs()
    g = golden["moe"]
    xv = x.numpy().reshape(-1)
    logits = oracle.gemv_mv(Wr.numpy(), xv)
    assert maxabs(logits, g["logits"]) <= GEMV_TOL
    e = int(np.argmax(logits.astype(np.float32)))
    assert e == int(g["expert"][0])
    hidden = oracle.gemv_mv(W1[e].numpy(), xv, relu=True)
    assert maxabs(hidden, g["hidden"]) <= GEMV_TOL
    y = oracle.gemv_mv(W2[e].numpy(), hidden)
    assert maxabs(y, g["y"]) <= GEMV_TOL


# ---- GEMV: closed forms and invariants ---------------------------------------------------------------------
def _rand_half(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float16)


def test_gemv_zero_input_returns_bias_exactly():
    rng = np.random.default_rng(2)
    W, b = _rand_half(rng, 37, 50), _rand_half(rng, 37)
    y = oracle.gemv_mv(W, np.zeros(50, np.float16), b)
    assert np.array_equal(y.view(np.uint16), b.view(np.uint16))
    y = oracle.gemv_vm(np.zeros(37, np.float16), W, _rand_half(rng, 50)[:50])
    assert y.shape == (50,)


def test_gemv_one_hot_input_selects_a_column_plus_bias():
    rng = np.random.default_rng(3)
    W, b = _rand_half(rng, 40, 24), _rand_half(rng, 40)
    for j in (0, 7, 23):
        x = np.zeros(24, np.float16)
        x[j] = 1.0
        want = (W[:, j].astype(np.float64) + b.astype(np.float64)).astype(np.float16)  # one fp16 rounding
        assert np.array_equal(oracle.gemv_mv(W, x, b).view(np.uint16), want.view(np.uint16))


def test_gemv_identity_weight_returns_x_plus_bias():
    rng = np.random.default_rng(4)
    x, b = _rand_half(rng, 33), _rand_half(rng, 33)
    want = (x.astype(np.float64) + b.astype(np.float64)).astype(np.float16)
    assert np.array_equal(oracle.gemv_mv(np.eye(33, dtype=np.float16), x, b).view(np.uint16), want.view(np.uint16))
    assert np.array_equal(oracle.gemv_vm(x, np.eye(33, dtype=np.float16), b).view(np.uint16), want.view(np.uint16))


def test_gemv_vm_equals_mv_on_the_transpose_bit_for_bit():
    rng = np.random.default_rng(5)
    W, x, b = _rand_half(rng, 61, 45, scale=0.1), _rand_half(rng, 45), _rand_half(rng, 61)
    mv = oracle.gemv_mv(W, x, b, relu=True)
    vm = oracle.gemv_vm(x, np.ascontiguousarray(W.T), b, relu=True)
    assert np.array_equal(mv.view(np.uint16), vm.view(np.uint16))


def test_gemv_brute_force_float64_and_relu_after_bias():
    rng = np.random.default_rng(6)
    W, x, b = _rand_half(rng, 19, 300, scale=0.1), _rand_half(rng, 300), _rand_half(rng, 19)
    exact = W.astype(np.float64) @ x.astype(np.float64) + b.astype(np.float64)
    assert np.array_equal(oracle.gemv_mv(W, x, b).view(np.uint16), exact.astype(np.float16).view(np.uint16))
    relu = np.maximum(exact, 0.0).astype(np.float16)
    got = oracle.gemv_mv(W, x, b, relu=True)
    assert np.array_equal(got.view(np.uint16), relu.view(np.uint16))
    assert (exact < 0).any() and (exact > 0).any()
    # a dropped bias would change the result
    assert not np.array_equal(oracle.gemv_mv(W, x).view(np.uint16), got.view(np.uint16))


def test_dot_brute_force():
    rng = np.random.default_rng(7)
    a, b = _rand_half(rng, 1024, scale=0.3), _rand_half(rng, 1024, scale=0.3)
    want = np.float16(np.dot(a.astype(np.float64), b.astype(np.float64)))
    assert oracle.dot(a, b)[0] == want
    assert oracle.dot(a[:0], b[:0])[0] == 0


def test_add_is_the_fp16_sum_rounded_once_in_both_broadcast_forms():
    """oracle.add against LibTorch CPU's fp16 add (the op executeAtenAdd's fallback calls) and against the exact sum in
    float64 rounded once by numpy: element-wise, and one row added to every row.  Includes ties, a sum that overflows and
    cancellation to zero; a row taken for a column, a second rounding or a dropped operand changes a bit somewhere."""
    import torch
    rng = np.random.default_rng(9)
    a = _rand_half(rng, 7 * 40, scale=3.0).reshape(7, 40)
    b = _rand_half(rng, 7 * 40, scale=3.0).reshape(7, 40)
    a[0, :4] = np.array([1.0, 2048.0, 65504.0, 0.333251953125], dtype=np.float16)
    b[0, :4] = np.array([2.0 ** -11, 1.0, 65504.0, -0.333251953125], dtype=np.float16)   # tie to even, tie, overflow, zero
    row = _rand_half(rng, 40, scale=3.0)
    for other in (b, row):
        got = oracle.add(a, other)
        with np.errstate(over="ignore"):
            want_np = (a.astype(np.float64) + other.astype(np.float64)).astype(np.float16)
        want_torch = (torch.from_numpy(a) + torch.from_numpy(other)).numpy()
        assert got.shape == a.shape
        assert np.array_equal(got.view(np.uint16), want_np.view(np.uint16))
        assert np.array_equal(got.view(np.uint16), want_torch.view(np.uint16))
    assert not np.array_equal(oracle.add(a, row).view(np.uint16), oracle.add(a, b).view(np.uint16))
    assert np.isinf(oracle.add(a, b)[0, 2]) and oracle.add(a, b)[0, 3] == 0


def test_gemv_f32_port_matches_numpy():
    rng = np.random.default_rng(8)
    W, x, b = rng.standard_normal((9, 40)).astype(np.float32), rng.standard_normal(40).astype(np.float32), rng.standard_normal(9).astype(np.float32)
    assert np.allclose(oracle.gemv_mv_f32(W, x, b), W @ x + b, atol=1e-5)


# ---- LSTM: LibTorch golden vectors ------------------------------------------------------------------------
TINY = [f"L{L}_D{D}_b{b}" for L in (1, 2) for D in (1, 2) for b in (1, 0)]


def _tiny_case(golden, key):
    g = golden["lstm_tiny"]
    L, D, has_b = int(key[1]), int(key[4]), int(key[7])
    n = L * D * (4 if has_b else 2)
    params = [g[f"{key}_p{i}"] for i in range(n)]
    return g, L, D, has_b, params


@pytest.mark.parametrize("key", TINY)
def test_lstm_tiny_matches_libtorch(golden, key):
    g, L, D, has_b, params = _tiny_case(golden, key)
    x = g[key + "_x"]
    y, hn, cn = oracle.lstm(x.reshape(x.shape[0], -1), g[key + "_h0"], g[key + "_c0"], params, has_b, L, D == 2)
    assert maxabs(y, g[key + "_y"].reshape(y.shape)) <= 2e-3
    assert maxabs(hn, g[key + "_hn"].reshape(hn.shape)) <= 2e-3
    assert maxabs(cn, g[key + "_cn"].reshape(cn.shape)) <= 2e-3


def test_lstm_c3_final_state_matches_libtorch(golden):
    params, x, h0, c0 = workloads.lstm_inputs(3001, 240, 1024, 2, False, 200)
    y, hn, cn = oracle.lstm(x.numpy().reshape(200, 240), h0.numpy(), c0.numpy(), [p.numpy() for p in params], True, 2, False)
    g = golden["lstm_large"]
    assert maxabs(hn, g["c3_hn"].reshape(hn.shape)) <= LSTM_TOL
    assert maxabs(cn, g["c3_cn"].reshape(cn.shape)) <= LSTM_TOL
    assert maxabs(y[::25, ::16], g["c3_y_samples"]) <= LSTM_TOL


# ---- LSTM: closed forms and structure ---------------------------------------------------------------------
def _np_lstm_params(rng, I, H, L, D, has_b, scale=0.3):
    params = []
    for l in range(L):
        in_w = I if l == 0 else D * H
        for _ in range(D):
            params += [_rand_half(rng, 4 * H, in_w, scale=scale), _rand_half(rng, 4 * H, H, scale=scale)]
            if has_b:
                params += [_rand_half(rng, 4 * H, scale=scale), _rand_half(rng, 4 * H, scale=scale)]
    return params


def test_lstm_zero_weights_closed_form_in_the_biases():
    """With W = 0 the gates are constants: c_t = sig(f) c_{t-1} + sig(i) tanh(g), h_t = sig(o) tanh(c_t).
    Distinct bias values per gate make a wrong gate order fail."""
    H, I, T = 8, 8, 6
    b_ih = np.concatenate([np.full(H, 0.5), np.full(H, -1.0), np.full(H, 2.0), np.full(H, 0.25)]).astype(np.float16)
    b_hh = np.concatenate([np.full(H, 0.25), np.full(H, 0.5), np.full(H, -0.5), np.full(H, 1.0)]).astype(np.float16)
    params = [np.zeros((4 * H, I), np.float16), np.zeros((4 * H, H), np.float16), b_ih, b_hh]
    rng = np.random.default_rng(9)
    x = _rand_half(rng, T, I)
    c0 = np.full((1, H), 0.75, np.float16)
    y, hn, cn = oracle.lstm(x, np.zeros((1, H), np.float16), c0, params, True, 1, False)
    sig = lambda v: 1 / (1 + math.exp(-v))
    i, f, g, o = sig(0.75), sig(-0.5), math.tanh(1.5), sig(1.25)
    c = 0.75
    for t in range(T):
        c = f * c + i * g
        assert abs(float(y[t, 0]) - o * math.tanh(c)) <= 6e-4  # one fp16 rounding of a value below 1
    assert abs(float(cn[0, 0]) - c) <= 6e-4


def test_lstm_single_step_is_gemv_plus_pointwise():
    rng = np.random.default_rng(10)
    I, H = 24, 16
    params = _np_lstm_params(rng, I, H, 1, 1, True)
    x, h0, c0 = _rand_half(rng, 1, I), _rand_half(rng, 1, H, scale=0.5), _rand_half(rng, 1, H, scale=0.5)
    y, hn, cn = oracle.lstm(x, h0, c0, params, True, 1, False)
    f64 = lambda a: a.astype(np.float64)
    a = f64(params[0]) @ f64(x[0]) + f64(params[1]) @ f64(h0[0]) + f64(params[2]) + f64(params[3])
    sig = lambda v: 1 / (1 + np.exp(-v))
    c = sig(a[H:2 * H]) * f64(c0[0]) + sig(a[:H]) * np.tanh(a[2 * H:3 * H])
    h = sig(a[3 * H:]) * np.tanh(c)
    assert np.array_equal(hn[0].view(np.uint16), h.astype(np.float16).view(np.uint16))
    assert np.array_equal(cn[0].view(np.uint16), c.astype(np.float16).view(np.uint16))
    assert np.array_equal(y[0].view(np.uint16), hn[0].view(np.uint16))


def test_lstm_bidirectional_is_forward_plus_time_reversed():
    rng = np.random.default_rng(11)
    I, H, T = 8, 8, 7
    params = _np_lstm_params(rng, I, H, 1, 2, True)
    x = _rand_half(rng, T, I)
    h0, c0 = _rand_half(rng, 2, H, scale=0.5), _rand_half(rng, 2, H, scale=0.5)
    y, hn, cn = oracle.lstm(x, h0, c0, params, True, 1, True)
    yf, hf, cf = oracle.lstm(x, h0[:1], c0[:1], params[:4], True, 1, False)
    yb, hb, cb = oracle.lstm(x[::-1], h0[1:], c0[1:], params[4:], True, 1, False)
    assert np.array_equal(y[:, :H], yf) and np.array_equal(y[:, H:], yb[::-1])
    assert np.array_equal(hn[0], hf[0]) and np.array_equal(hn[1], hb[0])
    assert np.array_equal(cn[0], cf[0]) and np.array_equal(cn[1], cb[0])
    # hn of the backward direction is the state after consuming t = 0, i.e. y[0, H:]
    assert np.array_equal(hn[1], y[0, H:]) and np.array_equal(hn[0], y[T - 1, :H])


def test_lstm_two_layers_compose():
    rng = np.random.default_rng(12)
    I, H, T = 8, 16, 5
    params = _np_lstm_params(rng, I, H, 2, 2, False)
    x = _rand_half(rng, T, I)
    h0, c0 = _rand_half(rng, 4, H, scale=0.5), _rand_half(rng, 4, H, scale=0.5)
    y, hn, cn = oracle.lstm(x, h0, c0, params, False, 2, True)
    y0, hn0, cn0 = oracle.lstm(x, h0[:2], c0[:2], params[:4], False, 1, True)
    y1, hn1, cn1 = oracle.lstm(y0, h0[2:], c0[2:], params[4:], False, 1, True)
    assert np.array_equal(y, y1)
    assert np.array_equal(hn, np.concatenate([hn0, hn1])) and np.array_equal(cn, np.concatenate([cn0, cn1]))


def test_lstm_pack_layout_and_round_trip():
    """model_builder.cpp:226-319: weights of all layers first, then biases; per layer w_ih (fwd, bwd) then w_hh
    (fwd, bwd); gate chunks in order (0, 1, 3, 2)."""
    rng = np.random.default_rng(13)
    for L, D, has_b in [(1, 1, True), (2, 2, True), (2, 1, False), (1, 2, False)]:
        params = _np_lstm_params(rng, 8, 4, L, D, has_b)
        buf = oracle.lstm_pack_miopen(params, has_b, L, D == 2)
        per = 4 if has_b else 2
        reorder = lambda p: np.concatenate([np.split(p, 4, axis=0)[i] for i in (0, 1, 3, 2)]).reshape(-1)
        want = []
        for l in range(L):
            cell = lambda d, k: params[(l * D + d) * per + k]
            for k in (0, 1):
                for d in range(D):
                    want.append(reorder(cell(d, k)))
        if has_b:
            for l in range(L):
                cell = lambda d, k: params[(l * D + d) * per + k]
                for k in (2, 3):
                    for d in range(D):
                        want.append(reorder(cell(d, k)))
        assert np.array_equal(buf, np.concatenate(want))
        back = oracle.lstm_unpack_miopen(buf, [p.shape for p in params], has_b, L, D == 2)
        for a, b in zip(params, back):
            assert np.array_equal(a, b)


# ---- shape logic -----------------------------------------------------------------------------------------------
def _oracle_broadcast(s1, s2):
    rc, o1, o2 = oracle.gemm_broadcast(s1, s2)
    if rc == 1:
        return "abort", None, None
    if rc == 2:
        return "out_of_range", None, None
    return ("ok" if len(o1) == 4 and len(o2) == 4 else "short"), o1, o2


def _oracle_type(o1, o2):
    from shape_cases import TYPE_NAMES
    return TYPE_NAMES[oracle.get_gemm_type(o1, o2)]


def test_shape_logic_matches_the_hand_traced_table():
    """tests/golden/shape_logic_cases.json: traced by hand through utils.cpp:293-396, one or more cases per branch,
    the reference's unit-test shapes (custom_op_ut.cpp:27-28, 49-50, 76-77, 113-114) among them."""
    from shape_cases import check_hand_traced, hand_traced_cases
    check_hand_traced(_oracle_broadcast, _oracle_type)
    lines = " ".join(c["lines"] for c in hand_traced_cases())
    for branch in ("299-310", "311-315", "316-317", "320-323", "324-326", "327-329", "331-333", "335-339", "340-341",
                   "345-346", "347-348", "351-352", "353-354", "356-361", "362-365", "383-384", "385-386", "387-388",
                   "389-391", "392-394"):
        assert branch in lines, branch


def test_shape_logic_agrees_with_the_meaning_of_the_product():
    """Independent of the source's structure: class, element counts and padded shapes follow from the real matrix
    product wherever torch.matmul accepts the pair; the exceptions are the ones the source's lines produce."""
    from shape_cases import check_matmul_semantics
    n_checked, n_as_product, exceptions = check_matmul_semantics(_oracle_broadcast, _oracle_type)
    assert n_checked > 600 and n_as_product > 550
    assert exceptions["square_behind_rank4_row"] == 12 and exceptions["rank1_rank1"] == 3 and exceptions["rank1_leading_match"] == 12
