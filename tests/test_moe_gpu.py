"""The one-launch mixture-of-experts feed-forward step (pimhip_moe_ffn_step) against LibTorch CPU, the committed golden
vectors of the MoE configuration and the three-GEMV path it replaces.  Tolerance: max abs error 2e-3 on logits, hidden
and y (fp16 storage, fp32 sums); the expert index must match exactly (the seeded tokens' top-2 logit gap is checked to
exceed the tolerance)."""
import importlib.util
import os

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3


def maxabs(a, b):
    return float((torch.as_tensor(a).float().cpu().reshape(-1) - torch.as_tensor(b).float().cpu().reshape(-1)).abs().max())


def make(seed, E, d_model, d_ff, biases, scale=0.05):
    g = torch.Generator().manual_seed(seed)
    Wr = (scale * torch.randn(E, d_model, generator=g)).half()
    br = (0.1 * torch.randn(E, generator=g)).half() if biases else None
    W1 = [(scale * torch.randn(d_ff, d_model, generator=g)).half() for _ in range(E)]
    W2 = [(scale * torch.randn(d_model, d_ff, generator=g)).half() for _ in range(E)]
    b1 = [(0.1 * torch.randn(d_ff, generator=g)).half() for _ in range(E)] if biases else None
    b2 = [(0.1 * torch.randn(d_model, generator=g)).half() for _ in range(E)] if biases else None
    return g, Wr, br, W1, b1, W2, b2


def libtorch_cpu(x, Wr, br, W1, b1, W2, b2, act, scale_by_prob):
    """The block as the reference's operators compute it, on LibTorch CPU in fp16 (one rounding per tensor)."""
    logits = torch.nn.functional.linear(x, Wr, br)
    top2 = torch.topk(logits.float().reshape(-1), min(2, logits.numel())).values
    gap = float(top2[0] - top2[1]) if logits.numel() > 1 else 1.0
    e = int(torch.argmax(logits))
    hidden = torch.nn.functional.linear(x, W1[e], b1[e] if b1 is not None else None)
    if act == "aten::relu":
        hidden = torch.relu(hidden)
    y = torch.nn.functional.linear(hidden, W2[e], b2[e] if b2 is not None else None)
    if scale_by_prob:
        y = (y.float() * torch.softmax(logits.float(), -1).reshape(-1)[e]).half()
    return logits, e, hidden, y, gap


def dev(ts):
    return [t.to(DEV) for t in ts] if ts is not None else None


def test_moe_configuration_matches_golden_vectors_and_libtorch(ops, golden):
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(__file__), "golden", "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    Wr, W1, W2, x = mg.moe_inputs()
    g = golden["moe"]
    plan = ops.MoePlan((Wr.to(DEV), None), dev(W1), dev(W2))
    y, logits, expert = plan.forward(x.to(DEV))
    plan.status()
    assert int(expert.item()) == int(g["expert"][0])
    assert maxabs(logits, g["logits"]) <= TOL and maxabs(y, g["y"]) <= TOL
    want = libtorch_cpu(x, Wr, None, W1, None, W2, None, "aten::relu", False)
    assert want[4] > TOL and int(expert.item()) == want[1] and maxabs(y, want[3]) <= TOL
    # the three-GEMV path on the same expert
    e = want[1]
    hidden = ops.aten_linear(x.to(DEV), W1[e].to(DEV), act_type="aten::relu")
    y3 = ops.aten_linear(hidden, W2[e].to(DEV))
    assert maxabs(y, y3) <= TOL


CASES = [
    # E, d_model, d_ff, biases, act, scale_by_prob
    (8, 768, 3072, True, "aten::relu", True),
    (3, 136, 520, True, "none", False),        # ragged: rows per block 3 / 1, most blocks of the second product idle
    (1, 8, 8, False, "aten::relu", False),      # one expert, one 16-byte piece per row
    (64, 1024, 4096, False, "aten::relu", True),
    (5, 2048, 4096, True, "none", False),       # the largest shapes the step takes
    (16, 2040, 4088, True, "aten::relu", False),
    (4, 264, 24, False, "none", False),         # fewer hidden values than blocks
]


@pytest.mark.parametrize("E,d_model,d_ff,biases,act,scale_by_prob", CASES)
def test_moe_step_matches_libtorch_cpu(ops, E, d_model, d_ff, biases, act, scale_by_prob):
    s = 0.5 / d_model ** 0.5
    g, Wr, br, W1, b1, W2, b2 = make(100 + E + d_model, E, d_model, d_ff, biases, scale=s)
    plan = ops.MoePlan((Wr.to(DEV), br.to(DEV) if br is not None else None), dev(W1), dev(W2), dev(b1), dev(b2), act_type=act,
                       scale_by_router_prob=scale_by_prob)
    y = torch.empty(d_model, dtype=torch.float16, device=DEV)
    logits = torch.empty(E, dtype=torch.float16, device=DEV)
    expert = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    xd = torch.empty(d_model, dtype=torch.float16, device=DEV)
    step = plan.bind(xd, y, logits, expert)
    seen, checked = set(), 0
    for rep in range(12):                     # consecutive steps alternate between the two sets of exchange slots
        x = torch.randn(1, d_model, generator=g).half()
        want_logits, e, hidden, want_y, gap = libtorch_cpu(x, Wr, br, W1, b1, W2, b2, act, scale_by_prob)
        xd.copy_(x.reshape(-1))
        step()
        plan.status()
        assert maxabs(logits, want_logits) <= TOL
        if gap <= 2 * TOL:
            continue                          # too close to call between two roundings of the same sums
        checked += 1
        assert int(expert.item()) == e
        assert maxabs(y, want_y) <= TOL, (rep, e)
        seen.add(e)
    assert checked >= 6 and (E < 3 or len(seen) >= 2)   # more than one expert was taken


def test_moe_step_without_optional_outputs_and_in_a_hip_graph(ops):
    E, d_model, d_ff = 8, 768, 3072
    g, Wr, br, W1, b1, W2, b2 = make(7, E, d_model, d_ff, True, scale=0.02)
    plan = ops.MoePlan((Wr.to(DEV), br.to(DEV)), dev(W1), dev(W2), dev(b1), dev(b2))
    xd = torch.empty(d_model, dtype=torch.float16, device=DEV)
    y = torch.empty(d_model, dtype=torch.float16, device=DEV)
    step = plan.bind(xd, y)
    xs = [torch.randn(d_model, generator=g).half() for _ in range(6)]
    wants = [libtorch_cpu(x.view(1, -1), Wr, br, W1, b1, W2, b2, "aten::relu", False) for x in xs]
    xd.copy_(xs[0])
    step()
    torch.cuda.synchronize()
    assert maxabs(y, wants[0][3]) <= TOL
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step(torch.cuda.current_stream().cuda_stream)
            step(torch.cuda.current_stream().cuda_stream)   # an even and an odd launch count in every replay
    torch.cuda.current_stream().wait_stream(side)
    for x, want in zip(xs[1:], wants[1:]):
        xd.copy_(x)
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert maxabs(y, want[3]) <= TOL
        step()                                               # eager work between the replays
        torch.cuda.synchronize()
        assert maxabs(y, want[3]) <= TOL
    plan.status()


def test_moe_step_nan_and_limits(ops):
    E, d_model, d_ff = 4, 256, 512
    g, Wr, br, W1, b1, W2, b2 = make(9, E, d_model, d_ff, False)
    W1[2][5, 3] = float("nan")                # a NaN hidden value travels through the exchange and reaches every output
    Wr[2] = 0
    Wr[2, 0] = 4.0
    x = torch.randn(1, d_model, generator=g).half()
    x[0, 0] = 3.0                             # expert 2 wins by a wide margin
    plan = ops.MoePlan((Wr.to(DEV), None), dev(W1), dev(W2), act_type="none")
    y, logits, expert = plan.forward(x.to(DEV))
    plan.status()
    assert int(expert.item()) == 2 and bool(torch.isnan(y).all())
    y, _, _ = plan.forward(x.to(DEV))         # the next launch starts from empty slots all the same
    plan.status()
    assert bool(torch.isnan(y).all())
    with pytest.raises(ops.NNRuntimeException):
        ops.MoePlan((torch.zeros(2, 4096, dtype=torch.float16, device=DEV), None),
                    [torch.zeros(64, 4096, dtype=torch.float16, device=DEV)] * 2, [torch.zeros(4096, 64, dtype=torch.float16, device=DEV)] * 2)
    with pytest.raises(ops.NNRuntimeException):
        plan.bind(torch.zeros(8, dtype=torch.float16, device=DEV), torch.zeros(d_model, dtype=torch.float16, device=DEV))


def test_moe_step_whose_waits_give_up_still_gives_the_right_result(ops):
    """A wait that gives up costs time, not the result: the workgroups that waited in vain compute the missing hidden values
    themselves, inside the same launch.  Forced from the host with a spin limit of 0 (a wait whose first look fails gives up
    at once; every kernel still ends by itself): the step that timed out is right, the steps after it are right (they run
    self-sufficient until a step outside a capture has put the exchange back in order), the events are counted, and after
    the third the plan stops exchanging for good."""
    E, d_model, d_ff = 8, 768, 3072
    g, Wr, br, W1, b1, W2, b2 = make(11, E, d_model, d_ff, True, scale=0.02)
    plan = ops.MoePlan((Wr.to(DEV), br.to(DEV)), dev(W1), dev(W2), dev(b1), dev(b2))
    xs = [torch.randn(1, d_model, generator=g).half() for _ in range(10)]
    wants = [libtorch_cpu(x, Wr, br, W1, b1, W2, b2, "aten::relu", False) for x in xs]

    def check(i):
        y, _, expert = plan.forward(xs[i].to(DEV))
        plan.status()
        assert wants[i][4] <= 2 * TOL or (int(expert.item()) == wants[i][1] and maxabs(y, wants[i][3]) <= TOL), i

    check(0)
    assert plan.fallbacks() == (0, True)
    plan.set_spin_limit(0)
    events = 0
    for i in range(1, 8):
        check(i)                              # right whether or not a wait gave up in it
        now, exchanging = plan.fallbacks()
        assert now >= events and exchanging == (now < 3)
        events = now
    assert events >= 3                        # with 192 workgroups some first look fails in nearly every step
    plan.set_spin_limit(1 << 22)
    check(8)
    check(9)
    assert plan.fallbacks() == (events, False)   # nothing waits any more: no further events


def test_resident_kernels_of_three_kinds_on_three_streams_take_turns(ops):
    """The mixture-of-experts step, the decoder step and a pipelined LSTM sequence all need their blocks resident together.
    Issued back to back on three streams without any synchronisation between them, the library orders them one after
    another: every result equals the one computed alone, and no wait gives up."""
    from pimaicompiler_amd import workloads
    E, d_model, d_ff, H, T = 8, 768, 3072, 512, 24
    g, Wr, br, W1, b1, W2, b2 = make(21, E, d_model, d_ff, False, scale=0.02)
    moe = ops.MoePlan((Wr.to(DEV), None), dev(W1), dev(W2))
    xm = torch.randn(d_model, generator=g).half().to(DEV)
    ym = torch.empty(d_model, dtype=torch.float16, device=DEV)
    moe_step = moe.bind(xm, ym)
    dparams = []
    for k in range(3):
        dparams += [p.to(DEV) for p in workloads.lstm_inputs(300 + k, H if k == 0 else 2 * H, H, 1, False, 1)[0]]
    dec = ops.DecoderPlan(dparams, True, 3)
    xd = torch.randn(H, generator=g).half().to(DEV)
    hs = [(0.3 * torch.randn(H, generator=g)).half().to(DEV) for _ in range(3)]
    cs = [(0.3 * torch.randn(H, generator=g)).half().to(DEV) for _ in range(3)]
    hn, cn = [torch.empty_like(t) for t in hs], [torch.empty_like(t) for t in cs]
    ctx = torch.randn(H, generator=g).half().to(DEV)
    dec_step = dec.bind(xd, hs, cs, ctx=ctx, hn=hn, cn=cn)
    lp, lx, lh0, lc0 = workloads.lstm_inputs(310, H, H, 3, False, T)
    lstm = ops.LstmPlan([p.to(DEV) for p in lp], True, 3, False, T)
    lstm.set_mode(4)
    lx, lh0, lc0 = lx.reshape(T, H).to(DEV), lh0.to(DEV), lc0.to(DEV)
    # alone
    moe_step()
    dec_step()
    want_l = [t.clone() for t in lstm.forward(lx, lh0, lc0)]
    torch.cuda.synchronize()
    want_m, want_h = ym.clone(), [t.clone() for t in hn]
    s1, s2, s3 = torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.Stream()
    for s in (s1, s2, s3):
        s.wait_stream(torch.cuda.current_stream())
    ym.zero_()
    for t in hn:
        t.zero_()
    outs = tuple(torch.zeros_like(t) for t in want_l)
    for _ in range(12):
        moe_step(s1.cuda_stream)
        dec_step(s2.cuda_stream)
        lstm.forward(lx, lh0, lc0, s3.cuda_stream, out=outs)
    torch.cuda.synchronize()
    moe.status()
    dec.status()
    lstm.status()
    assert torch.equal(ym, want_m)
    assert all(torch.equal(a, b) for a, b in zip(hn, want_h))
    assert all(torch.equal(a, b) for a, b in zip(outs, want_l))
