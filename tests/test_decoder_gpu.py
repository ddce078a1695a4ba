"""The fused decoder step (pimhip_decoder_step: every layer's seq_len-1 LSTM cell, the attention context, the residual
sums and the classifier in one launch) against LibTorch CPU running the same wiring operator by operator in fp16, and
against the product's own operator-by-operator path.

Tolerances: max abs error <= 5e-3 on layer outputs, h, c and logits (fp32 gates and accumulation here, fp16 between
the operators in LibTorch), <= 2e-3 on the context (a GEMV output)."""
import pytest
import torch

from pimaicompiler_amd import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
STATE_TOL = 5e-3
GEMV_TOL = 2e-3


def maxabs(a, b):
    return float((a.detach().float().cpu().reshape(-1) - b.detach().float().cpu().reshape(-1)).abs().max())


class Case:
    """Random weights and one step's inputs for a decoder wiring; everything on the CPU in fp16."""

    def __init__(self, seed, H, in0, L, first_ctx, first_res, vocab, src_len):
        g = torch.Generator().manual_seed(seed)
        self.H, self.in0, self.L, self.first_ctx, self.first_res, self.vocab = H, in0, L, first_ctx, first_res, vocab
        self.params = []
        for k in range(L):
            in_w = (in0 + (H if first_ctx else 0)) if k == 0 else 2 * H
            self.params += workloads.lstm_inputs(seed + 10 + k, in_w, H, 1, False, 1)[0]
        self.x = torch.randn(in0, generator=g).half()
        self.h = [(0.3 * torch.randn(H, generator=g)).half() for _ in range(L)]
        self.c = [(0.3 * torch.randn(H, generator=g)).half() for _ in range(L)]
        self.enc = torch.randn(src_len, H, generator=g).half()
        self.att = torch.softmax(torch.randn(src_len, generator=g), -1).half()
        self.Wc = (0.02 * torch.randn(vocab, H, generator=g)).half() if vocab else None
        self.bc = (0.01 * torch.randn(vocab, generator=g)).half() if vocab else None

    def cpu_step(self, x, h, c):
        """The wiring with LibTorch CPU operators in fp16: returns ctx, outs, hn, cn, logits."""
        H = self.H
        ctx = torch.matmul(self.att.view(1, -1).float(), self.enc.float()).half()     # bmm: fp32 accumulate, one rounding
        inp = x.view(1, -1)
        outs, hns, cns = [], [], []
        for k in range(self.L):
            takes = k > 0 or self.first_ctx
            full = torch.cat([inp, ctx], 1) if takes else inp
            y, hn, cn = torch.lstm(full.view(1, 1, -1), (h[k].view(1, 1, H), c[k].view(1, 1, H)), self.params[4 * k:4 * k + 4],
                                   True, 1, 0.0, False, False, False)
            y = y.view(1, H)
            out = y + inp if k >= self.first_res else y
            outs.append(out.view(-1))
            hns.append(hn.view(-1))
            cns.append(cn.view(-1))
            inp = out
        logits = torch.addmm(self.bc, inp, self.Wc.t()).view(-1) if self.vocab else None
        return ctx.view(-1), outs, hns, cns, logits

    def plan(self, P):
        cls = (self.Wc.to(DEV), self.bc.to(DEV)) if self.vocab else None
        return P.DecoderPlan([p.to(DEV) for p in self.params], True, self.L, first_takes_context=self.first_ctx,
                             first_residual_layer=self.first_res, classifier=cls)


def run_fused(P, case, plan, x, h, c, n_ctx_outs=1, use_ctx_in=None):
    H, L = case.H, case.L
    nanv = lambda n: torch.full((n,), float("nan"), dtype=torch.float16, device=DEV)  # noqa: E731
    hn, cn, outs = [nanv(H) for _ in range(L)], [nanv(H) for _ in range(L)], [nanv(H) for _ in range(L)]
    ctx_outs = [nanv(H) for _ in range(n_ctx_outs)]
    logits = nanv(case.vocab) if case.vocab else None
    step = plan.bind(x.to(DEV), [t.to(DEV) for t in h], [t.to(DEV) for t in c],
                     att=None if use_ctx_in is not None else case.att.to(DEV), enc=None if use_ctx_in is not None else case.enc.to(DEV),
                     ctx=use_ctx_in, hn=hn, cn=cn, outs=outs, ctx_outs=ctx_outs, logits=logits)
    step()
    plan.status()
    return ctx_outs, outs, hn, cn, logits


def check(case, got, want, ctx_given=False):
    ctx_outs, outs, hn, cn, logits = got
    wctx, wouts, whn, wcn, wlogits = want
    for cbuf in ctx_outs:
        assert maxabs(cbuf, wctx) <= (0.0 if ctx_given else GEMV_TOL)
    for k in range(case.L):
        assert maxabs(outs[k], wouts[k]) <= STATE_TOL, k
        assert maxabs(hn[k], whn[k]) <= STATE_TOL, k
        assert maxabs(cn[k], wcn[k]) <= STATE_TOL, k
    if case.vocab:
        assert not bool(torch.isnan(logits).any())
        assert maxabs(logits, wlogits) <= STATE_TOL


# (H, in0, L, first_ctx, first_res, vocab, src_len)
WIRINGS = [
    (1024, 1024, 4, False, 2, 4096, 50),     # the whole GNMT decoder step
    (1024, 1024, 3, True, 1, 32000, 50),     # layers 1..3 + classifier, layer 0 and the attention scores outside
    (1024, 1024, 1, False, 9, 0, 50),        # a single plain cell, no classifier
    (1024, 2048, 2, False, 1, 1001, 7),      # wide plain input, ragged vocabulary
    (72, 40, 2, False, 1, 1001, 7),          # 9 pieces per row: the two halves of a row differ in length
    (8, 8, 4, True, 0, 5, 1),                # the smallest shapes, residual around every layer
    (520, 520, 4, False, 2, 640, 13),
    (256, 64, 3, False, 2, 0, 3),            # no classifier: the last layer's exchange is left out
    (1024, 1024, 4, False, 2, 1000, 100),    # 65..128 source positions: both halves of a unit's wavefront pair hold one
    (512, 512, 2, True, 1, 0, 300),          # more than 128 source positions: the tail loop; the plan's buffer grows past 64
]


@pytest.mark.parametrize("H,in0,L,first_ctx,first_res,vocab,src_len", WIRINGS)
def test_fused_decoder_step_matches_libtorch_cpu(ops, H, in0, L, first_ctx, first_res, vocab, src_len):
    case = Case(1000 + H + L, H, in0, L, first_ctx, first_res, vocab, src_len)
    print(f"decoder step H={H} in0={in0} L={L} first_ctx={first_ctx} first_res={first_res} vocab={vocab} S={src_len}", flush=True)
    plan = case.plan(ops)
    want = case.cpu_step(case.x, case.h, case.c)
    check(case, run_fused(ops, case, plan, case.x, case.h, case.c, n_ctx_outs=3), want)
    # the context handed in instead of att and enc: the same bits everywhere downstream of it
    got = run_fused(ops, case, plan, case.x, case.h, case.c, n_ctx_outs=1, use_ctx_in=want[0].to(DEV))
    check(case, got, want, ctx_given=True)


def test_one_plan_serves_sentences_of_different_lengths(ops):
    """set_encoder once per sentence: a long sentence after a short one makes the projection buffer grow, a short one after
    it reuses the larger buffer with another row pitch; every step is checked against the CPU."""
    H, L = 512, 3
    base = Case(4242, H, H, L, False, 2, 777, 5)
    plan = base.plan(ops)
    for i, S in enumerate((5, 150, 64, 9, 129)):
        g = torch.Generator().manual_seed(900 + S)
        base.enc = torch.randn(S, H, generator=g).half()
        base.att = torch.softmax(torch.randn(S, generator=g), -1).half()
        print(f"sentence {i}: S={S}", flush=True)
        want = base.cpu_step(base.x, base.h, base.c)
        check(base, run_fused(ops, base, plan, base.x, base.h, base.c, n_ctx_outs=2), want)


def test_encoder_buffer_refilled_in_place_is_projected_again(ops):
    """The next sentence lands in the same buffer, written by one of the path's own kernels through its raw pointer (no
    tensor version changes): set_encoder must project again, not recognise the buffer."""
    H, L, S = 256, 2, 11
    case = Case(5151, H, H, L, True, 0, 0, S)
    plan = case.plan(ops)
    enc_buf = torch.zeros(S, H, dtype=torch.float16, device=DEV)
    zeros = torch.zeros(S, H, dtype=torch.float16, device=DEV)
    att = case.att.to(DEV)
    hn = [torch.zeros(H, dtype=torch.float16, device=DEV) for _ in range(L)]
    cn = [torch.zeros(H, dtype=torch.float16, device=DEV) for _ in range(L)]
    step = None
    for i in range(3):
        g = torch.Generator().manual_seed(7000 + i)
        case.enc = torch.randn(S, H, generator=g).half()
        version = enc_buf._version
        ops.aten_add(case.enc.to(DEV), zeros, out=enc_buf)
        assert enc_buf._version == version
        plan.set_encoder(enc_buf)
        if step is None:
            step = plan.bind(case.x.to(DEV), [t.to(DEV) for t in case.h], [t.to(DEV) for t in case.c], att=att, hn=hn, cn=cn)
        step()
        plan.status()
        _, _, whn, wcn, _ = case.cpu_step(case.x, case.h, case.c)
        for k in range(L):
            assert maxabs(hn[k], whn[k]) <= STATE_TOL and maxabs(cn[k], wcn[k]) <= STATE_TOL, (i, k)


def test_fused_decoder_steps_update_the_state_in_place(ops):
    """A decoder loop: hn / cn are the buffers h_prev / c_prev are read from, three steps in a row, against the CPU
    running the same three steps; then the same three steps again into separate buffers give the same bits."""
    case = Case(77, 1024, 1024, 4, False, 2, 2048, 20)
    plan = case.plan(ops)
    g = torch.Generator().manual_seed(5)
    xs = [torch.randn(1024, generator=g).half() for _ in range(3)]
    h, c = [t.clone() for t in case.h], [t.clone() for t in case.c]
    hd, cd = [t.to(DEV) for t in case.h], [t.to(DEV) for t in case.c]
    xd = torch.zeros(1024, dtype=torch.float16, device=DEV)
    logits = torch.zeros(case.vocab, dtype=torch.float16, device=DEV)
    step = plan.bind(xd, hd, cd, att=case.att.to(DEV), enc=case.enc.to(DEV), logits=logits)     # in place
    all_logits = []
    for x in xs:
        xd.copy_(x.to(DEV))
        step()
        _, _, h, c, wl = case.cpu_step(x, h, c)
        plan.status()
        for k in range(4):
            assert maxabs(hd[k], h[k]) <= STATE_TOL and maxabs(cd[k], c[k]) <= STATE_TOL
        assert maxabs(logits, wl) <= STATE_TOL
        all_logits.append(logits.clone())
    h2, c2 = [t.to(DEV) for t in case.h], [t.to(DEV) for t in case.c]
    for i, x in enumerate(xs):
        hn, cn = [torch.empty_like(t) for t in h2], [torch.empty_like(t) for t in c2]
        plan.bind(x.to(DEV), h2, c2, att=case.att.to(DEV), enc=case.enc.to(DEV), hn=hn, cn=cn, logits=logits)()
        torch.cuda.synchronize()
        assert torch.equal(logits, all_logits[i])
        h2, c2 = hn, cn
    for k in range(4):
        assert torch.equal(h2[k], hd[k]) and torch.equal(c2[k], cd[k])


def test_fused_decoder_step_agrees_with_the_operator_by_operator_path(ops):
    """Same weights and inputs through pimhip_lstm_forward x 4, bmm, add x 2 and the classifier GEMV (eight launches):
    the same mathematics with another order of the fp32 sums."""
    case = Case(31, 1024, 1024, 4, False, 2, 32000, 50)
    H = 1024
    plan = case.plan(ops)
    got = run_fused(ops, case, plan, case.x, case.h, case.c, n_ctx_outs=1)
    prm = [p.to(DEV) for p in case.params]
    cell = [ops.LstmPlan(prm[4 * k:4 * k + 4], True, 1, False, 1) for k in range(4)]
    ctx = ops.aten_bmm(case.att.view(1, 1, -1).to(DEV), case.enc.view(1, -1, H).to(DEV)).view(1, H)
    inp, hs, cs = case.x.view(1, H).to(DEV), [], []
    for k in range(4):
        full = torch.cat([inp, ctx], 1) if k > 0 else inp
        y, hn, cn = cell[k].forward(full, case.h[k].view(1, H).to(DEV), case.c[k].view(1, H).to(DEV))
        out = ops.aten_add(y, inp) if k >= 2 else y
        hs.append(hn)
        cs.append(cn)
        inp = out
        assert maxabs(got[1][k], out) <= 1e-3
    logits = ops.custom_aten_addmm("none", case.bc.to(DEV), case.Wc.to(DEV), inp.t())
    assert maxabs(got[0][0], ctx) <= 1e-3
    for k in range(4):
        assert maxabs(got[2][k], hs[k]) <= 1e-3 and maxabs(got[3][k], cs[k]) <= 1e-3
    assert maxabs(got[4], logits) <= 2e-3


def test_fused_decoder_step_replays_from_a_graph(ops):
    case = Case(41, 1024, 1024, 4, False, 2, 32000, 50)
    plan = case.plan(ops)
    g = torch.Generator().manual_seed(9)
    xs = [torch.randn(1024, generator=g).half().to(DEV) for _ in range(3)]
    xd = torch.zeros(1024, dtype=torch.float16, device=DEV)
    h0, c0 = [t.to(DEV) for t in case.h], [t.to(DEV) for t in case.c]
    hn, cn = [torch.empty_like(t) for t in h0], [torch.empty_like(t) for t in c0]
    logits = torch.zeros(case.vocab, dtype=torch.float16, device=DEV)
    step = plan.bind(xd, h0, c0, att=case.att.to(DEV), enc=case.enc.to(DEV), hn=hn, cn=cn, logits=logits)
    eager = []
    for x in xs:
        xd.copy_(x)
        step()
        torch.cuda.synchronize()
        eager.append([logits.clone()] + [t.clone() for t in hn + cn])
    plan.status()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step(torch.cuda.current_stream())
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    scratch = torch.randn(1 << 20, device=DEV)
    for rep in range(2):
        for x, want in zip(xs, eager):
            xd.copy_(x)
            for t in hn + cn + [logits]:
                t.fill_(float("nan"))
            graph.replay()
            scratch = scratch * 1.0001 + 1.0
            torch.cuda.synchronize()
            for got, w in zip([logits] + hn + cn, want):
                assert torch.equal(got, w)
    plan.status()


def _undisturbed_and_forced(ops, case, steps, in_place, n_ctx_outs=1, use_ctx_in=None):
    """The same steps twice on one plan's weights: with the default poll limit, and with a limit of 0 (every wait gives up
    at its first unsuccessful look, forced from the host; every kernel still runs to its end).  Returns both records."""
    H, L = case.H, case.L
    g = torch.Generator().manual_seed(1234)
    xs = [torch.randn(case.in0, generator=g).half().to(DEV) for _ in range(steps)]
    records = []
    for limit in (1 << 22, 0):
        plan = case.plan(ops)
        plan.set_spin_limit(limit)
        h, c = [t.to(DEV) for t in case.h], [t.to(DEV) for t in case.c]
        nanv = lambda n: torch.full((n,), float("nan"), dtype=torch.float16, device=DEV)  # noqa: E731
        hn, cn = (h, c) if in_place else ([nanv(H) for _ in range(L)], [nanv(H) for _ in range(L)])
        outs, ctx_outs = [nanv(H) for _ in range(L)], [nanv(H) for _ in range(n_ctx_outs)]
        logits = nanv(case.vocab) if case.vocab else None
        xd = torch.zeros(case.in0, dtype=torch.float16, device=DEV)
        ctx = use_ctx_in
        step = plan.bind(xd, h, c, att=None if ctx is not None else case.att.to(DEV), enc=None if ctx is not None else case.enc.to(DEV),
                         ctx=ctx, hn=hn, cn=cn, outs=outs, ctx_outs=ctx_outs, logits=logits)
        rec = []
        for x in xs:
            xd.copy_(x)
            step()
            torch.cuda.synchronize()
            rec.append([t.clone() for t in hn + cn + outs + ctx_outs + ([logits] if case.vocab else [])])
            if not in_place:
                for a, b in zip(h + c, hn + cn):
                    a.copy_(b)
        plan.status()
        events, patient = plan.fallbacks()
        records.append((rec, events, patient))
    return records


@pytest.mark.parametrize("H,in0,L,first_ctx,first_res,vocab,src_len,in_place", [
    (1024, 1024, 4, False, 2, 1024, 10, True),     # the GNMT step, the state updated in place
    (1024, 1024, 4, False, 2, 1024, 10, False),
    (256, 64, 3, False, 2, 0, 3, True),            # no classifier: the last layer exchanges nothing
    (72, 40, 2, False, 1, 1001, 7, True),          # the two halves of a row differ in length
    (512, 512, 2, True, 1, 0, 300, True),          # a first layer that takes the context, more than 128 source positions
    (1024, 2048, 2, False, 1, 1001, 7, True),      # a wide plain input: its columns in a loop
    (8, 8, 4, True, 0, 5, 1, True),
])
def test_a_wait_that_gives_up_costs_time_not_the_result(ops, H, in0, L, first_ctx, first_res, vocab, src_len, in_place):
    """Forced from the host: with a poll limit of 0 every wait gives up at its first unsuccessful look, the waiting
    wavefronts make the missing entries themselves and the blocks park their new state until the launch's last block stores
    it.  Three steps in a row (each starts from the state the one before left, in place or not) give, bit for bit, what the
    undisturbed steps give; the events are counted and after the third the plan keeps its waits short."""
    case = Case(51 + H, H, in0, L, first_ctx, first_res, vocab, src_len)
    print(f"decoder step forced give-up H={H} in0={in0} L={L} vocab={vocab} in_place={in_place}", flush=True)
    (calm, calm_events, calm_patient), (forced, forced_events, forced_patient) = _undisturbed_and_forced(ops, case, 3, in_place)
    assert calm_events == 0 and calm_patient
    # (a grid of a few blocks may find every entry there at its first look: then nothing gave up in that step)
    assert forced_events == 3 if H >= 256 else forced_events <= 3
    assert forced_patient == (forced_events < 3)
    for i, (a, b) in enumerate(zip(calm, forced)):
        for j, (ta, tb) in enumerate(zip(a, b)):
            assert torch.equal(ta.view(torch.int16), tb.view(torch.int16)), (i, j, maxabs(ta, tb))
    # and the undisturbed steps are the right ones
    want = case.cpu_step(case.x, case.h, case.c)  # (only the first step's state tolerance is checked against the CPU below)
    plan = case.plan(ops)
    got = run_fused(ops, case, plan, case.x, case.h, case.c)
    check(case, got, want)


def test_a_given_context_and_a_wait_that_gives_up(ops):
    case = Case(61, 520, 520, 4, False, 2, 640, 13)
    ctx = case.cpu_step(case.x, case.h, case.c)[0].to(DEV)
    (calm, _, _), (forced, events, _) = _undisturbed_and_forced(ops, case, 2, True, use_ctx_in=ctx)
    assert events == 2
    for a, b in zip(calm, forced):
        for ta, tb in zip(a, b):
            assert torch.equal(ta.view(torch.int16), tb.view(torch.int16))


def test_decoder_plan_refuses_what_the_kernel_does_not_take(ops):
    prm = [p.to(DEV) for p in workloads.lstm_inputs(3, 2056, 2056, 1, False, 1)[0]]
    with pytest.raises(ops.NNRuntimeException, match="hidden_size"):
        ops.DecoderPlan(prm, True, 1)
    prm = [p.to(DEV) for p in workloads.lstm_inputs(3, 64, 64, 1, False, 1)[0]]
    with pytest.raises(ops.NNRuntimeException):
        ops.DecoderPlan(prm * 5, True, 5)
    plan = ops.DecoderPlan(prm, True, 1, first_residual_layer=9)
    v = torch.zeros(64, dtype=torch.float16, device=DEV)
    with pytest.raises(ops.NNRuntimeException, match="in place"):
        plan.bind(v.clone(), [v], [v.clone()])()          # one layer, no classifier: no exchange to order the update behind
