"""The one-launch RNN-transducer decoding step (pimhip_rnnt_step) against LibTorch CPU on seeded inputs, against the
launches it replaces (pimhip_lstm_forward at seq_len 1, pimhip_execute_gemv_cat2, pimhip_execute_gemv), and over a greedy
decoding loop whose encoder frames come from the reference's own RNNT feature file.  Tolerances: max abs error 5e-3 on
h / c (as for every LSTM here), 2e-3 on the joint network's hidden vector and logits given the same g (fp16 storage, fp32
sums), 1e-3 between the states and those of pimhip_lstm_forward at seq_len 1 (both fp16 roundings of nearly the same fp32
value)."""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL_STATE, TOL_JOINT = 5e-3, 2e-3


def maxabs(a, b):
    return float((torch.as_tensor(a).float().cpu().reshape(-1) - torch.as_tensor(b).float().cpu().reshape(-1)).abs().max())


def make(seed, L, I, H, F, J, V, biases=True):
    """Prediction network parameters ~ U(-1/sqrt(H), 1/sqrt(H)) in LibTorch order, joint network 0.05 randn."""
    g = torch.Generator().manual_seed(seed)
    k = 1.0 / H ** 0.5
    params = []
    for l in range(L):
        in_w = I if l == 0 else H
        shapes = [(4 * H, in_w), (4 * H, H)] + ([(4 * H,), (4 * H,)] if biases else [])
        params += [((2 * torch.rand(*s, generator=g) - 1) * k).half() for s in shapes]
    w1 = (0.05 * torch.randn(J, F + H, generator=g)).half()
    b1 = (0.1 * torch.randn(J, generator=g)).half() if biases else None
    w2 = (0.05 * torch.randn(V, J, generator=g)).half()
    b2 = (0.1 * torch.randn(V, generator=g)).half() if biases else None
    return g, params, (w1, b1, w2, b2)


def libtorch_cpu_step(params, joint, L, x, h, c, f, biases=True):
    """One step as the reference's operators compute it on LibTorch CPU in fp16: at::lstm at seq_len 1, then the joint
    network as two dependent addmm over f and g (RemoveCatForAddmm), relu, addmm."""
    w1, b1, w2, b2 = joint
    H, F = h.size(-1), f.numel()
    y, hn, cn = torch.lstm(x.reshape(1, 1, -1), (h.reshape(L, 1, H), c.reshape(L, 1, H)), params, biases, L, 0.0, False, False, False)
    g_vec = y.reshape(1, H)
    first = torch.nn.functional.linear(f.reshape(1, F), w1[:, :F], b1)
    hidden = torch.relu(first + torch.nn.functional.linear(g_vec, w1[:, F:]))
    logits = torch.nn.functional.linear(hidden, w2, b2)
    return hn.reshape(L, H), cn.reshape(L, H), hidden.reshape(-1), logits.reshape(-1)


def joint_cpu(joint, f, g_vec):
    w1, b1, w2, b2 = joint
    hidden = torch.relu(torch.nn.functional.linear(torch.cat([f.reshape(1, -1), g_vec.reshape(1, -1)], 1).float(), w1.float(),
                                                   b1.float() if b1 is not None else None)).half()
    return hidden.reshape(-1), torch.nn.functional.linear(hidden.float(), w2.float(), b2.float() if b2 is not None else None).half().reshape(-1)


def dev(ts):
    return [t.to(DEV) if t is not None else None for t in ts]


CASES = [
    # L, I, H, F, J, V, biases
    (2, 320, 320, 1024, 512, 29, True),      # the RNNT shapes
    (1, 64, 32, 128, 64, 5, True),
    (2, 1024, 512, 2048, 256, 130, False),
    (4, 72, 136, 200, 1024, 8, True),
    (3, 320, 320, 1024, 512, 29, False),
]


@pytest.mark.parametrize("L,I,H,F,J,V,biases", CASES)
def test_step_against_libtorch_cpu_and_the_launches_it_replaces(ops, L, I, H, F, J, V, biases):
    g, params, joint = make(100 + L + H, L, I, H, F, J, V, biases)
    x = torch.randn(I, generator=g).half()
    h = (0.5 * torch.randn(L, H, generator=g)).clamp(-1, 1).half()
    c = torch.randn(L, H, generator=g).half()
    f = torch.randn(F, generator=g).half()
    want_hn, want_cn, want_hidden, want_logits = libtorch_cpu_step(params, joint, L, x, h, c, f, biases)

    plan = ops.RnntPlan(dev(params), biases, L, tuple(dev(joint)))
    hn, cn = torch.empty(L, H, dtype=torch.float16, device=DEV), torch.empty(L, H, dtype=torch.float16, device=DEV)
    logits, hidden = torch.empty(V, dtype=torch.float16, device=DEV), torch.empty(J, dtype=torch.float16, device=DEV)
    xd, hd, cd, fd = x.to(DEV), h.to(DEV), c.to(DEV), f.to(DEV)
    plan.bind(xd, hd, cd, fd, hn, cn, logits, hidden)()
    torch.cuda.synchronize()
    assert plan.fallbacks() == (0, True)
    assert maxabs(hn, want_hn) <= TOL_STATE and maxabs(cn, want_cn) <= TOL_STATE
    # the joint network given the g this step produced (its own rounding only)
    hid_ref, log_ref = joint_cpu(joint, f, hn[L - 1].cpu())
    assert maxabs(hidden, hid_ref) <= TOL_JOINT and maxabs(logits, log_ref) <= TOL_JOINT
    assert maxabs(logits, want_logits) <= 4 * TOL_STATE and maxabs(hidden, want_hidden) <= 4 * TOL_STATE

    # the launches it replaces
    lplan = ops.LstmPlan(dev(params), biases, L, False, 1)
    _, hn2, cn2 = lplan.forward(xd.reshape(1, I), hd, cd)
    lplan.status()
    assert maxabs(hn2, hn) <= 1e-3 and maxabs(cn2, cn) <= 2e-3
    w1, b1, w2, b2 = dev(joint)
    hid2 = ops.aten_linear_cat2(fd.reshape(1, F), hn[L - 1].reshape(1, H), w1, b1, "aten::relu")
    log2 = ops.aten_linear(hid2, w2, b2)
    assert maxabs(hidden, hid2) <= 1e-3 and maxabs(logits, log2) <= TOL_JOINT

    # the step after a blank: only the frame changes, the prediction network does not run
    f2 = torch.randn(F, generator=g).half()
    logits2 = torch.empty(V, dtype=torch.float16, device=DEV)
    plan.bind(None, hn, None, f2.to(DEV), None, None, logits2, run_prediction=False)()
    torch.cuda.synchronize()
    _, log_ref2 = joint_cpu(joint, f2, hn[L - 1].cpu())
    assert maxabs(logits2, log_ref2) <= TOL_JOINT
    # ... and a full step again after it (the exchange's two sets keep alternating through steps of both kinds)
    hn3, cn3 = torch.empty_like(hn), torch.empty_like(cn)
    plan.bind(xd, hn, cn, fd, hn3, cn3, logits)()
    torch.cuda.synchronize()
    _, hn4, cn4 = lplan.forward(xd.reshape(1, I), hn, cn)
    assert maxabs(hn4, hn3) <= 1e-3 and maxabs(cn4, cn3) <= 2e-3
    assert plan.fallbacks() == (0, True)


def test_greedy_decoding_loop_over_frames_of_the_rnnt_feature_file(ops):
    """A greedy transducer decoding loop with the RNNT shapes: the encoder (2 layers, I = 240, H = 1024) runs over the first
    frames of the reference's feature file, then per frame the joint network decides between blank (next frame, joint
    network alone) and a symbol (prediction network advances on that symbol's embedding).  The same loop runs on LibTorch
    CPU in fp16; at every step where the CPU's top-2 logit gap exceeds the tolerance the choice must be the same, and the
    logits agree within tolerance along the whole path (the paths are kept together by following the CPU's choice)."""
    from pimaicompiler_amd import io, workloads
    T, L, I, H, F, J, V, blank = 40, 2, 320, 320, 1024, 512, 29, 28
    feat = io.load_tensor(os.path.join(os.path.dirname(__file__), "golden", "rnnt_feature_341x1x240_f16.bin"), [341, 1, 240], "FLOAT16")
    enc_params, _, eh0, ec0 = workloads.lstm_inputs(3001, 240, F, 2, False, T)
    frames = feat[:T]
    enc_cpu, _, _ = torch.lstm(frames, (eh0, ec0), enc_params, True, 2, 0.0, False, False, False)
    eplan = ops.LstmPlan(dev(enc_params), True, 2, False, T)
    enc_gpu, _, _ = eplan.forward(frames.reshape(T, 240).to(DEV), eh0.to(DEV), ec0.to(DEV))
    eplan.status()
    assert maxabs(enc_gpu, enc_cpu) <= TOL_STATE

    g, params, joint = make(777, L, I, H, F, J, V, True)
    embedding = (0.5 * torch.randn(V, I, generator=g)).half()
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    emb_d = embedding.to(DEV)
    state = [torch.zeros(L, H, dtype=torch.float16, device=DEV) for _ in range(4)]  # (h, c) twice: swapped per symbol
    h_c, c_c = torch.zeros(L, H, dtype=torch.float16), torch.zeros(L, H, dtype=torch.float16)
    logits = torch.empty(V, dtype=torch.float16, device=DEV)
    cur, symbols, compared, decided = 0, 0, 0, 0
    last = blank - 1                       # start-of-sequence symbol
    t, run_prediction = 0, True
    while t < T and symbols < 60:
        h_d, c_d, hn_d, cn_d = state[2 * cur], state[2 * cur + 1], state[2 * (1 - cur)], state[2 * (1 - cur) + 1]
        f_d = enc_gpu[t].reshape(F).contiguous()
        if run_prediction:
            plan.bind(emb_d[last].contiguous(), h_d, c_d, f_d, hn_d, cn_d, logits)()
            hn_c, cn_c, _, want = libtorch_cpu_step(params, joint, L, embedding[last], h_c, c_c, enc_cpu[t].reshape(F))
            h_c, c_c = hn_c, cn_c
            cur = 1 - cur
            h_d, c_d = hn_d, cn_d
            assert maxabs(h_d, h_c) <= TOL_STATE and maxabs(c_d, c_c) <= 2 * TOL_STATE, (t, symbols)
        else:
            plan.bind(None, h_d, None, f_d, None, None, logits, run_prediction=False)()
            _, want = joint_cpu(joint, enc_cpu[t].reshape(F), h_c[L - 1])
        torch.cuda.synchronize()
        assert maxabs(logits, want) <= 4 * TOL_STATE
        top2 = torch.topk(want.float(), 2)
        compared += 1
        if float(top2.values[0] - top2.values[1]) > 8 * TOL_STATE:
            assert int(torch.argmax(logits.float())) == int(top2.indices[0])
            decided += 1
        choice = int(top2.indices[0])
        # (a real model emits mostly blanks; with random weights the loop is made to by taking every third step's symbol)
        if choice == blank or compared % 3 != 0:
            t, run_prediction = t + 1, False
        else:
            last, symbols, run_prediction = choice, symbols + 1, True
    assert symbols >= 5 and decided >= 10
    assert plan.fallbacks() == (0, True)


def test_steps_recorded_into_a_graph_replay_like_eager_steps(ops):
    """Two steps per graph (a full step and the step after a blank), replayed several times with eager work in between: every
    replay gives what the eager steps give."""
    L, I, H, F, J, V = 2, 320, 320, 1024, 512, 29
    g, params, joint = make(31, L, I, H, F, J, V, True)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    x, f, f2 = (torch.randn(n, generator=g).half().to(DEV) for n in (I, F, F))
    h, c = torch.zeros(L, H, dtype=torch.float16, device=DEV), torch.zeros(L, H, dtype=torch.float16, device=DEV)
    hn, cn = torch.empty_like(h), torch.empty_like(c)
    la, lb = torch.empty(V, dtype=torch.float16, device=DEV), torch.empty(V, dtype=torch.float16, device=DEV)
    full = plan.bind(x, h, c, f, hn, cn, la)
    after_blank = plan.bind(None, hn, None, f2, None, None, lb, run_prediction=False)
    full()
    after_blank()
    torch.cuda.synchronize()
    want = [t.clone() for t in (hn, cn, la, lb)]
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            full(torch.cuda.current_stream().cuda_stream)
            after_blank(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(4):
        for t in (hn, cn, la, lb):
            t.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        for got, w in zip((hn, cn, la, lb), want):
            assert torch.equal(got, w), rep
        full()                                  # eager steps between the replays
        torch.cuda.synchronize()
    assert plan.fallbacks() == (0, True)


def test_a_step_whose_waits_give_up_still_gives_the_right_result(ops):
    """A wait that gives up costs time, not the result.  Forced from the host with a spin limit of 0 (a wait whose first look
    fails gives up at once; every kernel still ends by itself): every step is bit for bit what it is without the event, the
    events are counted, and after the third the plan stops exchanging for good."""
    L, I, H, F, J, V = 2, 320, 320, 1024, 512, 29
    g, params, joint = make(41, L, I, H, F, J, V, True)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    steps = []
    for i in range(10):
        steps.append(tuple(t.to(DEV) for t in (torch.randn(I, generator=g).half(), (0.3 * torch.randn(L, H, generator=g)).half(),
                                               torch.randn(L, H, generator=g).half(), torch.randn(F, generator=g).half())))

    def run(i, run_prediction=True):
        x, h, c, f = steps[i]
        hn, cn = torch.empty_like(h), torch.empty_like(c)
        logits, hidden = torch.empty(V, dtype=torch.float16, device=DEV), torch.empty(J, dtype=torch.float16, device=DEV)
        if run_prediction:
            plan.bind(x, h, c, f, hn, cn, logits, hidden)()
        else:
            plan.bind(None, h, None, f, None, None, logits, hidden, run_prediction=False)()
        torch.cuda.synchronize()
        return (hn, cn, logits, hidden) if run_prediction else (logits, hidden)

    wants = [run(i) for i in range(10)]
    wants_blank = [run(i, False) for i in range(10)]
    assert plan.fallbacks() == (0, True)
    plan.set_spin_limit(0)
    events = 0
    def same(got, want, what):
        for k, (a, b) in enumerate(zip(got, want)):
            bad = (a != b).reshape(-1).nonzero().reshape(-1)
            assert bad.numel() == 0, (what, k, bad.numel(), bad[:8].tolist(), maxabs(a, b))

    for i in range(8):
        same(run(i), wants[i], i)                 # right, to the bit, whether or not a wait gave up in it
        same(run(i, False), wants_blank[i], (i, "after a blank"))
        now, exchanging = plan.fallbacks()
        assert now >= events and exchanging == (now < 3)
        events = now
    assert events >= 3
    plan.set_spin_limit(1 << 22)
    for i in (8, 9):
        same(run(i), wants[i], i)
    assert plan.fallbacks() == (events, False)    # nothing waits any more: no further events


def test_arguments_the_step_refuses(ops):
    L, I, H, F, J, V = 2, 320, 320, 1024, 512, 29
    g, params, joint = make(51, L, I, H, F, J, V, True)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    x, f = torch.zeros(I, dtype=torch.float16, device=DEV), torch.zeros(F, dtype=torch.float16, device=DEV)
    h, c = torch.zeros(L, H, dtype=torch.float16, device=DEV), torch.zeros(L, H, dtype=torch.float16, device=DEV)
    logits = torch.empty(V, dtype=torch.float16, device=DEV)
    with pytest.raises(ops.NNRuntimeException, match="overlap"):
        plan.bind(x, h, c, f, h, c, logits)()                       # in-place state
    with pytest.raises(ops.NNRuntimeException, match="elements"):
        plan.bind(x, h, c, f[:512], torch.empty_like(h), torch.empty_like(c), logits)
    with pytest.raises(ops.NNRuntimeException, match="non-null"):
        plan.bind(None, h, c, f, torch.empty_like(h), torch.empty_like(c), logits)()
    # shapes beyond one workgroup per eight units / rows: the separate launches serve them
    g2, params2, joint2 = make(52, 2, 1024, 1024, 1024, 512, 29, False)
    with pytest.raises(ops.NNRuntimeException, match="workgroups"):
        ops.RnntPlan(dev(params2), False, 2, tuple(dev(joint2)))
