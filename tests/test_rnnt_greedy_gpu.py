"""The one-launch greedy decoding loop (pimhip_rnnt_greedy_decode) against the same loop driven from the host through
pimhip_rnnt_step (which tests/test_rnnt_gpu.py holds against LibTorch CPU): symbols, counts and final state bit for bit, as
both sum in the same order and round the state to fp16 between runs of the prediction network.  Integer outputs and fp16
bits: no tolerance.  One test holds the loop against LibTorch CPU directly, on the decisions that the last bits of a logit
cannot turn."""
import pytest
import torch

from test_rnnt_gpu import DEV, dev, joint_cpu, libtorch_cpu_step, make

pytestmark = pytest.mark.gpu


def model(seed, L, I, H, F, J, V, T, blank, blank_bias, biases=True, w2_scale=0.1):
    """A transducer with random weights whose joint network prefers `blank` by `blank_bias` (a real model emits mostly
    blanks; with plain random weights every frame would emit symbols up to the per-frame limit)."""
    g, params, joint = make(seed, L, I, H, F, J, V, biases)
    w1, b1, w2, b2 = joint
    w2 = (w2.float() * w2_scale).half()
    if b2 is not None:
        b2 = b2.clone()
        b2[blank] += blank_bias
    enc = torch.randn(T, F, generator=g).half().to(DEV)
    embedding = torch.randn(V, I, generator=g).half().to(DEV)
    x0 = torch.zeros(I, dtype=torch.float16, device=DEV)
    return params, (w1, b1, w2, b2), enc, embedding, x0


def argmax_like_torch(logits):
    """torch.argmax of the fp16 logits: the first maximum, a NaN counting as the largest."""
    nan = torch.isnan(logits)
    if bool(nan.any()):
        return int(nan.float().argmax())
    return int(torch.argmax(logits.float()))


def loop_driven_from_the_host(plan, enc, embedding, x0, blank, per_frame, max_symbols, h0=None, c0=None, run_prediction_first=True):
    """The loop of pimhip_rnnt_greedy_decode, one pimhip_rnnt_step and one read of the logits per iteration."""
    L, H = plan.num_layers, plan.hidden
    h = torch.zeros(L, H, dtype=torch.float16, device=DEV) if h0 is None else h0.clone()
    c = torch.zeros(L, H, dtype=torch.float16, device=DEV) if c0 is None else c0.clone()
    t, symbols, in_frame, run_prediction, label, steps = 0, [], 0, run_prediction_first, -1, 0
    while t < enc.size(0) and len(symbols) < max_symbols:
        if run_prediction:
            logits, h, c = plan.forward(x0 if label < 0 else embedding[label], h, c, enc[t], True)
        else:
            logits, _, _ = plan.forward(None, h, None, enc[t], False)
        k = argmax_like_torch(logits)
        steps += 1
        if k == blank:
            t, in_frame, run_prediction = t + 1, 0, False
        else:
            symbols.append(k)
            label, in_frame, run_prediction = k, in_frame + 1, True
            if in_frame >= per_frame:
                t, in_frame = t + 1, 0
    return symbols, t, steps, h, c, run_prediction, label


def check(got, want):
    symbols, result, hn, cn = got
    torch.cuda.synchronize()
    r = result.cpu().tolist()
    w_symbols, w_t, w_steps, w_h, w_c, w_pending, w_label = want
    assert r[0] == len(w_symbols) and symbols[: r[0]].cpu().tolist() == w_symbols
    assert (r[1], r[2], r[4], r[5]) == (w_t, w_steps, int(w_pending), w_label)
    assert torch.equal(hn, w_h) and torch.equal(cn, w_c)
    return r


CASES = [
    # L, I, H, F, J, V, T, blank, per_frame, max_symbols, blank_bias, biases
    (2, 320, 320, 1024, 512, 29, 120, 28, 30, None, 0.62, True),     # the RNNT shapes, mostly blanks
    (2, 320, 320, 1024, 512, 29, 60, 28, 7, None, 0.7, True),
    (2, 320, 320, 1024, 512, 29, 40, 28, 30, None, 0.3, True),       # mostly symbols: frames end at the per-frame limit
    (2, 320, 320, 1024, 512, 29, 50, 28, 2, 37, 0.4, True),          # ends at max_symbols
    (1, 64, 32, 128, 64, 5, 12, 0, 3, None, 0.3, True),
    (2, 136, 344, 1000, 504, 64, 30, 1, 4, None, 0.3, True),         # widths that are no multiples of 64, the most symbols
    (3, 72, 136, 200, 1024, 8, 40, 3, 4, None, 0.2, False),
    (4, 1024, 256, 2048, 512, 64, 25, 63, 5, None, 0.5, True),       # widest x and f, embedding rows read from memory
    (1, 64, 32, 128, 64, 5, 0, 0, 3, None, 0.3, True),               # no frames
    (1, 64, 32, 128, 64, 100, 30, 99, 3, None, 0.3, True),           # more symbols than a look at four steps takes
    (2, 64, 64, 256, 128, 300, 25, 7, 4, None, 0.3, True),           # ... and an embedding too large for LDS
]


@pytest.mark.parametrize("L,I,H,F,J,V,T,blank,per_frame,max_symbols,blank_bias,biases", CASES)
def test_one_launch_gives_what_the_loop_driven_from_the_host_gives(ops, L, I, H, F, J, V, T, blank, per_frame, max_symbols, blank_bias, biases):
    params, joint, enc, embedding, x0 = model(900 + L + H + T, L, I, H, F, J, V, T, blank, blank_bias, biases)
    plan = ops.RnntPlan(dev(params), biases, L, tuple(dev(joint)))
    cap = T * per_frame if max_symbols is None else max_symbols
    want = loop_driven_from_the_host(plan, enc, embedding, x0, blank, per_frame, cap)
    r = check(plan.greedy_decode(enc, embedding, x0, blank, per_frame, max_symbols), want)
    assert r[3] == 0 and plan.fallbacks() == (0, True)
    # again on the same plan (the exchange is refilled by every call), now with a state to start from
    h0 = (0.3 * torch.randn(L, H)).half().to(DEV)
    c0 = torch.randn(L, H).half().to(DEV)
    want = loop_driven_from_the_host(plan, enc, embedding, x0, blank, per_frame, cap, h0, c0)
    check(plan.greedy_decode(enc, embedding, x0, blank, per_frame, max_symbols, h0=h0, c0=c0), want)
    assert plan.fallbacks() == (0, True)


def test_the_mix_of_blanks_and_symbols_is_a_real_one(ops):
    """The cases here are meant to mix the two kinds of step: many frames pass with a blank, some emit symbols."""
    L, I, H, F, J, V, T, blank = 2, 320, 320, 1024, 512, 29, 60, 28
    params, joint, enc, embedding, x0 = model(6161, L, I, H, F, J, V, T, blank, 0.75)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    _, result, _, _ = plan.greedy_decode(enc, embedding, x0, blank)
    torch.cuda.synchronize()
    n, frames, steps = result.cpu().tolist()[:3]
    assert frames == T and n >= 30 and steps >= n + T // 2


def test_decoding_goes_on_where_a_chunk_of_frames_ended(ops):
    """Frames arrive in chunks: the second call starts from the first one's state, with the last symbol still to be fed to
    the prediction network or not as result[4] says.  Together they give what one call over all frames gives."""
    L, I, H, F, J, V, T, blank = 2, 320, 320, 1024, 512, 29, 90, 28
    params, joint, enc, embedding, x0 = model(4242, L, I, H, F, J, V, T, blank, 0.6)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    whole = plan.greedy_decode(enc, embedding, x0, blank, 1000)
    torch.cuda.synchronize()
    want_n = int(whole[1][0])
    want = whole[0][:want_n].cpu().tolist()
    for cut in (1, 37, 60):
        s1, r1, h1, c1 = plan.greedy_decode(enc[:cut], embedding, x0, blank, 1000)
        torch.cuda.synchronize()
        r1 = r1.cpu().tolist()
        assert r1[1] == cut
        x_next = x0 if r1[5] < 0 else embedding[r1[5]]
        s2, r2, h2, c2 = plan.greedy_decode(enc[cut:], embedding, x_next, blank, 1000, h0=h1, c0=c1, run_prediction_first=bool(r1[4]))
        torch.cuda.synchronize()
        r2 = r2.cpu().tolist()
        assert s1[: r1[0]].cpu().tolist() + s2[: r2[0]].cpu().tolist() == want, cut
        assert torch.equal(h2, whole[2]) and torch.equal(c2, whole[3])
    assert plan.fallbacks() == (0, True)


def test_a_loop_whose_waits_give_up_still_gives_the_right_result(ops):
    """Forced from the host with a spin limit of 0: the workgroups leave the loop at their first wait and one of them
    decodes the utterance by itself, inside the same launch, to the same bits.  The events count for the plan; after the
    third every launch is that one workgroup from the start."""
    L, I, H, F, J, V, T, blank = 2, 320, 320, 1024, 512, 29, 30, 28
    params, joint, enc, embedding, x0 = model(5151, L, I, H, F, J, V, T, blank, 0.55)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    want = loop_driven_from_the_host(plan, enc, embedding, x0, blank, 30, T * 30)
    assert len(want[0]) >= 10
    plan.set_spin_limit(0)
    for i in range(4):
        r = check(plan.greedy_decode(enc, embedding, x0, blank), want)
        assert r[3] == 1, i
    events, exchanging = plan.fallbacks()
    assert events >= 3 and not exchanging
    plan.set_spin_limit(1 << 22)
    r = check(plan.greedy_decode(enc, embedding, x0, blank), want)
    assert r[3] == 1 and plan.fallbacks() == (events, False)
    # a fresh plan is a team again
    plan2 = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    r = check(plan2.greedy_decode(enc, embedding, x0, blank), want)
    assert r[3] == 0 and plan2.fallbacks() == (0, True)


def test_a_workgroup_decoding_alone_handles_many_symbols_too(ops):
    L, I, H, F, J, V, T, blank = 1, 64, 32, 128, 64, 100, 20, 99
    params, joint, enc, embedding, x0 = model(5252, L, I, H, F, J, V, T, blank, 0.05)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    want = loop_driven_from_the_host(plan, enc, embedding, x0, blank, 3, T * 3)
    assert len(want[0]) >= 3
    plan.set_spin_limit(0)
    r = check(plan.greedy_decode(enc, embedding, x0, blank, 3), want)
    assert r[3] == 1


def test_the_loop_recorded_into_a_graph_replays_like_the_eager_call(ops):
    L, I, H, F, J, V, T, blank = 2, 320, 320, 1024, 512, 29, 60, 28
    params, joint, enc, embedding, x0 = model(6161, L, I, H, F, J, V, T, blank, 0.75)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    want = loop_driven_from_the_host(plan, enc, embedding, x0, blank, 30, T * 30)
    from pimaicompiler_amd import _lib
    from pimaicompiler_amd.ops import _check
    lib = _lib.load()
    symbols = torch.empty(T * 30, dtype=torch.int32, device=DEV)
    result = torch.zeros(8, dtype=torch.int32, device=DEV)
    hn = torch.empty(L, H, dtype=torch.float16, device=DEV)
    cn = torch.empty_like(hn)

    def call(stream):
        _check(lib.pimhip_rnnt_greedy_decode(plan._handle, enc.data_ptr(), T, embedding.data_ptr(), V, x0.data_ptr(), None, None, 1,
                                                 blank, 30, T * 30, symbols.data_ptr(), result.data_ptr(), hn.data_ptr(), cn.data_ptr(),
                                                 stream))

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(4):
        for t in (symbols, result, hn, cn):
            t.fill_(7)
        graph.replay()
        check((symbols, result, hn, cn), want)
        check(plan.greedy_decode(enc, embedding, x0, blank), want)      # eager calls between the replays
    assert plan.fallbacks() == (0, True)


def test_the_loop_against_libtorch_cpu_where_the_decisions_are_clear(ops):
    """The same loop on LibTorch CPU in fp16, operator by operator as the reference runs it (at::lstm at seq_len 1, the
    joint network's products, argmax).  Its logits differ from the GPU's in the last bits, so only decisions whose two best
    logits lie further apart than the tolerance can be held against it: the symbols must agree up to the first step where
    they do not (seeded: that step, if any, is always the same one), and that has to be a good way into the utterance."""
    L, I, H, F, J, V, T, blank, per_frame = 2, 320, 320, 1024, 512, 29, 40, 28, 3
    params, joint, enc, embedding, x0 = model(9191, L, I, H, F, J, V, T, blank, 1.5, w2_scale=1.0)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    symbols, result, hn, cn = plan.greedy_decode(enc, embedding, x0, blank, per_frame)
    torch.cuda.synchronize()
    got = symbols[: int(result[0])].cpu().tolist()
    enc_c, emb_c = enc.cpu(), embedding.cpu()
    h, c = torch.zeros(L, H, dtype=torch.float16), torch.zeros(L, H, dtype=torch.float16)
    t, want, in_frame, run_prediction, label, steps, clear = 0, [], 0, True, -1, 0, True
    while t < T and clear:
        if run_prediction:
            h, c, _, logits = libtorch_cpu_step(params, joint, L, x0.cpu() if label < 0 else emb_c[label], h, c, enc_c[t])
        else:
            _, logits = joint_cpu(joint, enc_c[t], h[L - 1])
        top2 = torch.topk(logits.float(), 2)
        if float(top2.values[0] - top2.values[1]) <= 2e-2:
            clear = False                       # a decision the last bits could turn: nothing behind it can be compared
            break
        k = int(top2.indices[0])
        steps += 1
        if k == blank:
            t, in_frame, run_prediction = t + 1, 0, False
        else:
            want.append(k)
            label, in_frame, run_prediction = k, in_frame + 1, True
            if in_frame >= per_frame:
                t, in_frame = t + 1, 0
    assert steps >= 40 and len(want) >= 10 and len(set(want)) >= 3      # a real mix, a good way in
    assert got[: len(want)] == want
    if clear:
        assert len(got) == len(want) and int(result[1]) == T
        assert float((hn.cpu().float() - h.float()).abs().max()) <= 5e-3


def test_an_utterance_from_the_rnnt_feature_file_end_to_end(ops):
    """The reference's own RNNT input (examples/runtime/resource/rnnt/inputs/feature.bin, 341 x 1 x 240 fp16, a fixture
    here) through an encoder of the RNNT shape (two LSTM layers, 240 -> 1024, one pipeline launch) and then the whole
    greedy loop in one launch: two launches of this library's per utterance where the reference interprets some thousand
    operators.  The loop's symbols and state against the loop driven from the host on the same encoder output."""
    import os
    from pimaicompiler_amd import io, workloads
    T, L, I, H, F, J, V, blank = 341, 2, 320, 320, 1024, 512, 29, 28
    feat = io.load_tensor(os.path.join(os.path.dirname(__file__), "golden", "rnnt_feature_341x1x240_f16.bin"), [341, 1, 240], "FLOAT16")
    enc_params, _, eh0, ec0 = workloads.lstm_inputs(3001, 240, F, 2, False, T)
    eplan = ops.LstmPlan(dev(enc_params), True, 2, False, T)
    enc, _, _ = eplan.forward(feat.reshape(T, 240).to(DEV), eh0.to(DEV), ec0.to(DEV))
    eplan.status()
    params, joint, _, embedding, x0 = model(777, L, I, H, F, J, V, 1, blank, 0.12)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    enc = enc.reshape(T, F).contiguous()
    want = loop_driven_from_the_host(plan, enc, embedding, x0, blank, 30, T * 30)
    r = check(plan.greedy_decode(enc, embedding, x0, blank), want)
    assert r[1] == T and r[3] == 0 and plan.fallbacks() == (0, True)
    assert 5 <= r[0] and r[2] >= T          # some frames emit, every frame is consumed


def test_ties_nans_and_an_empty_budget_are_decided_as_torch_argmax_decides_them(ops):
    """Equal logits: the first index wins.  A NaN among them: it counts as the largest.  No symbols allowed: nothing runs."""
    L, I, H, F, J, V, T = 1, 64, 32, 128, 64, 5, 6
    g, params, joint = make(8181, L, I, H, F, J, V, True)
    w1, b1, w2, b2 = joint
    flat = (w1, b1, torch.zeros_like(w2), torch.full_like(b2, 0.25))        # every logit 0.25
    enc = torch.randn(T, F, generator=g).half().to(DEV)
    embedding = torch.randn(V, I, generator=g).half().to(DEV)
    x0 = torch.zeros(I, dtype=torch.float16, device=DEV)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(flat)))
    for blank, per_frame in ((0, 3), (1, 3), (4, 2)):
        want = loop_driven_from_the_host(plan, enc, embedding, x0, blank, per_frame, T * per_frame)
        r = check(plan.greedy_decode(enc, embedding, x0, blank, per_frame), want)
        assert r[0] == (0 if blank == 0 else T * per_frame)                  # index 0 every time: a blank, or a symbol
    # a NaN in the embedding row of symbol 0 makes every later logit a NaN: index 0 again, by the other rule
    nan_emb = embedding.clone()
    nan_emb[0, 3] = float("nan")
    plan2 = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    want = loop_driven_from_the_host(plan2, enc, nan_emb, nan_emb[0], 4, 2, T * 2)
    symbols, result, hn, cn = plan2.greedy_decode(enc, nan_emb, nan_emb[0], 4, 2)
    torch.cuda.synchronize()
    r = result.cpu().tolist()
    assert r[0] == len(want[0]) == T * 2 and symbols[: r[0]].cpu().tolist() == want[0] == [0] * (T * 2)
    assert bool(torch.isnan(hn).all()) and bool(torch.isnan(want[3]).all())
    # no budget
    symbols, result, hn, cn = plan.greedy_decode(enc, embedding, x0, 1, 3, 0)
    torch.cuda.synchronize()
    assert result.cpu().tolist()[:3] == [0, 0, 0] and float(hn.abs().max()) == 0.0
    assert plan.fallbacks() == (0, True) and plan2.fallbacks() == (0, True)


def test_arguments_the_loop_refuses(ops):
    L, I, H, F, J, V, T = 2, 320, 320, 1024, 512, 29, 8
    params, joint, enc, embedding, x0 = model(7171, L, I, H, F, J, V, T, 28, 0.5)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    with pytest.raises(ops.NNRuntimeException, match="blank"):
        plan.greedy_decode(enc, embedding, x0, 29)
    with pytest.raises(ops.NNRuntimeException, match="rows"):
        plan.greedy_decode(enc, embedding[:20], x0, 28)
    with pytest.raises(ops.NNRuntimeException, match="max_symbols_per_frame"):
        plan.greedy_decode(enc, embedding, x0, 28, 0)
    with pytest.raises(ops.NNRuntimeException, match="x0"):
        plan.greedy_decode(enc, embedding, None, 28)
    with pytest.raises(ops.NNRuntimeException, match=r"\[T, 1024\]"):
        plan.greedy_decode(enc[:, :512], embedding, x0, 28)
    # more symbols than the loop kernel keeps logits for: the C ABI says so (the Python layer then drives the loop itself, below)
    g2, params2, joint2 = make(7272, 1, 64, 32, 128, 64, 600, True)
    plan2 = ops.RnntPlan(dev(params2), True, 1, tuple(dev(joint2)))
    import ctypes
    from pimaicompiler_amd import _lib
    z = lambda *shape: torch.zeros(*shape, dtype=torch.float16, device=DEV)  # noqa: E731
    e4, emb, x64, st = z(4, 128), z(600, 64), z(64), z(1, 32)
    sym, res = torch.zeros(8, dtype=torch.int32, device=DEV), torch.zeros(8, dtype=torch.int32, device=DEV)
    rc = _lib.load().pimhip_rnnt_greedy_decode(plan2._handle, e4.data_ptr(), 4, emb.data_ptr(), 600, x64.data_ptr(), None, None, 1, 0, 30, 8,
                                               sym.data_ptr(), res.data_ptr(), st.data_ptr(), st.clone().data_ptr(), None)
    assert rc == _lib.PIMHIP_ERR_UNSUPPORTED
    with pytest.raises(ops.NNRuntimeException, match="blank"):
        plan2.greedy_decode(e4, emb, x64, 600)


def test_a_vocabulary_the_loop_kernel_does_not_take_is_decoded_from_the_host(ops):
    """600 symbols: ops.RnntPlan.greedy_decode drives pimhip_rnnt_step itself and returns what the one-launch loop returns
    (same fields, same meaning); checked against this file's own host loop and, for the first steps, LibTorch CPU."""
    L, I, H, F, J, V, T, blank = 1, 64, 32, 128, 64, 600, 20, 599
    params, joint, enc, embedding, x0 = model(7373, L, I, H, F, J, V, T, blank, 0.35)
    plan = ops.RnntPlan(dev(params), True, L, tuple(dev(joint)))
    want = loop_driven_from_the_host(plan, enc, embedding, x0, blank, 3, T * 3)
    r = check(plan.greedy_decode(enc, embedding, x0, blank, 3), want)
    print(f"600 symbols from the host: {r[0]} symbols over {r[1]} frames in {r[2]} steps", flush=True)
    assert r[1] == T and r[0] > 0 and r[3] == 0
    # a budget of symbols ends the loop as it ends the kernel's
    want = loop_driven_from_the_host(plan, enc, embedding, x0, blank, 3, 4)
    check(plan.greedy_decode(enc, embedding, x0, blank, 3, 4), want)
