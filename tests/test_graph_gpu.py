"""A launch-bound decoder step (four LSTM layers at seq_len 1, the attention context, two residual adds, the 32000-way
classifier GEMV: eight launches) captured into a HIP graph and replayed.  None of these calls allocates, synchronises or records a
memset, so the capture holds kernels only; every replay is compared with the eager run of the same inputs, with eager
work and synchronisations between the replays."""
import pytest
import torch

from oracle import oracle
from pimaicompiler_amd import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
H = 1024


class DecoderStep:
    """Static buffers + the sequence of operator calls of one decoder step (GNMT-like wiring, random weights)."""

    def __init__(self, P, seed=0, vocab=32000, src_len=50):
        g = torch.Generator().manual_seed(seed)
        self.P = P
        in_w = [H, 2 * H, 2 * H, 2 * H]
        self.plans, self.state = [], []
        for k in range(4):
            params = workloads.lstm_inputs(seed + 10 + k, in_w[k], H, 1, False, 1)[0]
            self.plans.append(P.LstmPlan([p.to(DEV) for p in params], True, 1, False, 1))
            self.state.append(((0.1 * torch.randn(1, H, generator=g)).half().to(DEV), (0.1 * torch.randn(1, H, generator=g)).half().to(DEV)))
        self.enc = torch.randn(1, src_len, H, generator=g).half().to(DEV)          # encoder outputs
        self.att = torch.softmax(torch.randn(1, 1, src_len, generator=g), -1).half().to(DEV)
        self.Wc = (0.02 * torch.randn(vocab, H, generator=g)).half().to(DEV)
        self.bc = (0.01 * torch.randn(vocab, generator=g)).half().to(DEV)
        self.x = torch.zeros(1, H, dtype=torch.float16, device=DEV)                  # the step's input embedding
        self.cat = [torch.zeros(1, 2 * H, dtype=torch.float16, device=DEV) for _ in range(3)]   # [y_k, context] for layers 1..3
        self.y = [torch.zeros(1, H, dtype=torch.float16, device=DEV) for _ in range(4)]
        self.hn = [torch.zeros(1, H, dtype=torch.float16, device=DEV) for _ in range(4)]
        self.cn = [torch.zeros(1, H, dtype=torch.float16, device=DEV) for _ in range(4)]
        self.res = [torch.zeros(1, H, dtype=torch.float16, device=DEV) for _ in range(2)]
        self.logits = torch.zeros(1, vocab, dtype=torch.float16, device=DEV)
        self.ctx_views = [c.view(-1)[H:] for c in self.cat]
        self.y0_view = self.cat[0].view(-1)[:H].view(1, H)
        self.y1_view = self.cat[1].view(-1)[:H].view(1, H)
        self.res0_view = self.cat[2].view(-1)[:H].view(1, H)

    def run(self):
        P = self.P
        # layer 0 writes its output straight into the head of layer 1's input buffer
        self.plans[0].forward(self.x, *self.state[0], out=(self.y0_view, self.hn[0], self.cn[0]))
        # attention context into the tails of the three concatenation buffers with one launch
        P.aten_bmm(self.att, self.enc, outs=self.ctx_views)
        # layer 1's output and the residual sum go straight to the heads of the next layers' input buffers
        self.plans[1].forward(self.cat[0], *self.state[1], out=(self.y1_view, self.hn[1], self.cn[1]))
        self.plans[2].forward(self.cat[1], *self.state[2], out=(self.y[2], self.hn[2], self.cn[2]))
        P.aten_add(self.y[2], self.y1_view, out=self.res0_view)                          # residual
        self.plans[3].forward(self.cat[2], *self.state[3], out=(self.y[3], self.hn[3], self.cn[3]))
        P.aten_add(self.y[3], self.res0_view, out=self.res[1])
        lib, L = self.lib()
        rc = lib.pimhip_execute_gemv(self.logits.data_ptr(), self.res[1].data_ptr(), self.Wc.data_ptr(), self.bc.data_ptr(), H,
                                     self.Wc.size(0), 0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, torch.cuda.current_stream().cuda_stream)
        assert rc == 0

    @staticmethod
    def lib():
        from pimaicompiler_amd import _lib as L
        return L.load(), L

    def outputs(self):
        return [self.logits.clone(), self.res[1].clone()] + [t.clone() for t in self.hn + self.cn]


def test_decoder_step_replays_from_a_graph(ops):
    step = DecoderStep(ops, seed=3)
    g = torch.Generator().manual_seed(99)
    inputs = [torch.randn(1, H, generator=g).half().to(DEV) for _ in range(4)]
    step.x.copy_(inputs[0])
    step.run()                                   # warm-up outside the capture (plans, library state)
    torch.cuda.synchronize()
    eager = []
    for x in inputs:
        step.x.copy_(x)
        step.run()
        torch.cuda.synchronize()
        eager.append(step.outputs())
    assert not torch.equal(eager[0][0], eager[1][0])
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step.x.copy_(inputs[0])
        with torch.cuda.graph(graph, stream=side):
            step.run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    scratch = torch.randn(1 << 20, device=DEV)
    for rep in range(2):
        for x, want in zip(inputs, eager):
            step.x.copy_(x)
            for t in step.hn + step.cn + [step.logits]:
                t.fill_(float("nan"))            # a replay must rewrite every output
            graph.replay()
            scratch = scratch * 1.0001 + 1.0     # eager work between the replays
            torch.cuda.synchronize()
            for got, w in zip(step.outputs(), want):
                assert torch.equal(got, w)


def test_decoder_step_matches_libtorch_cpu(ops):
    step = DecoderStep(ops, seed=5, vocab=4096)
    g = torch.Generator().manual_seed(1)
    step.x.copy_(torch.randn(1, H, generator=g).half().to(DEV))
    step.run()
    torch.cuda.synchronize()
    # the same wiring on the CPU with LibTorch
    def cpu_lstm(k, inp):
        prm = [p.cpu() for p in step.plans[k].params]
        h0, c0 = step.state[k]
        y, hn, cn = torch.lstm(inp.cpu().view(1, 1, -1), (h0.cpu().view(1, 1, H), c0.cpu().view(1, 1, H)), prm, True, 1, 0.0, False, False, False)
        return y.view(1, H)
    y0 = cpu_lstm(0, step.x)
    ctx = torch.bmm(step.att.cpu().float(), step.enc.cpu().float()).half().view(1, H)
    y1 = cpu_lstm(1, torch.cat([y0, ctx], 1))
    y2 = cpu_lstm(2, torch.cat([y1, ctx], 1))
    r0 = y2 + y1
    y3 = cpu_lstm(3, torch.cat([r0, ctx], 1))
    r1 = y3 + r0
    logits = torch.addmm(step.bc.cpu(), r1, step.Wc.cpu().t())
    assert float((step.res[1].cpu().float() - r1.float()).abs().max()) <= 5e-3
    assert float((step.logits.cpu().float() - logits.float()).abs().max()) <= 5e-3


def test_sequence_forward_replays_from_a_graph(ops):
    """The persistent sequence kernel keeps its step count in device memory, so a recorded launch replays: every replay
    equals the eager launch bit for bit, with eager launches of the same plan between the replays.  The one thing a
    graph must not record, the re-initialisation of the exchange buffer after a change of mode, is refused."""
    I, Hs = 64, 256
    # (the first three run one recurrence per XCD: a bidirectional layer of 20 steps in automatic mode, mode 4 by request,
    # and a stack of three layers as a pipeline over the XCDs)
    # (the last two: residual sums around the upper layers, inside the pipeline and as add launches between the layers)
    for layers, bidir, T, mode, first_res in ((1, True, 20, 0, None), (1, False, 18, 4, None), (3, False, 21, 0, None), (2, False, 7, 0, None),
                                              (1, True, 7, 0, None), (1, False, 7, 0, None), (3, False, 21, 0, 1), (3, False, 7, 0, 1)):
        params, x, h0, c0 = workloads.lstm_inputs(7101 + layers + 2 * bidir + T, I, Hs, layers, bidir, T)
        plan = ops.LstmPlan([p.to(DEV) for p in params], True, layers, bidir, T)
        plan.set_mode(mode)
        plan.set_residual(first_res)
        xd, hd, cd = x.reshape(T, I).to(DEV), h0.to(DEV), c0.to(DEV)
        x2 = (0.5 * xd + 0.25).contiguous()
        eager = {k: [t.clone() for t in plan.forward(v, hd, cd)] for k, v in (("a", xd), ("b", x2))}
        torch.cuda.synchronize()
        plan.status()
        x_static = xd.clone()
        out = tuple(torch.zeros_like(t) for t in eager["a"])
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            plan.forward(x_static, hd, cd, out=out)                 # warm-up on the capture stream
            with torch.cuda.graph(graph, stream=side):
                plan.forward(x_static, hd, cd, out=out)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for rep in range(4):
            key, src = (("a", xd), ("b", x2))[rep & 1]
            x_static.copy_(src)
            for t in out:
                t.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            plan.status()
            for got, w in zip(out, eager[key]):
                assert torch.equal(got, w)
            if rep != 2:                                              # an odd number of eager launches in between as well
                again = plan.forward(x2, hd, cd)
                torch.cuda.synchronize()
                for got, w in zip(again, eager["b"]):
                    assert torch.equal(got, w)
    # a pending re-initialisation (mode 3 lays the single chain's entries out differently) is not recorded
    params, x, h0, c0 = workloads.lstm_inputs(7109, I, Hs, 1, False, 7)
    plan = ops.LstmPlan([p.to(DEV) for p in params], True, 1, False, 7)
    xd, hd, cd = x.reshape(7, I).to(DEV), h0.to(DEV), c0.to(DEV)
    eager = {"a": [t.clone() for t in plan.forward(xd, hd, cd)]}
    x_static = xd.clone()
    out = tuple(torch.zeros_like(t) for t in eager["a"])
    plan.set_mode(3)
    graph2 = torch.cuda.CUDAGraph()
    scratch_out = torch.empty_like(hd)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph2, stream=side):
            with pytest.raises(ops.NNRuntimeException, match="outside the capture"):
                plan.forward(x_static, hd, cd, out=out)
            ops.aten_add(hd, cd, out=scratch_out)                    # something to record
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    got = plan.forward(xd, hd, cd)
    torch.cuda.synchronize()
    plan.status()
    for g_, w in zip(got, eager["a"]):
        assert float((g_.float() - w.float()).abs().max()) <= 2e-3


def test_sliced_vm_product_replays_from_a_graph(ops):
    """An I_X_W product whose reduction is sliced over blocks uses a per-stream workspace: its first use on a stream
    allocates (refused while capturing, with a message that says what to do), later uses record one kernel and replay."""
    from pimaicompiler_amd import _lib as L
    lib = L.load()
    g = torch.Generator().manual_seed(11)
    K = N = 2048
    A = (0.02 * torch.randn(K, N, generator=g)).half().to(DEV)
    xs = [torch.randn(K, generator=g).half().to(DEV) for _ in range(2)]
    x, y = xs[0].clone(), torch.empty(N, dtype=torch.float16, device=DEV)

    def launch():
        return lib.pimhip_execute_gemv(y.data_ptr(), x.data_ptr(), A.data_ptr(), None, K, N, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W,
                                       torch.cuda.current_stream().cuda_stream)
    eager = []
    for xv in xs:
        x.copy_(xv)
        assert launch() == 0
        torch.cuda.synchronize()
        eager.append(y.clone())
        assert float((y.float() - (xv.float() @ A.float())).abs().max()) <= 2e-3
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    refused = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(refused, stream=side):
            assert launch() == L.PIMHIP_ERR_UNSUPPORTED
            assert b"before the capture" in lib.pimhip_last_error()
            y.add_(0)                                       # something to record
        assert launch() == 0                                # the warm-up the message asks for
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            assert launch() == 0
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for rep in range(4):
        x.copy_(xs[rep & 1])
        y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager[rep & 1])
