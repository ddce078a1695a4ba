"""The C ABI driven from two host threads on one GPU, each with a stream of its own: the reference runs one executor per
host thread (examples/runtime/source/pipeline_manager.cpp:230-295; every thread sets its device first, :234).  One thread
issues GEMVs in both operand orders (the sliced I_X_W product allocates its stream's workspace on first use), the other
seq_len-1 LSTM steps and short sequences of a plan of its own; both go through ctypes, which releases the interpreter lock
for the duration of a call, so the calls really overlap.  Every result is checked against the CPU oracle.
Tolerances: 2e-3 on GEMV outputs, 5e-3 on LSTM outputs (fp16 storage, fp32 accumulation)."""
import threading

import numpy as np
import pytest
import torch

from oracle import oracle
from pimaicompiler_amd import _lib as L
from pimaicompiler_amd import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_two_host_threads_share_the_library_on_one_gpu(ops):
    lib = L.load()
    rounds = 60
    errors = []
    W, x, b = workloads.gemv_inputs(2201, 1024, 2048)
    A = W.t().contiguous()                                   # [in, out] for the I_X_W order
    want_g = oracle.gemv_mv(W.numpy(), x.numpy().reshape(-1), b.numpy())
    params, xs, h0, c0 = workloads.lstm_inputs(2202, 256, 256, 2, False, 12)
    h0, c0 = (0.2 * torch.randn(2, 1, 256)).half(), (0.2 * torch.randn(2, 1, 256)).half()
    want_seq = oracle.lstm(xs.numpy().reshape(12, 256), h0.numpy().reshape(2, 256), c0.numpy().reshape(2, 256),
                           [p.numpy() for p in params], True, 2, False)
    want_step = oracle.lstm(xs.numpy().reshape(12, 256)[:1], h0.numpy().reshape(2, 256), c0.numpy().reshape(2, 256),
                            [p.numpy() for p in params], True, 2, False)
    Wd, Ad, xd, bd = W.to(DEV), A.to(DEV), x.to(DEV).reshape(-1), b.to(DEV)
    pd = [p.to(DEV) for p in params]
    xsd, h0d, c0d = xs.reshape(12, 256).to(DEV), h0.to(DEV), c0.to(DEV)
    torch.cuda.synchronize()
    start = threading.Barrier(2)

    def gemv_thread():
        try:
            torch.cuda.set_device(0)                        # as the reference's threads do before anything else
            s = torch.cuda.Stream()
            outs = [torch.zeros(1024, dtype=torch.float16, device=DEV) for _ in range(2 * rounds)]
            start.wait()
            for i in range(rounds):
                for j, (w, order) in enumerate(((Wd, L.PIMHIP_W_X_I), (Ad, L.PIMHIP_I_X_W))):
                    rc = lib.pimhip_execute_gemv(outs[2 * i + j].data_ptr(), xd.data_ptr(), w.data_ptr(), bd.data_ptr(), 2048, 1024, 0,
                                                 L.PIMHIP_ACT_NONE, order, s.cuda_stream)
                    assert rc == 0, lib.pimhip_last_error()
            s.synchronize()
            for o in outs:
                err = float(np.max(np.abs(o.float().cpu().numpy() - want_g.astype(np.float32))))
                assert err <= 2e-3, err
        except BaseException as e:  # noqa: BLE001 - handed to the main thread
            errors.append(e)

    def lstm_thread():
        try:
            torch.cuda.set_device(0)
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                plan = ops.LstmPlan(pd, True, 2, False, 12, stream=s)
            results = []
            start.wait()
            for i in range(rounds):
                T = 1 if i % 2 else 12
                results.append((T, plan.forward(xsd[:T], h0d, c0d, stream=s)))
            s.synchronize()
            plan.status()
            for T, (y, hn, cn) in results:
                want = want_step if T == 1 else want_seq
                for got, w in zip((y, hn, cn), want):
                    err = float(np.max(np.abs(got.float().cpu().numpy().reshape(-1) - w.astype(np.float32).reshape(-1))))
                    assert err <= 5e-3, (T, err)
        except BaseException as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=gemv_thread), threading.Thread(target=lstm_thread)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a thread is still running"
    if errors:
        raise errors[0]
    # the error text is per thread: a failure on one thread does not show up in the other's
    assert lib.pimhip_execute_gemv(None, None, None, None, 8, 8, 0, 0, 0, None) != 0
    seen = []
    t = threading.Thread(target=lambda: seen.append(lib.pimhip_last_error()))
    t.start()
    t.join()
    assert seen == [b""] and lib.pimhip_last_error() != b""
