"""Writes the LibTorch-CPU golden vectors of tests/golden/*.npz.

    python tests/golden/make_golden.py

Every vector is the output of the container's own LibTorch (torch CPU, fp16) on the seeded synthetic inputs of
oracle/oracle.py: at::addmm for the GEMV configurations, at::matmul + relu + argmax for the MoE step, at::lstm for
the LSTM configurations.  Nothing of the reference is imported or run.  Large configurations store the final
states and strided samples of the outputs; the small ones store inputs and outputs in full.
"""
import hashlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from oracle import oracle  # noqa: E402
from pimaicompiler_amd import workloads

torch.set_num_threads(8)

GEMV_CASES = {  # name -> (seed, out, in)
    "c1_1024x1024": (1001, 1024, 1024),
    "c2_4096x4096": (2001, 4096, 4096),
    "c2_16384x4096": (2002, 16384, 4096),
    "c2_4096x16384": (2003, 4096, 16384),
    "c2_32000x1024": (2004, 32000, 1024),
}


def digest(*tensors):
    h = hashlib.sha256()
    for t in tensors:
        h.update(t.contiguous().numpy().tobytes())
    return np.frombuffer(h.digest(), dtype=np.uint8)


def gemv_goldens():
    out = {}
    for name, (seed, n, k) in GEMV_CASES.items():
        W, x, b = workloads.gemv_inputs(seed, n, k)
        y = oracle.torch_addmm(b, x, W).reshape(-1)
        out[name + "_inputs_sha256"] = digest(W, x, b)
        if n <= 1024:
            out[name + "_y"] = y.numpy()
        else:
            idx = np.arange(0, n, n // 64)[:64]
            out[name + "_idx"] = idx
            out[name + "_y_samples"] = y.numpy()[idx]
            out[name + "_y_sum"] = np.array([y.double().sum().item()])
    np.savez(os.path.join(HERE, "gemv.npz"), **out)


def moe_inputs(seed=5001):
    g = torch.Generator().manual_seed(seed)
    Wr = (0.02 * torch.randn(8, 768, generator=g)).half()
    W1 = [(0.02 * torch.randn(3072, 768, generator=g)).half() for _ in range(8)]
    W2 = [(0.02 * torch.randn(768, 3072, generator=g)).half() for _ in range(8)]
    x = torch.randn(1, 768, generator=g).half()
    return Wr, W1, W2, x


def moe_golden():
    Wr, W1, W2, x = moe_inputs()
    logits = torch.matmul(x, Wr.t())
    e = int(torch.argmax(logits))
    top2 = torch.topk(logits.float().reshape(-1), 2).values
    assert float(top2[0] - top2[1]) > 2e-3, "router logits of the seeded token are too close; reseed"
    hidden = torch.relu(torch.matmul(x, W1[e].t()))
    y = torch.matmul(hidden, W2[e].t())
    np.savez(os.path.join(HERE, "moe.npz"), logits=logits.numpy().reshape(-1), expert=np.array([e]),
             hidden=hidden.numpy().reshape(-1), y=y.numpy().reshape(-1), inputs_sha256=digest(Wr, x, W1[e], W2[e]))


def lstm_tiny_goldens():
    out = {}
    case = 0
    for L in (1, 2):
        for bidir in (False, True):
            for has_b in (True, False):
                seed = 7000 + case
                params, x, h0, c0 = workloads.lstm_inputs(seed, 16, 32, L, bidir, 5, has_b)
                g = torch.Generator().manual_seed(seed + 500)
                h0 = (0.5 * torch.randn(h0.shape, generator=g)).half()
                c0 = (0.5 * torch.randn(c0.shape, generator=g)).half()
                y, hn, cn = oracle.torch_lstm(x, h0, c0, params, has_b, L, bidir)
                key = f"L{L}_D{2 if bidir else 1}_b{int(has_b)}"
                out[key + "_seed"] = np.array([seed])
                for i, p in enumerate(params):
                    out[f"{key}_p{i}"] = p.numpy()
                out[key + "_x"] = x.numpy()
                out[key + "_h0"] = h0.numpy()
                out[key + "_c0"] = c0.numpy()
                out[key + "_y"] = y.numpy()
                out[key + "_hn"] = hn.numpy()
                out[key + "_cn"] = cn.numpy()
                case += 1
    np.savez(os.path.join(HERE, "lstm_tiny.npz"), **out)


def lstm_large_goldens():
    out = {}
    # C3: RNNT-style, 2 layers unidirectional, I=240, H=1024, T=200.
    params, x, h0, c0 = workloads.lstm_inputs(3001, 240, 1024, 2, False, 200)
    y, hn, cn = oracle.torch_lstm(x, h0, c0, params, True, 2, False)
    out["c3_inputs_sha256"] = digest(x, *params)
    out["c3_hn"] = hn.numpy()
    out["c3_cn"] = cn.numpy()
    out["c3_y_samples"] = y.numpy().reshape(200, 1024)[::25, ::16]
    # C4: GNMT-style: four at::lstm calls (L0 bidirectional I=1024, L1 I=2048, L2, L3 I=1024), T=50, then the
    # 1024 -> 32000 GEMV on the last step's output.
    g_in = 1024
    seq = None
    for li, (in_w, bidir) in enumerate([(1024, True), (2048, False), (1024, False), (1024, False)]):
        params, x0, h0, c0 = workloads.lstm_inputs(4001 + li, in_w, 1024, 1, bidir, 50)
        if seq is None:
            seq = x0
        y, hn, cn = oracle.torch_lstm(seq, h0, c0, params, True, 1, bidir)
        out[f"c4_l{li}_hn"] = hn.numpy()
        out[f"c4_l{li}_cn"] = cn.numpy()
        out[f"c4_l{li}_y_samples"] = y.numpy().reshape(50, -1)[::7, ::32]
        seq = y
    W, _, b = workloads.gemv_inputs(4010, 32000, 1024)
    logits = oracle.torch_addmm(b, seq[-1].reshape(1, 1024), W).reshape(-1)
    idx = np.arange(0, 32000, 500)
    out["c4_logits_idx"] = idx
    out["c4_logits_samples"] = logits.numpy()[idx]
    out["c4_logits_argmax"] = np.array([int(torch.argmax(logits.float()))])
    np.savez(os.path.join(HERE, "lstm_large.npz"), **out)


if __name__ == "__main__":
    gemv_goldens()
    moe_golden()
    lstm_tiny_goldens()
    lstm_large_goldens()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
