"""Seeded synthetic inputs of the benchmark configurations (torch CPU generator, drawn in fp32, then .half()).

Shared by bench.py, the tests and the script that writes the golden vectors, so that all of them see the same
tensors for a given seed.  Nothing here computes a result."""
import math

import torch


def gemv_inputs(seed, out_w, in_w, bias=True):
    """W[out,in] = 0.02*randn, x[1,in] = 2*rand-1, b[out] = 0.01*randn, drawn in fp32 in that order, then .half()."""
    g = torch.Generator().manual_seed(seed)
    W = (0.02 * torch.randn(out_w, in_w, generator=g)).half()
    x = (2 * torch.rand(1, in_w, generator=g) - 1).half()
    b = (0.01 * torch.randn(out_w, generator=g)).half() if bias else None
    return W, x, b


def lstm_inputs(seed, input_size, hidden, num_layers, bidirectional, seq_len, has_biases=True):
    """Per layer and direction w_ih, w_hh, b_ih, b_hh ~ U(-1/sqrt(H), 1/sqrt(H)); x[T,1,I] = randn; zero h0, c0."""
    g = torch.Generator().manual_seed(seed)
    D = 2 if bidirectional else 1
    k = 1.0 / math.sqrt(hidden)
    params = []
    for l in range(num_layers):
        in_w = input_size if l == 0 else D * hidden
        for _ in range(D):
            shapes = [(4 * hidden, in_w), (4 * hidden, hidden)] + ([(4 * hidden,), (4 * hidden,)] if has_biases else [])
            for s in shapes:
                params.append(((2 * torch.rand(*s, generator=g) - 1) * k).half())
    x = torch.randn(seq_len, 1, input_size, generator=g).half()
    h0 = torch.zeros(num_layers * D, 1, hidden, dtype=torch.float16)
    c0 = torch.zeros(num_layers * D, 1, hidden, dtype=torch.float16)
    return params, x, h0, c0
