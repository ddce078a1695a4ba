"""pimhip_execute_gemv_static, the GEMV entry point that allocates nothing, against pimhip_execute_gemv.

Both run the same kernel with the same slicing, so the outputs must agree bit for bit (the bar for every GEMV here is
max abs error <= 2e-3 against the oracle; the test also holds the static entry point to it).  Two calls in a row
share the library's static scratch array, the second with a smaller input: it must not see anything the first left."""
import numpy as np
import pytest
import torch

from oracle import oracle
from pimaicompiler_amd import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GEMV_TOL = 2e-3


def _call(fn, weight, x, bias, in_w, out_w, act, order):
    out = torch.full((out_w,), float("nan"), dtype=torch.float16, device=DEV)
    rc = fn(out.data_ptr(), x.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None, in_w, out_w,
            0, act, order, torch.cuda.current_stream().cuda_stream)
    return rc, out


# (out, in): every one is sliced over K in the I_X_W order; the second of a pair is the smaller input.
PAIRS = [((4096, 4096), (1024, 1024)), ((1024, 4096), (512, 1344)), ((3072, 768), (768, 3072))]


@pytest.mark.parametrize("first,second", PAIRS)
def test_static_entry_point_matches_the_allocating_one_on_two_calls_in_a_row(ops, first, second):
    from pimaicompiler_amd import _lib as L
    lib = L.load()
    for (n, k) in (first, second):
        W, x, b = workloads.gemv_inputs(7000 + n + k, n, k, bias=True)
        want = oracle.gemv_mv(W.numpy(), x.numpy().reshape(-1), b.numpy(), relu=True)
        At = W.t().contiguous().to(DEV)
        xd, bd = x.to(DEV).reshape(-1), b.to(DEV)
        print(f"static gemv I_X_W out={n} in={k}", flush=True)
        rc, y_static = _call(lib.pimhip_execute_gemv_static, At, xd, bd, k, n, L.PIMHIP_ACT_RELU, L.PIMHIP_I_X_W)
        assert rc == 0, lib.pimhip_last_error()
        rc, y_alloc = _call(lib.pimhip_execute_gemv, At, xd, bd, k, n, L.PIMHIP_ACT_RELU, L.PIMHIP_I_X_W)
        assert rc == 0, lib.pimhip_last_error()
        torch.cuda.synchronize()
        assert torch.equal(y_static.view(torch.int16), y_alloc.view(torch.int16))
        err = float(np.max(np.abs(y_static.float().cpu().numpy() - want.astype(np.float32))))
        assert err <= GEMV_TOL, err
        # The other order needs no scratch and must pass through unchanged.
        Wd = W.to(DEV)
        rc, y_mv = _call(lib.pimhip_execute_gemv_static, Wd, xd, bd, k, n, L.PIMHIP_ACT_RELU, L.PIMHIP_W_X_I)
        assert rc == 0, lib.pimhip_last_error()
        rc, y_mv2 = _call(lib.pimhip_execute_gemv, Wd, xd, bd, k, n, L.PIMHIP_ACT_RELU, L.PIMHIP_W_X_I)
        assert rc == 0
        assert torch.equal(y_mv.view(torch.int16), y_mv2.view(torch.int16))


def test_static_entry_point_records_on_a_stream_it_has_never_seen(ops):
    """A sliced I_X_W product through pimhip_execute_gemv is refused on a capturing stream it has not run on before (it
    would have to allocate that stream's workspace); the static entry point records one kernel there, and every replay,
    with eager calls between the replays, gives the eager result."""
    from pimaicompiler_amd import _lib as L
    lib = L.load()
    n, k = 2048, 4096
    W, x, b = workloads.gemv_inputs(7100, n, k, bias=True)
    At, xd, bd = W.t().contiguous().to(DEV), x.to(DEV).reshape(-1), b.to(DEV)
    rc, eager = _call(lib.pimhip_execute_gemv_static, At, xd, bd, k, n, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W)
    assert rc == 0, lib.pimhip_last_error()
    torch.cuda.synchronize()
    out = torch.zeros(n, dtype=torch.float16, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.pimhip_execute_gemv_static(out.data_ptr(), xd.data_ptr(), At.data_ptr(), bd.data_ptr(), k, n, 0,
                                                L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.pimhip_last_error()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for rep in range(4):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), rep
        rc, again = _call(lib.pimhip_execute_gemv_static, At, xd, bd, k, n, L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(again.view(torch.int16), eager.view(torch.int16))
