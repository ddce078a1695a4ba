"""The executor level of the path: blob store, attribute-or-blob unboxing, cursor handling and the execute* functions.

CPU tests replace the operator layer by a recorder and check which operands each executor unboxes, in the order of
runtime/source/executor/op_executor/aten_ops_executor.cpp (addmm :181-254, linear :2029-2059, LSTM1 :2135-2307,
LSTM2 :2309-2399, matmul :2488-2525) and stream_ops_executor.cpp:27-50.  GPU tests run the same layers for real and
compare with the oracle and LibTorch CPU.
"""
import numpy as np
import pytest
import torch

from oracle import oracle
from pimaicompiler_amd import workloads
from pimaicompiler_amd import executor as E
from pimaicompiler_amd.executor import DataType, LayerType

TOL_GEMV = 2e-3
TOL_LSTM = 5e-3


class Recorder:
    """Stands in for pimaicompiler_amd.ops: records each call, returns a marker."""

    def __init__(self):
        self.calls = []

    def __getattr__(self, name):
        def f(*a, **k):
            self.calls.append((name, a, k))
            if name in ("aten_lstm1", "aten_lstm2"):
                return ("y", "hy", "cy")
            return name
        return f


@pytest.fixture
def rec(monkeypatch):
    r = Recorder()
    monkeypatch.setattr(E, "ops", r)
    monkeypatch.setattr(E.torch.cuda, "Stream", lambda *a, **k: object())
    return r


def _blobs(ex, **kv):
    for k, v in kv.items():
        i = int(k[1:])
        if isinstance(v, torch.Tensor):
            ex.update_blob(i, DataType.TENSOR, v)
        elif isinstance(v, (list, tuple)):
            ex.update_blob(i, DataType.LIST, v)
        elif v is None:
            ex.update_blob(i, DataType.NONE, None)
        elif isinstance(v, float):
            ex.update_blob(i, DataType.FLOAT64, v)
        else:
            ex.update_blob(i, DataType.INT64, v)


class _NoDevice:
    def __init__(self, device):
        pass

    def __enter__(self):
        return self

    def __exit__(self, *a):
        return False


@pytest.fixture
def ex(rec, monkeypatch):
    monkeypatch.setattr(E.torch.cuda, "device", _NoDevice)
    return E.StreamExecutor([])


# ---- host logic (CPU) -----------------------------------------------------------------------------------------------
def test_sentinels_are_the_reference_values():
    assert E.is_default_int(2 ** 31 - 1) and not E.is_default_int(0)
    assert E.is_default_int64(-2 ** 63) and not E.is_default_int64(1)
    assert E.is_default_double(1.7976931348623157e308) and not E.is_default_double(0.0)


def test_blob_store(ex):
    assert ex.find_blob(7) == (DataType.UNDEFINED, None) and not ex.check_valid_blob_id(7)
    ex.update_blob(7, DataType.INT64, 3)
    ex.update_blob(7, DataType.INT64, 4)        # update overwrites
    assert ex.find_blob(7) == (DataType.INT64, 4) and ex.check_valid_blob_id(7)


def test_addmm_unboxes_three_or_five_inputs_and_routes_none_bias_to_matmul(ex, rec):
    b, m1, m2 = torch.zeros(4), torch.zeros(1, 3), torch.zeros(3, 4)
    _blobs(ex, b0=b, b1=m1, b2=m2, b3=2, b4=5, b9=None)
    E.execute_aten_addmm(E.AtenAddmmLayer(LayerType.ATENADDMM, 0, [0, 1, 2], [10], act_type="aten::relu"), ex)
    name, a, k = rec.calls[-1]
    assert name == "custom_aten_addmm" and a[0] == "aten::relu" and a[1] is b and a[2] is m1 and a[3] is m2
    assert a[4:] == (1, 1) and k == {"stream": None} and ex.find_blob(10) == (DataType.TENSOR, "custom_aten_addmm")
    E.execute_aten_addmm(E.AtenAddmmLayer(LayerType.ATENADDMM, 0, [0, 1, 2, 3, 4], [11]), ex)
    assert rec.calls[-1][1][4:] == (2, 5)       # (beta, alpha) = inputs 3 and 4
    E.execute_aten_addmm(E.AtenAddmmLayer(LayerType.ATENADDMM, 0, [9, 1, 2], [12]), ex)
    assert rec.calls[-1][0] == "custom_aten_matmul" and rec.calls[-1][1] == (m1, m2)


def test_addmm_rejects_non_tensor_operands(ex):
    _blobs(ex, b0=torch.zeros(4), b1=3, b2=torch.zeros(3, 4))
    with pytest.raises(E.NNRuntimeException):
        E.execute_aten_addmm(E.AtenAddmmLayer(LayerType.ATENADDMM, 0, [0, 1, 2], [10]), ex)


def test_linear_takes_weight_and_bias_from_the_layer_ids(ex, rec):
    x, w, b = torch.zeros(1, 3), torch.zeros(4, 3), torch.zeros(4)
    _blobs(ex, b0=x, b20=w, b21=b)
    E.execute_aten_linear(E.AtenLinearLayer(LayerType.ATENLINEAR, 0, [0], [5], weight_ids=[20], bias_ids=[21]), ex)
    assert rec.calls[-1][1] == (x, w, b)
    E.execute_aten_linear(E.AtenLinearLayer(LayerType.ATENLINEAR, 0, [0], [5], weight_ids=[20]), ex)
    assert rec.calls[-1][1] == (x, w, None)


def test_lstm1_flags_from_attributes(ex, rec):
    x, h, c = torch.zeros(5, 1, 8), torch.zeros(2, 1, 8), torch.zeros(2, 1, 8)
    _blobs(ex, b0=x, b1=[h, c])
    params = [torch.zeros(1)]
    layer = E.AtenLSTM1Layer(LayerType.ATENLSTM1, 0, [0, 1], [7, 8, 9], has_biases=1, num_layers=2, dropout=0.0, train=0,
                             bidirectional=0, batch_first=0, param_vector=params)
    E.execute_aten_lstm1(layer, ex)
    name, a, _ = rec.calls[-1]
    assert name == "aten_lstm1" and a[0] is x and a[1] == (h, c) and a[2] is params
    assert a[3:] == (True, 2, 0.0, False, False, False)
    assert [ex.find_blob(i)[1] for i in (7, 8, 9)] == ["y", "hy", "cy"]


def test_lstm1_unset_attributes_come_from_the_following_blobs_in_order(ex, rec):
    """has_biases, num_layers, dropout, train, bidirectional, batch_first — each one only if its attribute is the
    sentinel; a parameter TensorList in slot 2 is skipped (aten_ops_executor.cpp:2162-2206)."""
    x, h, c = torch.zeros(5, 1, 8), torch.zeros(1, 1, 8), torch.zeros(1, 1, 8)
    _blobs(ex, b0=x, b1=[h, c], b2=[torch.zeros(1)], b3=1, b4=3, b5=0.25, b6=0, b7=1, b8=1)
    layer = E.AtenLSTM1Layer(LayerType.ATENLSTM1, 0, [0, 1, 2, 3, 4, 5, 6, 7, 8], [7, 7, 8, 9])
    E.execute_aten_lstm1(layer, ex)
    assert rec.calls[-1][1][3:] == (True, 3, 0.25, False, True, True)
    # mixed: num_layers and train fixed in the layer, the others from blobs 2.. in order
    _blobs(ex, b2=0, b3=0.5, b4=1, b5=0)
    layer = E.AtenLSTM1Layer(LayerType.ATENLSTM1, 0, [0, 1, 2, 3, 4, 5], [7, 8, 9], num_layers=4, train=0)
    E.execute_aten_lstm1(layer, ex)
    assert rec.calls[-1][1][3:] == (False, 4, 0.5, False, True, False)


def test_lstm1_needs_a_pair_of_states_and_three_outputs(ex):
    _blobs(ex, b0=torch.zeros(5, 1, 8), b1=torch.zeros(1, 1, 8), b2=[torch.zeros(1, 1, 8)] * 2)
    full = dict(has_biases=1, num_layers=1, dropout=0.0, train=0, bidirectional=0, batch_first=0)
    with pytest.raises(E.NNRuntimeException):
        E.execute_aten_lstm1(E.AtenLSTM1Layer(LayerType.ATENLSTM1, 0, [0, 1], [7, 8, 9], **full), ex)
    with pytest.raises(E.NNRuntimeException):
        E.execute_aten_lstm1(E.AtenLSTM1Layer(LayerType.ATENLSTM1, 0, [0, 2], [7, 8], **full), ex)


def test_lstm2_operand_order(ex, rec):
    data, bs, h, c = torch.zeros(5, 8), torch.ones(5, dtype=torch.int64), torch.zeros(1, 1, 8), torch.zeros(1, 1, 8)
    _blobs(ex, b0=data, b1=bs, b2=[h, c], b3=1, b4=1, b5=0.0, b6=0, b7=0)
    E.execute_aten_lstm2(E.AtenLSTM2Layer(LayerType.ATENLSTM2, 0, [0, 1, 2, 3, 4, 5, 6, 7], [10, 11, 12]), ex)
    name, a, _ = rec.calls[-1]
    assert name == "aten_lstm2" and a[0] is data and a[1] is bs and a[2] == (h, c)
    assert a[4:] == (True, 1, 0.0, False, False)


def test_multi_stream_issues_each_sibling_on_its_own_stream_and_moves_the_cursor(rec, monkeypatch):
    monkeypatch.setattr(E.torch.cuda, "device", _NoDevice)

    class FakeStream:
        def wait_stream(self, other):
            pass

    class FakeCtx(_NoDevice):
        pass

    monkeypatch.setattr(E.torch.cuda, "Stream", lambda *a, **k: FakeStream())
    monkeypatch.setattr(E.torch.cuda, "current_stream", lambda *a, **k: FakeStream())
    monkeypatch.setattr(E.torch.cuda, "stream", FakeCtx)
    subs = [E.AtenAddmmLayer(LayerType.ATENADDMM, 4, [0, 1, 2], [10]), E.NNLayer(LayerType.ATENMATMUL, 5, [1, 2], [11]),
            E.AtenAddmmLayer(LayerType.ATENADDMM, 6, [0, 1, 2], [12])]
    ms = E.MultiStreamLayer(LayerType.MULTISTREAM, 3, layers=subs)
    ex = E.StreamExecutor([ms])
    assert len(ex.get_streams()) == 3
    _blobs(ex, b0=torch.zeros(4), b1=torch.zeros(4, 3), b2=torch.zeros(3, 1))
    E.execute_multi_stream(ms, ex)
    assert [c[0] for c in rec.calls if c[0] != "initialize"] == ["custom_aten_addmm", "custom_aten_matmul", "custom_aten_addmm"]
    used = [c[2]["stream"] for c in rec.calls if c[0] != "initialize"]
    assert used == ex.get_streams()
    assert ex.cursor == 3 + 3                   # the loop's own increment then steps past the last duplicate
    bad = E.MultiStreamLayer(LayerType.MULTISTREAM, 0, layers=[E.NNLayer(LayerType.ATENBMM, 1, [1, 2], [11])])
    with pytest.raises(E.NNRuntimeException):
        E.execute_multi_stream(bad, ex)


def test_integer_add_stays_on_the_host(ex):
    _blobs(ex, b0=3, b1=4)
    E.execute_aten_add(E.AtenAddLayer(LayerType.ATENADD, 0, [0, 1], [2], alpha=2), ex)
    assert ex.find_blob(2) == (DataType.INT64, 11)


def test_add_reads_alpha_only_if_blob_id_two_exists(ex):
    """aten_ops_executor.cpp:59-66 asks checkValidBlobID(in_id) with the input index (2), not the third input's id."""
    _blobs(ex, b10=3, b11=4, b12=5)
    E.execute_aten_add(E.AtenAddLayer(LayerType.ATENADD, 0, [10, 11, 12], [20]), ex)
    assert ex.find_blob(20) == (DataType.INT64, 7)           # blob 2 does not exist: alpha = 1
    _blobs(ex, b2=0)
    E.execute_aten_add(E.AtenAddLayer(LayerType.ATENADD, 0, [10, 11, 12], [20]), ex)
    assert ex.find_blob(20) == (DataType.INT64, 23)          # blob 2 exists: alpha = blob 12 = 5


def test_builder_assigns_fresh_ids_and_orders_lstm_parameters(rec, monkeypatch):
    """model_builder.cpp:18-224: ids start after the largest output id; weights before biases per layer; the
    parameter vector is (w_ih, w_hh, b_ih, b_hh) per layer and direction."""
    monkeypatch.setattr(E.torch.cuda, "device", _NoDevice)
    w = [torch.full((1,), float(i)) for i in range(4)]      # l0 fwd w_ih, w_hh, l0 bwd w_ih, w_hh
    b = [torch.full((1,), 10.0 + i) for i in range(4)]
    lstm = E.AtenLSTM1Layer(LayerType.ATENLSTM1, 0, [0, 1], [4, 5, 6], has_biases=1, num_layers=1, dropout=0.0, train=0,
                            bidirectional=1, batch_first=0, weights=w, biases=b)
    lin = E.AtenLinearLayer(LayerType.ATENLINEAR, 1, [4], [9], weights=[torch.zeros(2, 2)], biases=[torch.zeros(2)])
    mb = E.ModelBuilder(device="cpu")
    ex = mb.build([lstm, lin])
    assert lstm.weight_ids == [10, 11, 12, 13] and lstm.bias_ids == [14, 15, 16, 17]
    assert lin.weight_ids == [18] and lin.bias_ids == [19]
    assert [float(p) for p in lstm.param_vector] == [0, 1, 10, 11, 2, 3, 12, 13]
    assert ex.find_blob(18)[1] is mb.preloaded_data_container[18][1]
    prep = [c for c in rec.calls if c[0] == "prepare_lstm"]
    assert len(prep) == 1 and prep[0][1][1:4] == (True, 1, True)


def test_builder_refuses_an_lstm_with_unset_flags(rec, monkeypatch):
    monkeypatch.setattr(E.torch.cuda, "device", _NoDevice)
    lstm = E.AtenLSTM2Layer(LayerType.ATENLSTM2, 0, [0, 1, 2], [4, 5, 6], has_biases=1, num_layers=1, train=0,
                            bidirectional=0, weights=[torch.zeros(1)] * 2, biases=[torch.zeros(1)] * 2)   # dropout unset
    with pytest.raises(E.NNRuntimeException):
        E.ModelBuilder(device="cpu").build([lstm])


# ---- on the GPU -------------------------------------------------------------------------------------------------------
DEV = "cuda:0"


def maxabs(a, b):
    return float((torch.as_tensor(a).detach().float().cpu().reshape(-1) - torch.as_tensor(b).detach().float().cpu().reshape(-1)).abs().max())


def _gate_graph(seed, n_gates, out_w, in_w):
    """T(x) already applied: x_t [in,1]; per gate an addmm(b_i, W_i, x_t) (odd gates: matmul(W_i, x_t)); the graph
    lists the MULTISTREAM layer followed by its duplicated sub-layers, as the reference's builder leaves them."""
    Ws, bs, x = [], [], None
    for i in range(n_gates):
        W, x, b = workloads.gemv_inputs(seed + i, out_w, in_w)
        Ws.append(W)
        bs.append(b)
    subs, blobs = [], {"b0": x.t().to(DEV)}
    for i in range(n_gates):
        blobs[f"b{10 + i}"] = Ws[i].to(DEV)
        blobs[f"b{20 + i}"] = bs[i].to(DEV)
        if i % 2 == 0:
            subs.append(E.AtenAddmmLayer(LayerType.ATENADDMM, 2 + i, [20 + i, 10 + i, 0], [30 + i],
                                         act_type="aten::relu" if i == 2 else "none"))
        else:
            subs.append(E.NNLayer(LayerType.ATENMATMUL, 2 + i, [10 + i, 0], [30 + i]))
    layers = [E.AtenLinearLayer(LayerType.ATENLINEAR, 0, [1], [2], weight_ids=[10], bias_ids=[20]),
              E.MultiStreamLayer(LayerType.MULTISTREAM, 1, layers=subs)] + subs
    layers.append(E.AtenLinearLayer(LayerType.ATENLINEAR, 2 + n_gates, [1], [3], weight_ids=[11]))
    blobs["b1"] = x.to(DEV)
    want = []
    for i in range(n_gates):
        want.append(oracle.gemv_mv(Ws[i].numpy(), x.numpy().reshape(-1), bs[i].numpy() if i % 2 == 0 else None, relu=(i == 2)))
    lin = [oracle.gemv_mv(Ws[0].numpy(), x.numpy().reshape(-1), bs[0].numpy()),
           oracle.gemv_mv(Ws[1].numpy(), x.numpy().reshape(-1), None)]
    return layers, blobs, want, lin


@pytest.mark.gpu
@pytest.mark.parametrize("grouped", [False, True])
def test_inference_loop_with_a_multi_stream_layer(ops, grouped):
    layers, blobs, want, lin = _gate_graph(100, 4, 512, 1024)
    ex = E.StreamExecutor(layers, device=0, grouped_multi_stream=grouped)
    _blobs(ex, **blobs)
    calls = []
    table = dict(E.OP_EXECUTORS)
    for t in (LayerType.ATENADDMM, LayerType.ATENMATMUL):
        table[t] = (lambda f: lambda l, e: (calls.append(l.id), f(l, e)))(E.OP_EXECUTORS[t])
    ex.inference(table)
    torch.cuda.synchronize()
    assert calls == []                          # the duplicated sub-layers are skipped by the cursor move
    for i, w in enumerate(want):
        y = ex.find_blob(30 + i)[1]
        assert list(y.shape) == [512, 1] and maxabs(y, w) <= TOL_GEMV
    assert list(ex.find_blob(2)[1].shape) == [1, 512]
    assert maxabs(ex.find_blob(2)[1], lin[0]) <= TOL_GEMV and maxabs(ex.find_blob(3)[1], lin[1]) <= TOL_GEMV


@pytest.mark.gpu
def test_grouped_and_streamed_multi_stream_agree_bit_for_bit(ops):
    outs = []
    for grouped in (False, True):
        layers, blobs, _, _ = _gate_graph(7, 4, 1024, 1024)
        ex = E.StreamExecutor(layers, device=0, grouped_multi_stream=grouped)
        _blobs(ex, **blobs)
        ex.inference()
        torch.cuda.synchronize()
        outs.append([ex.find_blob(30 + i)[1].cpu() for i in range(4)])
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.gpu
def test_addmm_vm_order_and_none_bias(ops):
    W, x, b = workloads.gemv_inputs(3, 320, 256)
    A = W.t().contiguous()
    ex = E.StreamExecutor([], device=0)
    _blobs(ex, b0=b.to(DEV), b1=x.to(DEV), b2=A.to(DEV), b3=None)
    E.execute_aten_addmm(E.AtenAddmmLayer(LayerType.ATENADDMM, 0, [0, 1, 2], [5]), ex)
    E.execute_aten_addmm(E.AtenAddmmLayer(LayerType.ATENADDMM, 0, [3, 1, 2], [6]), ex)
    E.execute_aten_matmul(E.NNLayer(LayerType.ATENMATMUL, 0, [1, 2], [7]), ex)
    assert list(ex.find_blob(5)[1].shape) == [1, 320]
    assert maxabs(ex.find_blob(5)[1], oracle.gemv_vm(x.numpy().reshape(-1), A.numpy(), b.numpy())) <= TOL_GEMV
    no_bias = oracle.gemv_vm(x.numpy().reshape(-1), A.numpy(), None)
    assert maxabs(ex.find_blob(6)[1], no_bias) <= TOL_GEMV and torch.equal(ex.find_blob(6)[1], ex.find_blob(7)[1])


@pytest.mark.gpu
def test_constant_weights_of_the_vm_order_are_laid_out_once_at_preload(ops):
    """preload_constants keeps a constant right operand of addmm / matmul transposed in memory behind the same shape and
    values: the products take the W_X_I kernel on it and agree with the products on the row-major original (both within
    the GEMV tolerance of the oracle); constants with another use keep their layout."""
    W, x, b = workloads.gemv_inputs(4, 1024, 512)
    A = W.t().contiguous()                                   # [in, out], the operand of y = x . A
    layers = [E.AtenAddmmLayer(LayerType.ATENADDMM, 0, [0, 1, 2], [5]), E.NNLayer(LayerType.ATENMATMUL, 0, [1, 2], [6]),
              E.NNLayer(LayerType.ATENMATMUL, 0, [3, 1], [7])]            # blob 3 is a left operand too: untouched
    ex = E.StreamExecutor(layers, device=0)
    relaid = ex.preload_constants({0: b, 2: A, 3: W})
    assert relaid == [2]
    a_dev = ex.find_blob(2)[1]
    assert list(a_dev.shape) == [512, 1024] and a_dev.stride() == (1, 512) and torch.equal(a_dev.cpu(), A)
    assert ex.find_blob(3)[1].is_contiguous()
    ex.update_blob(1, DataType.TENSOR, x.to(DEV))
    E.execute_aten_addmm(layers[0], ex)
    E.execute_aten_matmul(layers[1], ex)
    want = oracle.gemv_vm(x.numpy().reshape(-1), A.numpy(), b.numpy())
    assert list(ex.find_blob(5)[1].shape) == [1, 1024] and maxabs(ex.find_blob(5)[1], want) <= TOL_GEMV
    assert maxabs(ex.find_blob(6)[1], oracle.gemv_vm(x.numpy().reshape(-1), A.numpy(), None)) <= TOL_GEMV
    # the same product on the row-major original (the I_X_W kernel)
    direct = ops.custom_aten_addmm("none", b.to(DEV), x.to(DEV), A.to(DEV))
    assert maxabs(direct, want) <= TOL_GEMV


@pytest.mark.gpu
@pytest.mark.parametrize("bidirectional,num_layers", [(False, 2), (True, 1)])
def test_lstm1_layer_with_flags_from_blobs(ops, bidirectional, num_layers):
    params, x, h0, c0 = workloads.lstm_inputs(11, 64, 128, num_layers, bidirectional, 9)
    g = torch.Generator().manual_seed(5)
    h0 = (0.1 * torch.randn(h0.shape, generator=g)).half()
    c0 = (0.1 * torch.randn(c0.shape, generator=g)).half()
    ex = E.StreamExecutor([], device=0)
    _blobs(ex, b0=x.to(DEV), b1=[h0.to(DEV), c0.to(DEV)], b2=[p.to(DEV) for p in params], b3=1, b4=num_layers, b5=0.0, b6=0,
           b7=int(bidirectional), b8=0)
    layer = E.AtenLSTM1Layer(LayerType.ATENLSTM1, 0, list(range(9)), [20, 21, 22], param_vector=[p.to(DEV) for p in params])
    E.execute_aten_lstm1(layer, ex)
    D = 2 if bidirectional else 1
    y, hn, cn = oracle.lstm(x.numpy().reshape(9, 64), h0.numpy(), c0.numpy(), [p.numpy() for p in params], True, num_layers,
                            bidirectional)
    ty, thn, tcn = oracle.torch_lstm(x, h0, c0, params, True, num_layers, bidirectional)
    got = [ex.find_blob(i)[1] for i in (20, 21, 22)]
    assert list(got[0].shape) == [9, 1, D * 128] and list(got[1].shape) == [num_layers * D, 1, 128]
    for g_, o_, t_ in zip(got, (y, hn, cn), (ty, thn, tcn)):
        assert maxabs(g_, o_) <= TOL_LSTM and maxabs(g_, t_) <= TOL_LSTM


@pytest.mark.gpu
def test_lstm1_layer_with_residual_sums_folded_in(ops):
    """A record a graph rewrite has folded GNMT's aten::add layers into: three layers, sums around the upper two, against
    one at::lstm and one at::add per layer on LibTorch CPU."""
    T, H = 24, 256
    params, x, h0, c0 = workloads.lstm_inputs(13, 2 * H, H, 3, False, T)
    ex = E.StreamExecutor([], device=0)
    _blobs(ex, b0=x.to(DEV), b1=[h0.to(DEV), c0.to(DEV)])
    layer = E.AtenLSTM1Layer(LayerType.ATENLSTM1, 0, [0, 1], [20, 21, 22], has_biases=1, num_layers=3, dropout=0.0, train=0,
                             bidirectional=0, batch_first=0, param_vector=[p.to(DEV) for p in params], first_residual_layer=1)
    E.execute_aten_lstm1(layer, ex)
    cur, hs = x, []
    for l in range(3):
        y, hn, _ = torch.lstm(cur, (h0[l:l + 1], c0[l:l + 1]), params[4 * l:4 * l + 4], True, 1, 0.0, False, False, False)
        hs.append(hn)
        cur = y + cur if l >= 1 else y
    got = [ex.find_blob(i)[1] for i in (20, 21, 22)]
    assert list(got[0].shape) == [T, 1, H]
    assert maxabs(got[0], cur) <= TOL_LSTM and maxabs(got[1], torch.cat(hs, 0)) <= TOL_LSTM
    # the same record without the attribute is a plain stack again (the cached plan is told so on every call)
    layer.first_residual_layer = -1
    E.execute_aten_lstm1(layer, ex)
    ty, _, _ = torch.lstm(x, (h0, c0), params, True, 3, 0.0, False, False, False)
    assert maxabs(ex.find_blob(20)[1], ty) <= TOL_LSTM


@pytest.mark.gpu
def test_lstm2_layer_on_the_rnnt_feature_shape(ops):
    params, x, h0, c0 = workloads.lstm_inputs(12, 240, 256, 2, False, 21)
    ex = E.StreamExecutor([], device=0)
    _blobs(ex, b0=x.reshape(21, 240).to(DEV), b1=torch.ones(21, dtype=torch.int64), b2=[h0.to(DEV), c0.to(DEV)])
    layer = E.AtenLSTM2Layer(LayerType.ATENLSTM2, 0, [0, 1, 2], [20, 21, 22], has_biases=1, num_layers=2, dropout=0.0,
                             train=0, bidirectional=0, param_vector=[p.to(DEV) for p in params])
    E.execute_aten_lstm2(layer, ex)
    y, hn, cn = oracle.lstm(x.numpy().reshape(21, 240), h0.numpy(), c0.numpy(), [p.numpy() for p in params], True, 2, False)
    got = [ex.find_blob(i)[1] for i in (20, 21, 22)]
    assert list(got[0].shape) == [21, 256]
    for g_, o_ in zip(got, (y, hn, cn)):
        assert maxabs(g_, o_) <= TOL_LSTM


@pytest.mark.gpu
def test_add_and_bmm_layers(ops):
    g = torch.Generator().manual_seed(9)
    a, b = torch.randn(1, 1, 1024, generator=g).half(), torch.randn(1, 1, 1024, generator=g).half()
    q, keys = (0.1 * torch.randn(1, 1, 40, generator=g)).half(), torch.randn(1, 40, 1024, generator=g).half()
    ex = E.StreamExecutor([], device=0)
    _blobs(ex, b0=a.to(DEV), b1=b.to(DEV), b2=q.to(DEV), b3=keys.to(DEV), b4=1)
    a_d = a.to(DEV)
    _blobs(ex, b0=a_d)
    E.execute_aten_add(E.AtenAddLayer(LayerType.ATENADD, 0, [0, 1, 4], [5]), ex)
    E.execute_aten_bmm(E.NNLayer(LayerType.ATENBMM, 0, [2, 3], [6]), ex)
    assert np.array_equal(ex.find_blob(5)[1].cpu().numpy(), oracle.add(a.numpy(), b.numpy()).reshape(1, 1, 1024))
    assert ex.find_blob(5)[1].data_ptr() == a_d.data_ptr()      # the custom add writes over `self` (C = A in the reference)
    # GNMT residual add: the sum goes to the head of a concatenation buffer, `self` stays as it was
    exg = E.StreamExecutor([], model_type="GNMT", device=0)
    cat = torch.full((1, 1, 2048), 3.0, dtype=torch.float16, device=DEV)
    a2 = a.to(DEV)
    _blobs(exg, b0=a2, b1=b.to(DEV), b70=cat)
    E.execute_aten_add(E.AtenAddLayer(LayerType.ATENADD, 0, [0, 1], [5], cat_mem_id=70), exg)
    assert np.array_equal(cat[..., :1024].cpu().numpy(), oracle.add(a.numpy(), b.numpy()).reshape(1, 1, 1024))
    assert bool((cat[..., 1024:] == 3.0).all()) and torch.equal(a2.cpu(), a) and exg.find_blob(5)[1].data_ptr() == cat.data_ptr()
    want = oracle.gemv_vm(q.numpy().reshape(-1), keys.numpy().reshape(40, 1024), None)
    assert list(ex.find_blob(6)[1].shape) == [1, 1, 1024] and maxabs(ex.find_blob(6)[1], want) <= TOL_GEMV


@pytest.mark.gpu
def test_built_model_lstm_then_linear_on_the_rnnt_feature(ops):
    """Preload + inference of a two-layer LSTM followed by a linear on its last output row."""
    from pimaicompiler_amd import io
    import os
    feat = io.load_tensor(os.path.join(os.path.dirname(__file__), "golden", "rnnt_feature_341x1x240_f16.bin"), [341, 1, 240], "FLOAT16")
    x = feat[:30].contiguous()
    params, _, h0, c0 = workloads.lstm_inputs(21, 240, 128, 2, False, 30)
    W, _, b = workloads.gemv_inputs(22, 64, 128)
    lstm = E.AtenLSTM1Layer(LayerType.ATENLSTM1, 0, [0, 1], [2, 3, 4], has_biases=1, num_layers=2, dropout=0.0, train=0,
                            bidirectional=0, batch_first=0, weights=[params[i] for i in (0, 1, 4, 5)],
                            biases=[params[i] for i in (2, 3, 6, 7)])
    lin = E.AtenLinearLayer(LayerType.ATENLINEAR, 1, [3], [5], weights=[W], biases=[b])
    ex = E.ModelBuilder(device=0).build([lstm, lin])
    assert [tuple(p.shape) for p in lstm.param_vector] == [tuple(p.shape) for p in params]
    _blobs(ex, b0=x.to(DEV), b1=[h0.to(DEV), c0.to(DEV)])
    ex.inference()
    y, hn, cn = oracle.lstm(x.numpy().reshape(30, 240), h0.numpy(), c0.numpy(), [p.numpy() for p in params], True, 2, False)
    assert maxabs(ex.find_blob(2)[1], y) <= TOL_LSTM and maxabs(ex.find_blob(3)[1], hn) <= TOL_LSTM
    want = np.stack([oracle.gemv_mv(W.numpy(), hn[l], b.numpy()) for l in range(2)])
    got = ex.find_blob(5)[1]
    assert list(got.shape) == [2, 1, 64] and maxabs(got, want) <= 5e-3


@pytest.mark.gpu
def test_gnmt_decoder_steps_write_into_the_state_and_attention_buffers(ops):
    """Four decoder layers, three decode steps.  Layer k reads (h, c) from rows 2k, 2k+1 of the state buffer and writes
    them back there (aten_ops_executor.cpp:2238-2270; miopen_ops_executor.cpp:196-217); layers 0 and 1 put their output
    into the first H columns of the attention concatenation buffer (:2272-2287).  Checked against LibTorch CPU run
    layer by layer with explicit states."""
    H, steps = 256, 3
    g = torch.Generator().manual_seed(31)
    layer_params = [workloads.lstm_inputs(40 + k, H, H, 1, False, 1)[0] for k in range(4)]
    state = (0.2 * torch.randn(8, 1, H, generator=g)).half()
    xs = torch.randn(steps, 4, 1, 1, H, generator=g).half()           # an independent input per step and layer
    ex = E.StreamExecutor([], model_type="GNMT", device=0)
    state_d, att_d = state.to(DEV), torch.zeros(1, 1, 2 * H, dtype=torch.float16, device=DEV)
    att_d[..., H:] = 7.0                                                # the other half belongs to another producer
    ex.update_blob(100, DataType.TENSOR, state_d)
    ex.update_blob(101, DataType.TENSOR, att_d)
    layers = []
    for k in range(4):
        layers.append(E.AtenLSTM1Layer(LayerType.ATENLSTM1, k, [10 + k, 20 + k], [30 + k, 40 + k, 50 + k], has_biases=1,
                                       num_layers=1, dropout=0.0, train=0, bidirectional=0, batch_first=0,
                                       param_vector=[p.to(DEV) for p in layer_params[k]], match_custom_opt=True,
                                       custom_opt_number=k, custom_cat_mem_id=100, output_cat_mem_id=101 if k < 2 else -1))
    ref_state = state.clone()
    for t in range(steps):
        for k in range(4):
            flat = ex.find_blob(100)[1].view(-1)
            h0 = flat[2 * k * H:(2 * k + 1) * H].view(1, 1, H)           # the decoder slices its state out of the buffer
            c0 = flat[(2 * k + 1) * H:(2 * k + 2) * H].view(1, 1, H)
            ex.update_blob(10 + k, DataType.TENSOR, xs[t, k].to(DEV))
            ex.update_blob(20 + k, DataType.LIST, [h0, c0])
            E.execute_aten_lstm1(layers[k], ex)
            wy, wh, wc = oracle.torch_lstm(xs[t, k], ref_state[2 * k:2 * k + 1], ref_state[2 * k + 1:2 * k + 2], layer_params[k],
                                           True, 1, False)
            ref_state[2 * k], ref_state[2 * k + 1] = wh[0], wc[0]
            y = ex.find_blob(30 + k)[1]
            assert maxabs(y, wy) <= TOL_LSTM
            if k < 2:
                assert y.data_ptr() == att_d.data_ptr() and maxabs(att_d[..., :H], wy) <= TOL_LSTM
                assert bool((att_d[..., H:] == 7.0).all())
            assert ex.find_blob(40 + k)[1].data_ptr() == state_d.data_ptr() + 2 * k * H * 2
    assert maxabs(state_d, ref_state) <= TOL_LSTM


@pytest.mark.gpu
def test_decoder_step_record_runs_the_token_as_one_launch(ops):
    """The same four cells as one DecoderStepLayer (layers 1..3 on cat(previous output, context), residual sums from layer
    2 on, the classifier): three tokens of two sentences through the dispatch loop, state updated in place in the state
    buffer blob, against LibTorch CPU running the chain operator by operator."""
    H, S, V = 256, 11, 300
    g = torch.Generator().manual_seed(41)
    params = [workloads.lstm_inputs(60 + k, H if k == 0 else 2 * H, H, 1, False, 1)[0] for k in range(4)]
    Wc, bc = (0.05 * torch.randn(V, H, generator=g)).half(), (0.01 * torch.randn(V, generator=g)).half()
    state = (0.2 * torch.randn(8, 1, H, generator=g)).half()
    cells = [E.AtenLSTM1Layer(LayerType.ATENLSTM1, k, [], [], has_biases=1, num_layers=1, dropout=0.0, train=0, bidirectional=0,
                              batch_first=0, param_vector=[p.to(DEV) for p in params[k]], match_custom_opt=True,
                              custom_opt_number=k, custom_cat_mem_id=100) for k in range(4)]
    layer = E.DecoderStepLayer(LayerType.DECODERSTEP, 0, [1, 2, 3], [30, 31, 32, 33, 40], cells=cells, first_takes_context=False,
                               first_residual_layer=2, classifier_weight_id=50, classifier_bias_id=51)
    ex = E.StreamExecutor([layer], model_type="GNMT", device=0)
    state_d = state.to(DEV)
    _blobs(ex, b100=state_d, b50=Wc.to(DEV), b51=bc.to(DEV))
    ref = state.clone()
    enc_buf = torch.zeros(1, S, H, dtype=torch.float16, device=DEV)     # the same blob is refilled for the next sentence
    ex.update_blob(3, DataType.TENSOR, enc_buf)
    for sentence in range(2):
        enc = torch.randn(1, S, H, generator=g).half()
        enc_buf.copy_(enc.to(DEV))
        ex.same_sentence = False
        for token in range(3):
            x = torch.randn(1, 1, H, generator=g).half()
            att = torch.softmax(torch.randn(1, 1, S, generator=g), -1).half()
            _blobs(ex, b1=x.to(DEV), b2=att.to(DEV))
            ex.inference()
            ex.same_sentence = True
            ctx = torch.bmm(att.float(), enc.float()).half()
            inp = x
            for k in range(4):
                full = inp if k == 0 else torch.cat([inp, ctx], 2)
                y, hn, cn = torch.lstm(full, (ref[2 * k:2 * k + 1], ref[2 * k + 1:2 * k + 2]), params[k], True, 1, 0.0, False, False, False)
                ref[2 * k], ref[2 * k + 1] = hn[0], cn[0]
                inp = y + inp if k >= 2 else y
                assert maxabs(ex.find_blob(30 + k)[1], inp) <= TOL_LSTM, (sentence, token, k)
            logits = torch.addmm(bc, inp.view(1, H), Wc.t())
            got = ex.find_blob(40)[1]
            assert list(got.shape) == [1, V] and maxabs(got, logits) <= TOL_LSTM
            assert maxabs(state_d, ref) <= TOL_LSTM


@pytest.mark.gpu
def test_gnmt_attention_context_lands_in_three_concatenation_buffers(ops):
    """aten_ops_executor.cpp:680-737: y[1,1,1024] = p[1,1,50] . enc[1,50,1024] at offset 1024 of three buffers."""
    g = torch.Generator().manual_seed(8)
    p_att, enc = torch.rand(1, 1, 50, generator=g).half(), torch.randn(1, 50, 1024, generator=g).half()
    ex = E.StreamExecutor([], model_type="GNMT", device=0)
    cats = [torch.full((1, 1, 2048), float(i + 1), dtype=torch.float16, device=DEV) for i in range(3)]
    _blobs(ex, b0=p_att.to(DEV), b1=enc.to(DEV), b60=cats[0], b61=cats[1], b62=cats[2])
    E.execute_aten_bmm(E.AtenBmmLayer(LayerType.ATENBMM, 0, [0, 1], [5], cat_mem_ids=[60, 61, 62]), ex)
    want = oracle.gemv_vm(p_att.numpy().reshape(-1), enc.numpy().reshape(50, 1024), None)
    out = ex.find_blob(5)[1]
    assert list(out.shape) == [1, 1, 1024] and out.data_ptr() == cats[0].data_ptr() + 2048
    for i, c in enumerate(cats):
        assert maxabs(c[..., 1024:], want) <= 4e-3 and bool((c[..., :1024] == float(i + 1)).all())
    assert torch.equal(cats[0][..., 1024:], cats[1][..., 1024:]) and torch.equal(cats[0][..., 1024:], cats[2][..., 1024:])
