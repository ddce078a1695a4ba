"""Executor-level entry points of the hot path: layer records, the blob store and the `execute*` functions.

Mirrors, for the layer types on this path only, what the reference's interpreter does per layer
(paths relative to the reference tree):

    StreamExecutor.update_blob / find_blob   runtime/source/executor/stream_executor.cpp:260-280
    execute_aten_addmm[_with_stream]         runtime/source/executor/op_executor/aten_ops_executor.cpp:181-254
    execute_aten_matmul[_with_stream]        aten_ops_executor.cpp:2488-2525
    execute_aten_linear                      aten_ops_executor.cpp:2029-2059
    execute_aten_lstm1 / execute_aten_lstm2  aten_ops_executor.cpp:2135-2399; the GNMT decoder's state and attention
                                             buffers (:2238-2302) are written in place, as the reference's MIOpen
                                             route does (miopen_ops_executor.cpp:170-228)
    execute_aten_add / execute_aten_bmm      aten_ops_executor.cpp:43-179, 668-747 (custom-kernel branches)
    execute_multi_stream                     runtime/source/executor/op_executor/stream_ops_executor.cpp:27-50
    StreamExecutor.inference                 the dispatch loop, stream_executor.cpp:153-186, for these layer types

A layer attribute that holds the reference's "unset" sentinel (ir/include/common/utils.hpp:19-23: INT32_MAX for
int, INT64_MIN for int64, DBL_MAX for double) is taken from the next input blob instead, in the reference's order.
Tensors are torch tensors on the GPU; the arithmetic is in libpimhip.so via pimaicompiler_amd.ops.
"""
import enum
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch

from . import ops
from .ops import NNRuntimeException

INT32_MAX = 2 ** 31 - 1
INT64_MIN = -2 ** 63
DBL_MAX = 1.7976931348623157e308


def is_default_int(v):
    return v == INT32_MAX


def is_default_int64(v):
    return v == INT64_MIN


def is_default_double(v):
    return abs(v - DBL_MAX) <= 2.220446049250313e-16


class LayerType(enum.Enum):
    """The LayerType values of ir/include/types.h that reach this path."""
    ATENADD = "aten::add"
    ATENADDMM = "aten::addmm"
    ATENBMM = "aten::bmm"
    ATENLINEAR = "aten::linear"
    ATENLSTM1 = "aten::lstm1"
    ATENLSTM2 = "aten::lstm2"
    ATENMATMUL = "aten::matmul"
    MULTISTREAM = "multi_stream"
    DECODERSTEP = "pimhip::decoder_step"    # no counterpart in ir/include/types.h: see DecoderStepLayer


class DataType(enum.Enum):
    UNDEFINED = 0
    TENSOR = 1
    INT64 = 2
    FLOAT64 = 3
    LIST = 4
    NONE = 5


@dataclass
class NNLayer:
    """ir::NNLayer reduced to what the executors read: type, id (= position), input / output STensor ids."""
    type: LayerType
    id: int = 0
    in_stensor_ids: List[int] = field(default_factory=list)
    out_stensor_ids: List[int] = field(default_factory=list)
    name: str = ""


@dataclass
class AtenAddmmLayer(NNLayer):          # ir/include/layers/aten_addmm_layer.h
    act_type: str = "none"              # "none" | "aten::relu" | "aten::max", set by FuseActivation


@dataclass
class AtenLinearLayer(NNLayer):         # ir/include/layers/aten_linear_layer.h
    weights: List[torch.Tensor] = field(default_factory=list)        # host tensors until the model is preloaded
    biases: List[torch.Tensor] = field(default_factory=list)
    weight_ids: List[int] = field(default_factory=list)
    bias_ids: List[int] = field(default_factory=list)


@dataclass
class AtenLSTM1Layer(NNLayer):          # ir/include/layers/aten_lstm1_layer.h
    has_biases: int = INT32_MAX
    num_layers: int = INT64_MIN
    dropout: float = DBL_MAX
    train: int = INT32_MAX
    bidirectional: int = INT32_MAX
    batch_first: int = INT32_MAX
    weights: List[torch.Tensor] = field(default_factory=list)        # per layer x direction: w_ih, w_hh
    biases: List[torch.Tensor] = field(default_factory=list)         # per layer x direction: b_ih, b_hh
    weight_ids: List[int] = field(default_factory=list)
    bias_ids: List[int] = field(default_factory=list)
    param_vector: List[torch.Tensor] = field(default_factory=list)   # LibTorch order, built at model-build time
    # GNMT decoder (aten_lstm1_layer.h: match_custom_opt_, custom_opt_number_, custom_cat_mem_id_): layer number k of the
    # decoder keeps (h, c) in rows 2k, 2k+1 of the state buffer blob `custom_cat_mem_id`; layers 0 and 1 also put their
    # output into the first H columns of the attention concatenation buffer, whose blob id the reference looks up
    # through the following cat layer (aten_ops_executor.cpp:2277-2282) and this record carries directly.
    match_custom_opt: bool = False
    custom_opt_number: int = 0
    custom_cat_mem_id: int = -1
    output_cat_mem_id: int = -1
    # Not in the reference's record: set by a graph rewrite that has folded the aten::add layers of a residual stack
    # (out = lstm(in) + in from this layer of the record on) into it; negative = no such sums.
    first_residual_layer: int = -1


@dataclass
class AtenLSTM2Layer(NNLayer):          # ir/include/layers/aten_lstm2_layer.h
    has_biases: int = INT32_MAX
    num_layers: int = INT64_MIN
    dropout: float = DBL_MAX
    train: int = INT32_MAX
    bidirectional: int = INT32_MAX
    weights: List[torch.Tensor] = field(default_factory=list)
    biases: List[torch.Tensor] = field(default_factory=list)
    weight_ids: List[int] = field(default_factory=list)
    bias_ids: List[int] = field(default_factory=list)
    param_vector: List[torch.Tensor] = field(default_factory=list)


@dataclass
class AtenAddLayer(NNLayer):            # ir/include/layers/aten_add_layer.h
    alpha: int = INT64_MIN
    # GNMT: blob id of the concatenation buffer whose first n elements receive the sum of the outputs of decoder layers
    # 2 and 1 (the reference derives both the condition and the id from the neighbouring layers,
    # aten_ops_executor.cpp:129-148); -1: none.
    cat_mem_id: int = -1


@dataclass
class AtenBmmLayer(NNLayer):            # ir/include/layers/aten_bmm_layer.h
    # GNMT: the blob ids of the three concatenation buffers whose second half receives the attention context.  The
    # reference finds them by walking the graph from this layer (aten_ops_executor.cpp:680-705).
    cat_mem_ids: List[int] = field(default_factory=list)


@dataclass
class DecoderStepLayer(NNLayer):
    """No counterpart in the reference's IR: the per-token chain of its GNMT decoder, which its interpreter runs as
    separate layers (executeAtenLSTM1 per cell with the state in the buffer blob, executeAtenBmm for the context,
    executeAtenAdd for the residual sums, executeAtenAddmm for the classifier), as ONE record that runs as one launch.

    cells: the AtenLSTM1Layer records of the chain, bottom to top, as the model builder leaves them (param_vector set,
    custom_opt_number = k and custom_cat_mem_id = the state buffer blob: rows 2k, 2k+1 hold (h, c) of cell k and are
    updated in place).  in_stensor_ids: [x, attention weights, encoder outputs], or [x, context] when the context is
    computed elsewhere.  out_stensor_ids: one id per cell for its output (y, or y + input from first_residual_layer on),
    then the id of the logits when classifier ids are given.  The encoder outputs are projected once per sentence: set
    StreamExecutor.same_sentence while the blob keeps the sentence it had at the previous token."""
    cells: List[AtenLSTM1Layer] = field(default_factory=list)
    first_takes_context: bool = False
    first_residual_layer: int = 2
    classifier_weight_id: int = -1      # blob ids of W [vocab, H] and b [vocab] (or -1)
    classifier_bias_id: int = -1


@dataclass
class MultiStreamLayer(NNLayer):        # ir/include/layers/multi_stream_layer.h
    layers: List[NNLayer] = field(default_factory=list)

    @property
    def layer_num(self):
        return len(self.layers)


class StreamExecutor:
    """Blob store + streams + cursor, as far as the hot-path executors use them (stream_executor.h:30-179)."""

    def __init__(self, layers: Optional[List[NNLayer]] = None, model_type: str = "", device=0, grouped_multi_stream=False):
        self.layers = layers or []
        self.model_type = model_type
        self.device = device
        self.global_blobs: Dict[int, Any] = {}     # id -> (DataType, value)
        self.cursor = 0
        self.streams: List[torch.cuda.Stream] = []
        # True: sibling GEMVs of a MULTISTREAM layer go out as one grouped launch instead of one stream each.
        self.grouped_multi_stream = grouped_multi_stream
        # True while the encoder outputs a DecoderStepLayer attends over are those of its previous call (their projection
        # is then not computed again); a driver sets it after the first token of a sentence and clears it for the next one.
        self.same_sentence = False
        ops.initialize(device)
        width = max([l.layer_num for l in self.layers if isinstance(l, MultiStreamLayer)], default=0)
        self.set_streams(width)

    # stream_executor.h:124-133
    def set_streams(self, n):
        with torch.cuda.device(self.device):
            self.streams = [torch.cuda.Stream() for _ in range(n)]

    def get_streams(self):
        return self.streams

    def update_blob(self, blob_id, dtype, value):
        self.global_blobs[blob_id] = (dtype, value)

    def preload_constants(self, constants):
        """The prim::Constant pass of preProcess (stream_executor.cpp:59-134, prim_ops_executor.cpp:101): constant tensors
        go to the GPU and into the blob store once.

        A 2-D constant that the graph uses only as the right operand of addmm / matmul (y = x . A, the I_X_W order, A
        stored [in, out]) is kept TRANSPOSED in memory behind the same logical shape and values: every later product
        then streams contiguous rows with the W_X_I kernel instead of the column-sliced I_X_W one, at no cost per call,
        where the reference makes such operands contiguous on every call (aten_ops.cpp:630-632).  Returns the ids whose
        layout was changed."""
        right, other = set(), set()
        for layer in _flatten(self.layers):
            ids = list(layer.in_stensor_ids)
            if layer.type == LayerType.ATENADDMM and len(ids) >= 3:
                right.add(ids[2])
                other.update(ids[:2])
            elif layer.type == LayerType.ATENMATMUL and len(ids) >= 2:
                right.add(ids[1])
                other.add(ids[0])
            else:
                other.update(ids)
        relaid = []
        dev = torch.device("cuda", self.device) if isinstance(self.device, int) else self.device
        for blob_id, t in constants.items():
            t = t.to(dev)
            if blob_id in right and blob_id not in other and t.dim() == 2 and t.dtype == torch.float16 and t.is_contiguous() \
                    and min(t.shape) > 1:
                t = t.t().contiguous().t()   # [in, out] with strides (1, in): the same values, rows of A^T contiguous
                relaid.append(blob_id)
            self.update_blob(blob_id, DataType.TENSOR, t)
        return relaid

    def find_blob(self, blob_id):
        return self.global_blobs.get(blob_id, (DataType.UNDEFINED, None))

    def check_valid_blob_id(self, blob_id):
        return blob_id in self.global_blobs

    def set_cursor(self, c):
        self.cursor = c

    def inference(self, executors=None):
        """The dispatch loop (stream_executor.cpp:153-186) over self.layers; MULTISTREAM sets the cursor itself."""
        table = executors or OP_EXECUTORS
        self.cursor = 0
        while self.cursor < len(self.layers):
            layer = self.layers[self.cursor]
            table[layer.type](layer, self)
            self.cursor += 1


class ModelBuilder:
    """Weight preload for the layers of this path (runtime/source/builder/model_builder.cpp:18-224).

    pre_process finds the first free blob id; preload_model moves each LINEAR / LSTM layer's weights and biases to the
    GPU under fresh ids, and for an LSTM whose flags are all set builds the LibTorch-ordered parameter vector.  Where
    the reference then packs a MIOpen weight buffer (reArangeLstmWeights, :226-319), this build prepares the recurrence
    plan (bias sums, projection and exchange buffers) for the layer once, so no call allocates later.
    """

    def __init__(self, device=0):
        self.device = torch.device("cuda", device) if isinstance(device, int) else torch.device(device)
        self.preload_id = 0
        self.preloaded_data_container: Dict[int, Any] = {}

    def pre_process(self, layers):
        for layer in _flatten(layers):
            for i in layer.out_stensor_ids:
                self.preload_id = max(self.preload_id, i)
        self.preload_id += 1

    def load_weight_and_bias(self, weight_data, bias_data):
        ids = ([], [])
        for dst, group in zip(ids, (weight_data, bias_data)):
            for t in group:
                self.preloaded_data_container[self.preload_id] = (DataType.TENSOR, t.to(self.device))
                dst.append(self.preload_id)
                self.preload_id += 1
        return ids

    @staticmethod
    def feasible_for_lstm_weight_process(layer):
        unset = [is_default_int(layer.has_biases), is_default_int64(layer.num_layers), is_default_double(layer.dropout),
                 is_default_int(layer.train), is_default_int(layer.bidirectional)]
        if isinstance(layer, AtenLSTM1Layer):
            unset.append(is_default_int(layer.batch_first))
        return not any(unset)

    def build_lstm_parameter_vector(self, layer):
        assert layer.bidirectional in (0, 1)
        params = []
        for i in range(layer.num_layers * (layer.bidirectional + 1)):
            params.append(self.preloaded_data_container[layer.weight_ids[2 * i]][1])
            params.append(self.preloaded_data_container[layer.weight_ids[2 * i + 1]][1])
            if layer.has_biases:
                params.append(self.preloaded_data_container[layer.bias_ids[2 * i]][1])
                params.append(self.preloaded_data_container[layer.bias_ids[2 * i + 1]][1])
        layer.param_vector = params

    def preload_model(self, layers, lstm_seq_len=64):
        for layer in _flatten(layers):
            if layer.type in (LayerType.ATENLSTM1, LayerType.ATENLSTM2, LayerType.ATENLINEAR):
                if not layer.weights:
                    continue
                layer.weight_ids, layer.bias_ids = self.load_weight_and_bias(layer.weights, layer.biases)
                if layer.type == LayerType.ATENLINEAR:
                    continue
                if not self.feasible_for_lstm_weight_process(layer):
                    raise NNRuntimeException(f"Failed to pre-process weights for: {layer.name}")
                self.build_lstm_parameter_vector(layer)
                ops.prepare_lstm(layer.param_vector, bool(layer.has_biases), layer.num_layers, bool(layer.bidirectional),
                                 lstm_seq_len)

    def build(self, layers, **executor_args):
        """pre_process + preload_model + a StreamExecutor whose blob store starts from the preloaded container."""
        self.pre_process(layers)
        self.preload_model(layers)
        ex = StreamExecutor(layers, device=self.device.index or 0, **executor_args)
        ex.global_blobs.update(self.preloaded_data_container)
        return ex


def _flatten(layers):
    for layer in layers:
        yield layer
        if isinstance(layer, MultiStreamLayer):
            yield from layer.layers


def _tensor(executor, blob_id, what):
    dtype, v = executor.find_blob(blob_id)
    if not isinstance(v, torch.Tensor):
        raise NNRuntimeException(f"{what}: blob {blob_id} is not a tensor ({dtype})")
    return v


# ---- GEMV family ---------------------------------------------------------------------------------------------------
def execute_aten_addmm_with_stream(layer, executor, stream):
    ids = layer.in_stensor_ids
    _, iv_self = executor.find_blob(ids[0])
    mat1, mat2 = _tensor(executor, ids[1], "addmm mat1"), _tensor(executor, ids[2], "addmm mat2")
    alpha = beta = 1
    if len(ids) == 5:
        beta, alpha = int(executor.find_blob(ids[3])[1]), int(executor.find_blob(ids[4])[1])
    if iv_self is None:
        out = ops.custom_aten_matmul(mat1, mat2, stream=stream)
    else:
        out = ops.custom_aten_addmm(layer.act_type, iv_self, mat1, mat2, beta, alpha, stream=stream)
    executor.update_blob(layer.out_stensor_ids[0], DataType.TENSOR, out)


def execute_aten_addmm(layer, executor):
    execute_aten_addmm_with_stream(layer, executor, None)


def execute_aten_matmul_with_stream(layer, executor, stream):
    ids = layer.in_stensor_ids
    out = ops.custom_aten_matmul(_tensor(executor, ids[0], "matmul self"), _tensor(executor, ids[1], "matmul other"), stream=stream)
    executor.update_blob(layer.out_stensor_ids[0], DataType.TENSOR, out)


def execute_aten_matmul(layer, executor):
    execute_aten_matmul_with_stream(layer, executor, None)


def execute_aten_linear(layer, executor):
    x = _tensor(executor, layer.in_stensor_ids[0], "linear input")
    w = _tensor(executor, layer.weight_ids[0], "linear weight")
    b = _tensor(executor, layer.bias_ids[0], "linear bias") if layer.bias_ids else None
    executor.update_blob(layer.out_stensor_ids[0], DataType.TENSOR, ops.aten_linear(x, w, b))


def execute_multi_stream(layer, executor):
    subs = layer.layers
    for sub in subs:
        if sub.type not in (LayerType.ATENADDMM, LayerType.ATENMATMUL):
            raise NNRuntimeException(f"Unsupported layer type: {sub.type.value} found in multi-stream execution.")
    if executor.grouped_multi_stream and _groupable(subs, executor):
        _execute_grouped(subs, executor)
    else:
        streams = executor.get_streams()
        cur = torch.cuda.current_stream()
        for i, sub in enumerate(subs):
            streams[i].wait_stream(cur)   # the siblings' inputs were produced on the current stream
            with torch.cuda.stream(streams[i]):
                if sub.type == LayerType.ATENADDMM:
                    execute_aten_addmm_with_stream(sub, executor, streams[i])
                else:
                    execute_aten_matmul_with_stream(sub, executor, streams[i])
        # The reference's streams are ordered against its null stream implicitly; these are not, so the issuing
        # stream waits (on the GPU, not the host) for the siblings before any consumer is enqueued.
        for i in range(len(subs)):
            cur.wait_stream(streams[i])
    # The graph keeps the duplicated sub-layers right after this one; the main loop's increment skips the last of them.
    executor.set_cursor(layer.id + layer.layer_num)


def _mv_operands(sub, executor):
    """(x, W, bias, act) if the sub-layer is an MV product W[out,in] . x[in,1] on dense 2-D weights, else None."""
    ids = sub.in_stensor_ids
    if sub.type == LayerType.ATENADDMM:
        bias, w, x, act = executor.find_blob(ids[0])[1], executor.find_blob(ids[1])[1], executor.find_blob(ids[2])[1], sub.act_type
        if len(ids) == 5:
            return None
    else:
        bias, w, x, act = None, executor.find_blob(ids[0])[1], executor.find_blob(ids[1])[1], "none"
    if not (isinstance(w, torch.Tensor) and isinstance(x, torch.Tensor)) or w.dim() != 2 or not w.is_contiguous():
        return None
    if x.dim() != 2 or x.size(1) != 1 or x.size(0) != w.size(1) or w.size(1) % 8 != 0:
        return None
    if bias is not None and not (isinstance(bias, torch.Tensor) and bias.numel() == w.size(0)):
        return None
    if any(t is not None and (t.dtype != torch.float16 or not t.is_cuda) for t in (x, w, bias)):
        return None
    if act not in ("none", "aten::relu"):
        act = "none"            # only ReLU is an activation for the kernels (aten_ops.cpp:641-643)
    return x, w, bias, act


def _groupable(subs, executor):
    return all(_mv_operands(s, executor) is not None for s in subs)


def _execute_grouped(subs, executor):
    quad = [_mv_operands(s, executor) for s in subs]
    outs = ops.execute_gemv_group([q[0] for q in quad], [q[1] for q in quad], [q[2] for q in quad], [q[3] for q in quad])
    for s, o in zip(subs, outs):
        executor.update_blob(s.out_stensor_ids[0], DataType.TENSOR, o.view(-1, 1))


# ---- LSTM ----------------------------------------------------------------------------------------------------------
def _lstm_flags(layer, executor, in_id, with_batch_first):
    ids = layer.in_stensor_ids
    # A TensorList of parameters may sit in the inputs; the layer's own param_vector is used instead (:2162-2168).
    if len(ids) > in_id and isinstance(executor.find_blob(ids[in_id])[1], (list, tuple)):
        in_id += 1

    def take(value, is_default):
        nonlocal in_id
        if is_default(value):
            value = executor.find_blob(ids[in_id])[1]
            in_id += 1
        return value

    has_biases = int(take(layer.has_biases, is_default_int))
    num_layers = int(take(layer.num_layers, is_default_int64))
    dropout = float(take(layer.dropout, is_default_double))
    train = int(take(layer.train, is_default_int))
    bidirectional = int(take(layer.bidirectional, is_default_int))
    batch_first = int(take(layer.batch_first, is_default_int)) if with_batch_first else 0
    return has_biases, num_layers, dropout, train, bidirectional, batch_first


def _unique_in_order(ids):
    out = []
    for i in ids:
        if not out or out[-1] != i:
            out.append(i)
    return out


def _gnmt_lstm_destinations(layer, executor, x, out_ids, hidden, num_layers, bidirectional, batch_first):
    """Where a GNMT decoder LSTM writes (y, hy, cy), or None for fresh tensors.

    The reference's LibTorch route rebuilds the concatenation tensors with slice + cat after the call
    (aten_ops_executor.cpp:2238-2302); its MIOpen route hands the kernel pointers into them
    (miopen_ops_executor.cpp:170-228).  The latter is what happens here: the step kernel stores straight into the
    consumers' buffers and no copy is made."""
    if executor.model_type != "GNMT" or num_layers != 1 or bidirectional:
        return None
    seq_len = x.size(1) if batch_first else x.size(0)
    prev = [executor.find_blob(i)[1] for i in out_ids]
    if seq_len == 1 and all(isinstance(t, torch.Tensor) and t.is_contiguous() and t.dtype == torch.float16 for t in prev) and \
            [t.numel() for t in prev] == [hidden, hidden, hidden]:
        return tuple(prev)                       # the buffers of the previous decoder step are written again
    if not layer.match_custom_opt:
        return None
    k = layer.custom_opt_number
    state = executor.find_blob(layer.custom_cat_mem_id)[1]
    if not isinstance(state, torch.Tensor) or not state.is_contiguous() or state.numel() < (2 * k + 2) * hidden:
        raise NNRuntimeException(f"blob {layer.custom_cat_mem_id} cannot hold the state of decoder layer {k}")
    flat = state.view(-1)
    hy = flat[2 * k * hidden:(2 * k + 1) * hidden].view(1, 1, hidden)
    cy = flat[(2 * k + 1) * hidden:(2 * k + 2) * hidden].view(1, 1, hidden)
    y = None
    if k in (0, 1) and layer.output_cat_mem_id >= 0 and seq_len == 1:
        cat = executor.find_blob(layer.output_cat_mem_id)[1]
        if isinstance(cat, torch.Tensor) and cat.is_contiguous() and cat.numel() >= hidden:
            y = cat.view(-1)[:hidden].view(1, 1, hidden)
    if y is None:
        y = torch.empty((seq_len, hidden), dtype=torch.float16, device=x.device)
    return y, hy, cy


def execute_aten_lstm1(layer, executor):
    ids = layer.in_stensor_ids
    x = _tensor(executor, ids[0], "lstm input")
    hx = executor.find_blob(ids[1])[1]
    if not isinstance(hx, (list, tuple)) or len(hx) != 2:
        raise NNRuntimeException("lstm hx must be a TensorList (h0, c0)")
    has_biases, num_layers, dropout, train, bidirectional, batch_first = _lstm_flags(layer, executor, 2, True)
    out_ids = _unique_in_order(layer.out_stensor_ids)
    if len(out_ids) != 3:
        raise NNRuntimeException("lstm needs three output ids")
    out = _gnmt_lstm_destinations(layer, executor, x, out_ids, hx[0].size(-1), num_layers, bool(bidirectional), bool(batch_first))
    y, hy, cy = ops.aten_lstm1(x, tuple(hx), layer.param_vector, bool(has_biases), num_layers, dropout, bool(train),
                               bool(bidirectional), bool(batch_first), out=out,
                               first_residual_layer=layer.first_residual_layer if layer.first_residual_layer >= 0 else None)
    for i, v in zip(out_ids, (y, hy, cy)):
        executor.update_blob(i, DataType.TENSOR, v)


def execute_aten_lstm2(layer, executor):
    ids = layer.in_stensor_ids
    data = _tensor(executor, ids[0], "lstm data")
    batch_sizes = _tensor(executor, ids[1], "lstm batch_sizes")
    hx = executor.find_blob(ids[2])[1]
    if not isinstance(hx, (list, tuple)) or len(hx) != 2:
        raise NNRuntimeException("lstm hx must be a TensorList (h0, c0)")
    has_biases, num_layers, dropout, train, bidirectional, _ = _lstm_flags(layer, executor, 3, False)
    y, hy, cy = ops.aten_lstm2(data, batch_sizes, tuple(hx), layer.param_vector, bool(has_biases), num_layers, dropout,
                               bool(train), bool(bidirectional))
    out_ids = _unique_in_order(layer.out_stensor_ids)
    if len(out_ids) != 3:
        raise NNRuntimeException("lstm needs three output ids")
    for i, v in zip(out_ids, (y, hy, cy)):
        executor.update_blob(i, DataType.TENSOR, v)


# ---- the decoder loop's custom-kernel users ---------------------------------------------------------------------------
def execute_aten_add(layer, executor):
    ids = layer.in_stensor_ids
    a, b = executor.find_blob(ids[0])[1], executor.find_blob(ids[1])[1]
    alpha = layer.alpha
    if is_default_int64(alpha):
        # As written in the reference (aten_ops_executor.cpp:57-70): with three inputs it asks whether blob id 2 (the
        # input *index*, not in_stensor_id[2]) is valid before reading the third input.
        alpha = int(executor.find_blob(ids[2])[1]) if len(ids) == 3 and executor.check_valid_blob_id(2) else 1
    if isinstance(a, int) and isinstance(b, int):
        executor.update_blob(layer.out_stensor_ids[0], DataType.INT64, a + b * alpha)
        return
    if not isinstance(a, torch.Tensor):
        raise NNRuntimeException("Unsupported input type for aten::add")
    if isinstance(b, torch.Tensor) and a.dtype == torch.float16 and ops.custom_add_applies(a, b):
        # The custom kernel writes the sum over `self` (C = A, aten_ops_executor.cpp:121-123), or, for the GNMT
        # residual add, into the head of a concatenation buffer; alpha is ignored by the kernel (custom_ops.h:415-433).
        dst = a if a.is_contiguous() else a.contiguous()
        if executor.model_type == "GNMT" and layer.cat_mem_id >= 0:
            cat = _tensor(executor, layer.cat_mem_id, "add concatenation buffer")
            if not cat.is_contiguous() or cat.numel() < a.numel():
                raise NNRuntimeException(f"blob {layer.cat_mem_id} cannot take the sum")
            dst = cat.view(-1)[:a.numel()].view(a.shape)
        out = ops.aten_add(a, b, alpha=alpha, out=dst)
    else:
        out = torch.add(a, b, alpha=alpha)
    executor.update_blob(layer.out_stensor_ids[0], DataType.TENSOR, out)


def execute_aten_bmm(layer, executor):
    ids = layer.in_stensor_ids
    a, b = _tensor(executor, ids[0], "bmm self"), _tensor(executor, ids[1], "bmm other")
    outs = None
    cat_ids = getattr(layer, "cat_mem_ids", [])
    if executor.model_type == "GNMT" and cat_ids:
        # y goes to elements [n, 2n) of every concatenation buffer: one launch with several destinations replaces the
        # reference's kernel plus two device copies (aten_ops_executor.cpp:694-737).
        n = b.size(-1)
        outs = []
        for cid in cat_ids:
            cat = _tensor(executor, cid, "bmm concatenation buffer")
            if not cat.is_contiguous() or cat.numel() < 2 * n:
                raise NNRuntimeException(f"blob {cid} cannot take the attention context at offset {n}")
            outs.append(cat.view(-1)[n:2 * n])
    out = ops.aten_bmm(a, b, outs=outs)
    if outs:
        out = out.view(1, 1, -1)
    executor.update_blob(layer.out_stensor_ids[0], DataType.TENSOR, out)


def execute_decoder_step(layer, executor):
    """One decoder token as one launch (ops.DecoderPlan / pimhip_decoder_step).  The plan is made on the first call and kept
    on the record; the cells' states are read from and written to their rows of the state buffer blob."""
    cells = layer.cells
    n = len(cells)
    if n < 1 or any(len(c.param_vector) != 4 for c in cells):
        raise NNRuntimeException("a decoder step needs its cells' parameter vectors (w_ih, w_hh, b_ih, b_hh per cell)")
    ids = layer.in_stensor_ids
    x = _tensor(executor, ids[0], "decoder step input")
    H = cells[0].param_vector[1].size(1)
    plan = getattr(layer, "_plan", None)
    if plan is None:
        cls = None
        if layer.classifier_weight_id >= 0:
            cls = (_tensor(executor, layer.classifier_weight_id, "classifier weight"),
                   _tensor(executor, layer.classifier_bias_id, "classifier bias") if layer.classifier_bias_id >= 0 else None)
        plan = ops.DecoderPlan([t for c in cells for t in c.param_vector], True, n, first_takes_context=layer.first_takes_context,
                               first_residual_layer=layer.first_residual_layer, classifier=cls)
        layer._plan = plan
    att = enc = ctx = None
    if len(ids) >= 3:
        att, enc = _tensor(executor, ids[1], "attention weights"), _tensor(executor, ids[2], "encoder outputs")
        if not (getattr(executor, "same_sentence", False) and plan._enc is not None):
            plan.set_encoder(enc.reshape(-1, H).contiguous())
    elif len(ids) == 2:
        ctx = _tensor(executor, ids[1], "context")
    h_prev, c_prev = [], []
    for c in cells:
        state = _tensor(executor, c.custom_cat_mem_id, "decoder state buffer")
        k = c.custom_opt_number
        if not state.is_contiguous() or state.numel() < (2 * k + 2) * H:
            raise NNRuntimeException(f"blob {c.custom_cat_mem_id} cannot hold the state of decoder cell {k}")
        flat = state.view(-1)
        h_prev.append(flat[2 * k * H:(2 * k + 1) * H])
        c_prev.append(flat[(2 * k + 1) * H:(2 * k + 2) * H])
    outs = [torch.empty(1, 1, H, dtype=torch.float16, device=x.device) for _ in range(n)]
    logits = torch.empty(1, plan.vocab, dtype=torch.float16, device=x.device) if plan.vocab else None
    flat1 = lambda t: t.contiguous().view(-1)  # noqa: E731
    step = plan.bind(flat1(x), h_prev, c_prev, att=flat1(att) if att is not None else None, ctx=flat1(ctx) if ctx is not None else None,
                     outs=[o.view(-1) for o in outs], logits=logits.view(-1) if logits is not None else None)   # state in place
    step()
    for k in range(n):
        executor.update_blob(layer.out_stensor_ids[k], DataType.TENSOR, outs[k])
    if logits is not None:
        executor.update_blob(layer.out_stensor_ids[n], DataType.TENSOR, logits)


# registerOp (stream_executor.cpp:433-576) for the layer types of this path
OP_EXECUTORS = {
    LayerType.DECODERSTEP: execute_decoder_step,
    LayerType.ATENADD: execute_aten_add,
    LayerType.ATENADDMM: execute_aten_addmm,
    LayerType.ATENBMM: execute_aten_bmm,
    LayerType.ATENLINEAR: execute_aten_linear,
    LayerType.ATENLSTM1: execute_aten_lstm1,
    LayerType.ATENLSTM2: execute_aten_lstm2,
    LayerType.ATENMATMUL: execute_aten_matmul,
    LayerType.MULTISTREAM: execute_multi_stream,
}
