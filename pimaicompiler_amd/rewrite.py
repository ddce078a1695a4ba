"""The graph rewrites that decide which shapes and operand orders reach the GEMV kernels, on a minimal op list.

The reference does this in six passes over its IR (compiler/source/frontend/optimizer/, run in this order by
pass_manager.cpp:36-82):

    convert_linear_to_addmm   linear(x, W, b)              -> addmm(b, x, W)                 convert_linear_to_addmm.cpp:37-65
    remove_cat_for_addmm      addmm(b, cat([f, g]), W)     -> addmm(addmm(b, f, W1), g, W2)  remove_cat_for_addmm.cpp:46-191
    swap_addmm_inputs         addmm(b, x, Wconst)          -> T(addmm(b, Wconst, T(x)))      swap_addmm_inputs.cpp:36-99
    swap_matmul_inputs        matmul(x, Wconst2d)          -> T(matmul(Wconst2d, T(x)))      swap_matmul_inputs.cpp:42-106
    fuse_activation           relu(T(addmm(...)))          -> T(addmm(..., act="aten::relu")) fuse_activation.cpp:73-107

`apply_reference_passes` restates them on `Graph` below, wiring for wiring (the weight constant of a linear is
[out, in], so convert + swap together compute x . W^T + b as W . x^T, the MV order).  `lower_to_hot_path` then does
what the reference leaves to run time: every  T -> addmm/matmul(Wconst, .) -> T  sandwich becomes ONE fused
`gemv` op on the weight's own row-major bytes (bias and ReLU in the epilogue), so the two transposes and the
`.contiguous()` copies of customAtenAddmm (runtime/source/executor/op_executor/aten_ops.cpp:630-632, 663-665)
disappear.  `multi_stream_execution` restates the middle-end pass of the same name
(compiler/source/middlend/optimizer/stream_execution/multi_stream_execution.cpp:20-290): sibling products that feed
one join and hang off one common start are collected into a single `multi_stream` op, which runs as ONE grouped launch
here where the reference gives each sibling its own stream.  `execute` runs a graph through the operator layer
(pimaicompiler_amd.ops) on the GPU.

`gemv_over_cat` is an alternative to remove_cat_for_addmm: the product over cat([f, g]) stays ONE op on the whole weight
that reads f and g where they lie (one launch instead of the reference's two dependent ones).

`fuse_decoder_step` has no counterpart in the reference: it collects the per-token chain of the GNMT decoder — the
seq_len-1 `aten::lstm` cells that read cat(previous output, context), the residual `aten::add`s, the attention `aten::bmm`
and the classifier — which the reference's interpreter runs operator by operator (executeAtenLSTM1 / executeAtenBmm /
executeAtenAdd / executeAtenAddmm, runtime/source/executor/op_executor/aten_ops_executor.cpp:2135-2307, 668-747, 43-179,
181-216), into one `pimhip::decoder_step` op, which `execute` runs as ONE launch (ops.DecoderPlan).

`fuse_lstm_stack` has no counterpart either: consecutive one-layer `aten::lstm` ops over a whole sequence, each reading
only the sequence the one before wrote (the GNMT encoder's layers above the bidirectional one, which the reference runs
as one executeAtenLSTM1 call each), become ONE `aten::lstm` with `num_layers = n`, LibTorch's own multi-layer form, so
that the layers run as a pipeline in one launch (layer k starts step t as soon as layer k - 1 has finished it) instead
of one after the other.

remove_cat_for_addmm is restated for any split point; the reference hard-codes the RNNT joint shapes
([1,1024] + [1,320] against a [512,1344] weight, compiler/include/frontend/optimizer/remove_cat_for_addmm.h:77-79).
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


@dataclass
class Op:
    type: str                 # "aten::linear", "aten::addmm", "aten::matmul", "aten::transpose", "aten::relu",
                              # "aten::cat", "prim::ListConstruct", "prim::Constant", "pimhip::gemv"
    inputs: List[int]
    outputs: List[int]
    attrs: Dict = field(default_factory=dict)


@dataclass
class Graph:
    ops: List[Op]
    inputs: List[int]
    outputs: List[int]
    constants: Dict[int, Optional[torch.Tensor]] = field(default_factory=dict)   # tensor id -> value (None = None)
    next_id: int = 0

    def new_id(self):
        ids = [i for op in self.ops for i in op.inputs + op.outputs] + self.inputs + self.outputs + list(self.constants)
        self.next_id = max([self.next_id] + [i + 1 for i in ids])
        self.next_id += 1
        return self.next_id - 1

    def producer(self, tid):
        for op in self.ops:
            if tid in op.outputs:
                return op
        return None

    def consumers(self, tid):
        return [op for op in self.ops if tid in op.inputs]

    def is_constant(self, tid):
        return tid in self.constants

    def types(self):
        return [op.type for op in self.ops]


# ---- the reference's passes ----------------------------------------------------------------------------------------
def convert_linear_to_addmm(g: Graph):
    for op in g.ops:
        if op.type == "aten::linear":
            x, w, b = op.inputs
            op.type, op.inputs = "aten::addmm", [b, x, w]
            op.attrs = {"act_type": "none"}


def remove_cat_for_addmm(g: Graph):
    for lst in [op for op in g.ops if op.type == "prim::ListConstruct" and len(op.inputs) == 2]:
        users = g.consumers(lst.outputs[0])
        if len(users) != 1 or users[0].type != "aten::cat":
            continue
        cat = users[0]
        users = g.consumers(cat.outputs[0])
        if len(users) != 1 or users[0].type != "aten::addmm" or users[0].inputs[1] != cat.outputs[0]:
            continue
        addmm = users[0]
        w_id = addmm.inputs[2]
        if not g.is_constant(w_id):
            continue
        first, second = lst.inputs
        split = lst.attrs.get("first_width")   # width of the first concatenated tensor (1024 in the reference)
        w = g.constants[w_id]
        if split is None or not 0 < split < w.size(1):
            continue
        w1_id, w2_id, mid = g.new_id(), g.new_id(), g.new_id()
        g.constants[w1_id] = w[:, :split].contiguous()
        g.constants[w2_id] = w[:, split:].contiguous()
        if len(g.consumers(w_id)) == 1:
            del g.constants[w_id]
        out = addmm.outputs[0]
        pos = g.ops.index(addmm)
        addmm.inputs, addmm.outputs = [addmm.inputs[0], first, w1_id], [mid]
        g.ops.insert(pos + 1, Op("aten::addmm", [mid, second, w2_id], [out], {"act_type": "none"}))
        g.ops.remove(lst)
        g.ops.remove(cat)


def _sandwich(g: Graph, op: Op, data_slot: int, weight_slot: int):
    """T(data) before `op`, operands swapped, T(result) after it (swap_addmm_inputs.cpp:42-97)."""
    data, out = op.inputs[data_slot], op.outputs[0]
    data_t, res = g.new_id(), g.new_id()
    pos = g.ops.index(op)
    g.ops.insert(pos, Op("aten::transpose", [data], [data_t], {"dim0": -2, "dim1": -1}))
    op.inputs[data_slot], op.inputs[weight_slot] = op.inputs[weight_slot], data_t
    op.outputs = [res]
    g.ops.insert(pos + 2, Op("aten::transpose", [res], [out], {"dim0": -2, "dim1": -1}))


def swap_addmm_inputs(g: Graph):
    for op in [o for o in g.ops if o.type == "aten::addmm" and len(o.inputs) >= 3 and g.is_constant(o.inputs[2])]:
        _sandwich(g, op, 1, 2)


def swap_matmul_inputs(g: Graph):
    for op in [o for o in g.ops if o.type == "aten::matmul" and len(o.inputs) == 2 and g.is_constant(o.inputs[1])]:
        if g.constants[op.inputs[1]].dim() == 2:
            _sandwich(g, op, 0, 1)


def fuse_activation(g: Graph):
    for relu in [o for o in g.ops if o.type == "aten::relu"]:
        pred = g.producer(relu.inputs[0])
        if pred is None or pred.type != "aten::transpose" or len(g.consumers(pred.outputs[0])) != 1:
            continue
        host = g.producer(pred.inputs[0])
        if host is None or host.type != "aten::addmm" or len(g.consumers(host.outputs[0])) != 1:
            continue
        host.attrs["act_type"] = "aten::relu"
        pred.outputs = [relu.outputs[0]]
        g.ops.remove(relu)


def apply_reference_passes(g: Graph):
    for p in (convert_linear_to_addmm, remove_cat_for_addmm, swap_addmm_inputs, swap_matmul_inputs, fuse_activation):
        p(g)
    return g


# ---- lowering onto the fused kernels -------------------------------------------------------------------------------
def lower_to_hot_path(g: Graph):
    """T(x) -> addmm(b, Wconst, .) / matmul(Wconst, .) -> T  becomes  gemv(x, W, b?, act): y = act(x . W^T + b)."""
    for op in [o for o in g.ops if o.type in ("aten::addmm", "aten::matmul")]:
        w_slot, d_slot = (1, 2) if op.type == "aten::addmm" else (0, 1)
        if not g.is_constant(op.inputs[w_slot]) or g.constants[op.inputs[w_slot]].dim() != 2:
            continue
        t_in = g.producer(op.inputs[d_slot])
        users = g.consumers(op.outputs[0])
        if t_in is None or t_in.type != "aten::transpose" or len(users) != 1 or users[0].type != "aten::transpose":
            continue
        if len(g.consumers(t_in.outputs[0])) != 1:
            continue
        t_out = users[0]
        bias = op.inputs[0] if op.type == "aten::addmm" else None
        op.type = "pimhip::gemv"
        op.inputs = [t_in.inputs[0], op.inputs[w_slot]] + ([bias] if bias is not None else [])
        op.outputs = t_out.outputs
        op.attrs = {"act_type": op.attrs.get("act_type", "none"), "has_bias": bias is not None}
        g.ops.remove(t_in)
        g.ops.remove(t_out)
    return g


def gemv_over_cat(g: Graph):
    """linear(cat([f, g], last dim), Wconst, b) [-> relu]  becomes one `pimhip::gemv_cat2` op on the whole weight
    (ops.aten_linear_cat2: one launch that reads f and g where they lie), where the reference's RemoveCatForAddmm makes two
    dependent addmm launches on the two column blocks of the weight (remove_cat_for_addmm.cpp:46-191).  Run it before
    apply_reference_passes; what it leaves alone (a cat with another reader, more than two parts, a weight that is not a
    constant) goes the reference's way."""
    for lst in [op for op in g.ops if op.type == "prim::ListConstruct" and len(op.inputs) == 2]:
        users = g.consumers(lst.outputs[0])
        if len(users) != 1 or users[0].type != "aten::cat" or users[0].attrs.get("dim", -1) not in (-1,) or lst.outputs[0] in g.outputs:
            continue
        cat = users[0]
        users = g.consumers(cat.outputs[0])
        if len(users) != 1 or users[0].type != "aten::linear" or users[0].inputs[0] != cat.outputs[0] or cat.outputs[0] in g.outputs:
            continue
        lin = users[0]
        if not g.is_constant(lin.inputs[1]) or g.constants[lin.inputs[1]] is None or g.constants[lin.inputs[1]].dim() != 2:
            continue
        has_bias = len(lin.inputs) > 2 and not (g.is_constant(lin.inputs[2]) and g.constants[lin.inputs[2]] is None)
        out, act = lin.outputs[0], "none"
        nxt = g.consumers(out)
        relu = nxt[0] if len(nxt) == 1 and nxt[0].type == "aten::relu" and out not in g.outputs else None
        if relu is not None:
            out, act = relu.outputs[0], "aten::relu"
            g.ops.remove(relu)
        lin.type = "pimhip::gemv_cat2"
        lin.inputs = [lst.inputs[0], lst.inputs[1], lin.inputs[1]] + ([lin.inputs[2]] if has_bias else [])
        lin.outputs = [out]
        lin.attrs = {"act_type": act, "has_bias": has_bias}
        g.ops.remove(lst)
        g.ops.remove(cat)
    return g


# ---- sibling products into one op ------------------------------------------------------------------------------------
_STREAM_TYPES = ("aten::addmm", "aten::matmul", "pimhip::gemv")


def _producers(g: Graph, op: Op):
    """Distinct non-constant ops that produce the inputs of `op`, in input order."""
    out = []
    for t in op.inputs:
        p = None if g.is_constant(t) else g.producer(t)
        if p is not None and p.type != "prim::Constant" and all(p is not q for q in out):
            out.append(p)
    return out


def _backward(g: Graph, root: Op, max_level: int, stop=None):
    """Breadth-first list of `root` and its non-constant ancestors, at most `max_level` levels up, not beyond `stop`."""
    seen, frontier = [root], [root]
    for _ in range(max_level):
        nxt = []
        for op in frontier:
            if op is stop:
                continue
            for p in _producers(g, op):
                if all(p is not q for q in seen):
                    seen.append(p)
                    nxt.append(p)
        frontier = nxt
    return seen


def multi_stream_execution(g: Graph, max_search_level: int = 10):
    """A join (an op with several non-constant producers) whose branches each contain a product, all hanging off one
    common start op: the products become one `multi_stream` op placed after the branches' preparation ops
    (multi_stream_execution.cpp: fitCondition :20-72, backwardToCheckAndFindStartLayer :96-228, process :230-290)."""
    for join in list(g.ops):
        if all(join is not o for o in g.ops):
            continue
        branches = _producers(g, join)
        if len(branches) < 2:
            continue
        members = []
        for b in branches:
            found = next((o for o in _backward(g, b, max_search_level) if o.type in _STREAM_TYPES), None)
            if found is None or any(found is m for m in members):
                members = []
                break
            members.append(found)
        if len(members) < 2:
            continue
        # no product may feed another one
        if any(any(a is x for x in _backward(g, m, max_search_level)[1:]) for m in members for a in members if a is not m):
            continue
        ancestors = [_backward(g, m, max_search_level)[1:] for m in members]
        start = next((a for a in ancestors[0] if a.type not in _STREAM_TYPES and all(any(a is x for x in anc) for anc in ancestors[1:])), None)
        if start is None:
            continue
        prep = []
        for m in members:
            for a in _backward(g, m, max_search_level, stop=start)[1:]:
                if a is not start and all(a is not q for q in prep):
                    prep.append(a)
        pos_start = g.ops.index(start)
        if any(g.ops.index(a) < pos_start for a in prep):
            continue                     # a branch takes something from before the start: leave the order alone
        prep.sort(key=g.ops.index)
        for a in prep + members:
            g.ops.remove(a)
        at = g.ops.index(start) + 1
        g.ops[at:at] = prep
        group = Op("multi_stream", [t for m in members for t in m.inputs], [t for m in members for t in m.outputs],
                   {"layers": members})
        g.ops.insert(at + len(prep), group)
    return g


# ---- the decoder's per-token chain into one op -----------------------------------------------------------------------
_DECODER_MAX_LAYERS = 4
_DECODER_MAX_HIDDEN = 1024


def _lstm_input_form(g: Graph, op: Op):
    """(in, ctx, [cat op, list op]) when the cell's input is cat([in, ctx]) along the last dim, else (input, None, [])."""
    cat = g.producer(op.inputs[0])
    if cat is not None and cat.type == "aten::cat" and cat.attrs.get("dim", -1) in (-1, 2):
        lst = g.producer(cat.inputs[0])
        if (lst is not None and lst.type == "prim::ListConstruct" and len(lst.inputs) == 2 and
                len(g.consumers(cat.outputs[0])) == 1 and len(g.consumers(lst.outputs[0])) == 1 and
                cat.outputs[0] not in g.outputs and lst.outputs[0] not in g.outputs):
            return lst.inputs[0], lst.inputs[1], [cat, lst]
    return op.inputs[0], None, []


def _lstm_output_form(g: Graph, op: Op, in_tid):
    """(out, residual add or None): out = y + in when y feeds exactly one add with the cell's own input, else y."""
    y = op.outputs[0]
    users = g.consumers(y)
    if len(users) == 1 and users[0].type == "aten::add" and y not in g.outputs and sorted(users[0].inputs) == sorted([y, in_tid]) \
            and y != in_tid and users[0].attrs.get("alpha", 1) == 1:
        return users[0].outputs[0], users[0]
    return y, None


def _depends_on(g: Graph, tid, ops_):
    """True if tensor `tid` is computed from an output of one of `ops_`."""
    seen, todo = set(), [tid]
    while todo:
        t = todo.pop()
        if t in seen:
            continue
        seen.add(t)
        p = g.producer(t)
        if p is None:
            continue
        if any(p is o for o in ops_):
            return True
        todo.extend(p.inputs)
    return False


def _single_step_cell(g: Graph, op: Op):
    """An aten::lstm op this pass may take: one layer, one direction, constant fp16 weights with biases, H within the
    fused kernel's range."""
    if op.type != "aten::lstm" or len(op.inputs) != 7 or len(op.outputs) != 3:
        return False
    if op.attrs.get("num_layers", 1) != 1 or op.attrs.get("bidirectional", False) or not op.attrs.get("has_biases", True):
        return False
    if op.attrs.get("seq_len", 1) != 1:
        return False
    if not all(g.is_constant(t) and g.constants[t] is not None for t in op.inputs[3:7]):
        return False
    w_ih, w_hh = g.constants[op.inputs[3]], g.constants[op.inputs[4]]
    H = w_hh.size(1)
    return (w_ih.dtype == torch.float16 and w_hh.dim() == 2 and w_ih.dim() == 2 and tuple(w_hh.shape) == (4 * H, H) and
            w_ih.size(0) == 4 * H and H % 8 == 0 and 8 <= H <= _DECODER_MAX_HIDDEN and w_ih.size(1) % 8 == 0)


def fuse_decoder_step(g: Graph):
    """Chains of seq_len-1 cells  lstm_0(x | cat(x, ctx)) -> [add] -> cat(., ctx) -> lstm_1 -> [add] -> ...  (the same ctx in
    every cat, residual adds from some layer on), optionally with the attention bmm that produces ctx and the linear
    classifier on the last output, become one `pimhip::decoder_step` op at the position of the chain's first op.

    Left alone: cells whose weights are not constants, a pre-residual y with another consumer (the fused step only
    stores out_k, hn_k, cn_k), a context that is computed from the chain itself (in GNMT the attention query is layer
    0's output: the chain then starts at layer 1), a cell whose initial state is computed from the cells below it (the chain
    ends in front of it), chains of fewer than two cells."""
    taken = []
    for first in list(g.ops):
        if all(first is not o for o in g.ops) or any(first is o for o in taken) or not _single_step_cell(g, first):
            continue
        # ---- follow the chain upwards from `first`
        forms, ctx, cur = [], None, first
        while cur is not None and len(forms) < _DECODER_MAX_LAYERS and _single_step_cell(g, cur) and all(cur is not o for o in taken):
            in_tid, c_tid, glue = _lstm_input_form(g, cur)
            H = g.constants[cur.inputs[4]].size(1)
            own_w = g.constants[cur.inputs[3]].size(1) - (H if c_tid is not None else 0)   # width of the cell's own input
            if own_w < 8:
                break
            if forms:
                # a later cell reads cat(previous output, the chain's context)
                if in_tid != forms[-1]["out"] or c_tid is None or (ctx is not None and c_tid != ctx) or H != forms[0]["H"] or own_w != H:
                    break
            elif c_tid is not None and own_w != H:
                break                          # a first cell on cat(x, ctx) needs x as wide as the hidden state
            if c_tid is not None:
                ctx = c_tid
            out, add = _lstm_output_form(g, cur, in_tid)
            if add is not None and own_w != H:
                out, add = cur.outputs[0], None  # y + x with x of another width is not this wiring's residual
            forms.append(dict(cell=cur, in_tid=in_tid, takes_ctx=c_tid is not None, glue=glue, out=out, add=add, H=H))
            cur = None
            for u in g.consumers(out):
                if u.type != "prim::ListConstruct" or len(u.inputs) != 2 or u.inputs[0] != out:
                    continue
                cats = g.consumers(u.outputs[0])
                cells_ = g.consumers(cats[0].outputs[0]) if len(cats) == 1 and cats[0].type == "aten::cat" else []
                if len(cells_) == 1 and cells_[0].type == "aten::lstm" and cells_[0].inputs[0] == cats[0].outputs[0]:
                    cur = cells_[0]
                    break
        # ---- residual adds must be contiguous from some layer on; cut the chain where they stop being so
        n = len(forms)
        for k in range(n):
            if forms[k]["add"] is None and any(forms[q]["add"] is not None for q in range(k)):
                n = k
                break
        forms = forms[:n]
        # ---- a cell's initial state must not be computed from the chain below it (the previous cell's hn handed on, say):
        # the fused op reads every h0 / c0 before any cell runs, so the chain is cut in front of such a cell
        for k in range(1, len(forms)):
            below = [m for f in forms[:k] for m in [f["cell"]] + ([f["add"]] if f["add"] is not None else [])]
            if any(_depends_on(g, t, below) for t in forms[k]["cell"].inputs[1:3]):
                forms = forms[:k]
                break
        # ---- the context must not be computed from the chain
        if ctx is not None and forms and _depends_on(g, ctx, [f["cell"] for f in forms]):
            continue                          # (the chain that starts one cell later is found when the loop reaches that cell)
        if len(forms) < 2:
            continue
        first_res = next((k for k in range(len(forms)) if forms[k]["add"] is not None), len(forms))
        members = []
        for f in forms:
            members += f["glue"] + [f["cell"]] + ([f["add"]] if f["add"] is not None else [])
        # ---- the attention bmm, when the chain is the context's only consumer
        att = enc = None
        bmm = g.producer(ctx) if ctx is not None else None
        if (bmm is not None and bmm.type == "aten::bmm" and ctx not in g.outputs and
                all(any(u is m for m in members) for u in g.consumers(ctx))):
            att, enc = bmm.inputs
            members.append(bmm)
        # ---- the classifier on the last output
        last_out = forms[-1]["out"]
        cls = next((u for u in g.consumers(last_out)
                    if u.type in ("aten::linear", "pimhip::gemv") and u.inputs[0] == last_out and g.is_constant(u.inputs[1]) and
                    g.constants[u.inputs[1]] is not None and g.constants[u.inputs[1]].dim() == 2 and g.constants[u.inputs[1]].size(1) == forms[0]["H"] and
                    u.attrs.get("act_type", "none") == "none"), None)
        if cls is not None:
            members.append(cls)
        # ---- the fused op goes where the chain starts, or right after the last producer of something it reads if that is
        # later; no operator before that place may read what the chain computes
        external = [forms[0]["in_tid"]] + [t for f in forms for t in f["cell"].inputs[1:3]]
        external += [att, enc] if att is not None else ([ctx] if ctx is not None else [])
        pos = min(g.ops.index(m) for m in members)
        for t in external:
            prod = g.producer(t)
            if prod is not None:
                pos = max(pos, g.ops.index(prod) + 1)
        produced = {t for m in members for t in m.outputs}
        if any(all(o is not m for m in members) and produced.intersection(o.inputs) for o in g.ops[:pos]):
            continue
        pos -= sum(1 for m in members if g.ops.index(m) < pos)     # index after the members have been taken out
        cls_bias = None
        if cls is not None and len(cls.inputs) > 2 and (cls.type == "aten::linear" or cls.attrs.get("has_bias")):
            cls_bias = cls.inputs[2]
        L = len(forms)
        fused = Op("pimhip::decoder_step",
                   [forms[0]["in_tid"]] + ([att, enc] if att is not None else ([ctx] if ctx is not None else [])) +
                   [f["cell"].inputs[1] for f in forms] + [f["cell"].inputs[2] for f in forms],
                   [f["out"] for f in forms] + [f["cell"].outputs[1] for f in forms] + [f["cell"].outputs[2] for f in forms] +
                   ([cls.outputs[0]] if cls is not None else []),
                   {"num_layers": L, "hidden": forms[0]["H"], "first_takes_context": forms[0]["takes_ctx"],
                    "first_residual_layer": first_res, "context": "bmm" if att is not None else ("given" if ctx is not None else "none"),
                    "params": [t for f in forms for t in f["cell"].inputs[3:7]],
                    "classifier": (cls.inputs[1], cls_bias) if cls is not None else None,
                    "out_shapes": "as the operators' ([1, 1, H] per layer, classifier as its operator would)"})
        for m in members:
            g.ops.remove(m)
        g.ops.insert(pos, fused)
        taken.append(fused)
    return g


# ---- consecutive sequence layers into one multi-layer op -------------------------------------------------------------
def _sequence_layer(g: Graph, op: Op):
    """A one-layer, one-direction aten::lstm over a padded sequence with constant fp16 weights and biases (seq_len-1 cells
    are fuse_decoder_step's)."""
    if op.type != "aten::lstm" or len(op.inputs) != 7 or len(op.outputs) != 3:
        return False
    a = op.attrs
    if a.get("num_layers", 1) != 1 or a.get("bidirectional", False) or not a.get("has_biases", True) or a.get("batch_first", False):
        return False
    if a.get("seq_len", 0) == 1:
        return False
    if not all(g.is_constant(t) and g.constants[t] is not None for t in op.inputs[3:7]):
        return False
    w_ih, w_hh = g.constants[op.inputs[3]], g.constants[op.inputs[4]]
    return (w_ih.dtype == torch.float16 and w_hh.dtype == torch.float16 and w_ih.dim() == 2 and w_hh.dim() == 2 and
            w_hh.size(0) == 4 * w_hh.size(1) and w_ih.size(0) == w_hh.size(0))


def fuse_lstm_stack(g: Graph):
    """lstm_a(x, h0_a, c0_a) -> lstm_b(y_a, h0_b, c0_b) -> ...  becomes  lstm(x, cat(h0_a, h0_b, ..), cat(c0_a, c0_b, ..))
    with num_layers = n and the parameters of the layers in order, placed where the chain's last op was.  The stacked
    hn / cn are sliced back into the tensors the single ops produced, for whoever reads them.

    A layer may carry a residual sum, out = lstm(in) + in (the GNMT encoder's upper layers): from the first such layer on
    every layer of the chain has to, and the fused op is then a `pimhip::lstm_stack` with `first_residual_layer` (an
    aten::lstm has no such wiring; ops.LstmPlan.set_residual runs it as the same one-launch pipeline).

    A layer joins the chain when the sequence before it is read by nothing but that layer (and its own residual sum) and
    is not a graph output, its input width is the hidden size of the layer before (as in a multi-layer aten::lstm) and its
    hidden size is the same.  Left alone: layers whose y is read before the sum, layers whose initial state is computed
    from the chain itself, chains whose intermediate hn / cn are read before the chain's end, a plain layer above one with
    a residual sum."""
    taken = set()
    for first in list(g.ops):
        if id(first) in taken or all(first is not o for o in g.ops) or not _sequence_layer(g, first):
            continue

        def form(op):
            """(out, add op or None) of a layer: its residual sum when y feeds exactly one add with the layer's own input."""
            out, add = _lstm_output_form(g, op, op.inputs[0])
            if add is not None and g.constants[op.inputs[3]].size(1) != g.constants[op.inputs[4]].size(1):
                return op.outputs[0], None
            return out, add

        chain, adds = [first], [form(first)[1]]
        cur = form(first)[0]
        while True:
            last = chain[-1]
            users = g.consumers(cur)
            cand = [u for u in users if u.type == "aten::lstm" and u.inputs[0] == cur]
            if len(cand) != 1 or cur in g.outputs:
                break
            nxt = cand[0]
            H = g.constants[last.inputs[4]].size(1)
            if not _sequence_layer(g, nxt) or g.constants[nxt.inputs[4]].size(1) != H or g.constants[nxt.inputs[3]].size(1) != H:
                break
            n_out, n_add = form(nxt)
            allowed = [nxt] + ([n_add] if n_add is not None else [])
            if any(all(u is not a for a in allowed) for u in users) or sum(u.inputs.count(cur) for u in users) != len(allowed):
                break  # somebody else reads the sequence in between
            if n_add is None and any(a is not None for a in adds):
                break  # a plain layer above one with a residual sum
            if any(_depends_on(g, t, chain) for t in nxt.inputs[1:3]):
                break
            if nxt.attrs.get("seq_len", 0) != last.attrs.get("seq_len", 0):
                break
            chain.append(nxt)
            adds.append(n_add)
            cur = n_out
        # a first layer with a residual sum whose y has another reader was refused by form(); nothing else to check there.
        # The intermediate hn / cn must not be read before the place the fused op takes (the last op's).
        while len(chain) >= 2:
            tail = adds[-1] if adds[-1] is not None else chain[-1]
            end = next(i for i, o in enumerate(g.ops) if o is tail)
            early = False
            for o in chain[:-1]:
                for t in o.outputs[1:3]:
                    for user in g.consumers(t):
                        if next(i for i, q in enumerate(g.ops) if q is user) < end:
                            early = True
            if not early:
                break
            chain.pop()
            adds.pop()
        if len(chain) < 2:
            continue
        n = len(chain)
        first_res = next((k for k, a in enumerate(adds) if a is not None), n)
        out_tid = adds[-1].outputs[0] if adds[-1] is not None else chain[-1].outputs[0]
        state, pre = [], []
        for slot in (1, 2):
            ids = [o.inputs[slot] for o in chain]
            if all(g.is_constant(t) and g.constants[t] is not None for t in ids):
                tid = g.new_id()
                g.constants[tid] = torch.cat([g.constants[t].reshape(1, 1, -1) for t in ids], 0)
            else:
                lst = g.new_id()
                pre.append(Op("prim::ListConstruct", ids, [lst]))
                tid = g.new_id()
                pre.append(Op("aten::cat", [lst], [tid], {"dim": 0}))
            state.append(tid)
        hn_all, cn_all = g.new_id(), g.new_id()
        params = [t for o in chain for t in o.inputs[3:7]]
        attrs = dict(chain[0].attrs)
        attrs["num_layers"] = n
        if first_res < n:
            attrs["first_residual_layer"] = first_res
        fused = Op("aten::lstm" if first_res == n else "pimhip::lstm_stack", [chain[0].inputs[0]] + state + params,
                   [out_tid, hn_all, cn_all], attrs)
        post = []
        for k, o in enumerate(chain):
            for t, src in ((o.outputs[1], hn_all), (o.outputs[2], cn_all)):
                if g.consumers(t) or t in g.outputs:
                    post.append(Op("aten::slice", [src], [t], {"dim": 0, "start": k, "end": k + 1}))
        gone = chain + [a for a in adds if a is not None]
        tail = adds[-1] if adds[-1] is not None else chain[-1]
        end = next(i for i, o in enumerate(g.ops) if o is tail)
        g.ops[end:end + 1] = pre + [fused] + post
        g.ops = [o for o in g.ops if all(o is not c for c in gone)]
        taken.update(id(o) for o in gone)
    return g


def _as_row_major_weight(t):
    """For a [..1.., in, out] tensor that is a transposed view of a dense row-major [out, in] matrix: that matrix."""
    if t.dim() < 2 or any(d != 1 for d in t.shape[:-2]) or t.dtype != torch.float16:
        return None
    m = t.reshape(t.shape[-2:]) if t.dim() == 2 else t[(0,) * (t.dim() - 2)]
    if m.stride(0) == 1 and m.stride(1) == m.size(0) and m.size(0) % 8 == 0 and m.data_ptr() % 16 == 0:
        return m.t()
    return None


# ---- execution through the operator layer ----------------------------------------------------------------------------
def _run_decoder_step(op: Op, env, ops, same_sentence):
    """One pimhip::decoder_step op: the plan is made on first use and kept on the op; outputs are new tensors shaped as the
    operators it replaces would shape them."""
    at = op.attrs
    L, H = at["num_layers"], at["hidden"]
    plan = at.get("_plan")
    if plan is None:
        cls = None
        if at["classifier"] is not None:
            w_t, b_t = at["classifier"]
            cls = (env[w_t], env[b_t] if b_t is not None else None)
        plan = ops.DecoderPlan([env[t] for t in at["params"]], True, L, first_takes_context=at["first_takes_context"],
                               first_residual_layer=at["first_residual_layer"], classifier=cls)
        at["_plan"] = plan
    x = env[op.inputs[0]]
    att = enc = ctx = None
    i = 1
    if at["context"] == "bmm":
        att, enc = env[op.inputs[1]], env[op.inputs[2]]
        i = 3
        if not (same_sentence and plan._enc is not None):
            plan.set_encoder(enc.reshape(-1, H).contiguous())
    elif at["context"] == "given":
        ctx = env[op.inputs[1]]
        i = 2
    flat = lambda t: t.contiguous().view(-1)  # noqa: E731
    h_prev = [flat(env[t]) for t in op.inputs[i:i + L]]
    c_prev = [flat(env[t]) for t in op.inputs[i + L:i + 2 * L]]
    new = lambda: torch.empty(1, 1, H, dtype=torch.float16, device=x.device)  # noqa: E731
    outs, hn, cn = [new() for _ in range(L)], [new() for _ in range(L)], [new() for _ in range(L)]
    logits = None
    if plan.vocab:
        logits = torch.empty(list(outs[-1].shape[:-1]) + [plan.vocab], dtype=torch.float16, device=x.device)
    step = plan.bind(flat(x), h_prev, c_prev, att=flat(att) if att is not None else None, ctx=flat(ctx) if ctx is not None else None,
                     hn=[t.view(-1) for t in hn], cn=[t.view(-1) for t in cn], outs=[t.view(-1) for t in outs],
                     logits=logits.view(-1) if logits is not None else None)
    step()
    for k in range(L):
        env[op.outputs[k]], env[op.outputs[L + k]], env[op.outputs[2 * L + k]] = outs[k], hn[k], cn[k]
    if logits is not None:
        env[op.outputs[3 * L]] = logits


def execute(g: Graph, feeds: Dict[int, torch.Tensor], device="cuda:0", same_sentence=False):
    """Runs the op list with pimaicompiler_amd.ops; returns the graph outputs.  Constants are moved to `device`.
    `same_sentence`: the encoder outputs a fused decoder step attends over are the ones of the previous call (their
    projection is then not computed again)."""
    from . import ops

    env = {k: (v.to(device) if v is not None else None) for k, v in g.constants.items()}
    env.update({k: v.to(device) for k, v in feeds.items()})
    for op in g.ops:
        a = [env[i] for i in op.inputs]
        if op.type == "aten::linear":
            r = ops.aten_linear(a[0], a[1], a[2])
        elif op.type == "aten::addmm":
            r = ops.custom_aten_addmm(op.attrs.get("act_type", "none"), a[0], a[1], a[2])
        elif op.type == "aten::matmul":
            r = ops.custom_aten_matmul(a[0], a[1])
        elif op.type == "pimhip::gemv":
            r = ops.aten_linear(a[0], a[1], a[2] if op.attrs["has_bias"] else None, act_type=op.attrs["act_type"])
        elif op.type == "pimhip::gemv_cat2":
            r = ops.aten_linear_cat2(a[0], a[1], a[2], a[3] if op.attrs["has_bias"] else None, act_type=op.attrs["act_type"])
        elif op.type == "multi_stream":
            subs = op.attrs["layers"]
            if all(m.type == "pimhip::gemv" for m in subs):
                xs = [env[m.inputs[0]] for m in subs]
                outs = ops.execute_gemv_group(xs, [env[m.inputs[1]] for m in subs],
                                              [env[m.inputs[2]] if m.attrs["has_bias"] else None for m in subs],
                                              [m.attrs["act_type"] for m in subs])
                for m, x, o in zip(subs, xs, outs):
                    env[m.outputs[0]] = o.view(list(x.shape[:-1]) + [o.numel()])
            elif all(m.type == "aten::matmul" and _as_row_major_weight(env[m.inputs[1]]) is not None and
                     env[m.inputs[0]].numel() == env[m.inputs[1]].size(-2) for m in subs):
                # x . T(W_i) with W_i a dense [out, in] slice (the Switch Transformer wiring): the transposed view is the
                # MV order on the slice's own bytes, so these siblings also go out as one grouped launch.
                xs = [env[m.inputs[0]] for m in subs]
                ws = [_as_row_major_weight(env[m.inputs[1]]) for m in subs]
                outs = ops.execute_gemv_group(xs, ws)
                for m, x, o in zip(subs, xs, outs):
                    other = env[m.inputs[1]]
                    shape = list(other.shape) if other.dim() > x.dim() else list(x.shape)
                    shape[-1], shape[-2] = o.numel(), 1
                    env[m.outputs[0]] = o.view(shape)
            else:
                for m in subs:
                    am = [env[i] for i in m.inputs]
                    env[m.outputs[0]] = (ops.custom_aten_addmm(m.attrs.get("act_type", "none"), am[0], am[1], am[2])
                                         if m.type == "aten::addmm" else ops.custom_aten_matmul(am[0], am[1]))
            continue
        elif op.type == "pimhip::decoder_step":
            _run_decoder_step(op, env, ops, same_sentence)
            continue
        elif op.type == "pimhip::lstm_stack":
            n = op.attrs["num_layers"]
            y, hn, cn = ops.aten_lstm1(a[0], (a[1], a[2]), a[3:3 + 4 * n], True, n, 0.0, False, False, False,
                                       first_residual_layer=op.attrs["first_residual_layer"])
            env[op.outputs[0]], env[op.outputs[1]], env[op.outputs[2]] = y, hn, cn
            continue
        elif op.type == "aten::lstm":
            n = op.attrs.get("num_layers", 1)
            bidir = bool(op.attrs.get("bidirectional", False))
            y, hn, cn = ops.aten_lstm1(a[0], (a[1], a[2]), a[3:3 + 4 * n * (2 if bidir else 1)], True, n, 0.0, False, bidir,
                                       bool(op.attrs.get("batch_first", False)))
            env[op.outputs[0]], env[op.outputs[1]], env[op.outputs[2]] = y, hn, cn
            continue
        elif op.type == "aten::bmm":
            r = ops.aten_bmm(a[0], a[1])
        elif op.type == "aten::contiguous":
            r = a[0].contiguous()
        elif op.type == "aten::slice":
            r = a[0].narrow(op.attrs["dim"], op.attrs["start"], op.attrs["end"] - op.attrs["start"])
        elif op.type == "aten::add":
            r = ops.aten_add(a[0], a[1])
        elif op.type == "aten::transpose":
            r = a[0].transpose(op.attrs["dim0"], op.attrs["dim1"])
        elif op.type == "aten::relu":
            r = torch.relu(a[0])
        elif op.type == "prim::ListConstruct":
            r = list(a)
        elif op.type == "aten::cat":
            r = torch.cat(a[0], dim=op.attrs.get("dim", -1))
        else:
            raise ValueError(f"op {op.type} is not part of this path")
        env[op.outputs[0]] = r
    return [env[i] for i in g.outputs]
