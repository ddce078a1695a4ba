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


def _as_row_major_weight(t):
    """For a [..1.., in, out] tensor that is a transposed view of a dense row-major [out, in] matrix: that matrix."""
    if t.dim() < 2 or any(d != 1 for d in t.shape[:-2]) or t.dtype != torch.float16:
        return None
    m = t.reshape(t.shape[-2:]) if t.dim() == 2 else t[(0,) * (t.dim() - 2)]
    if m.stride(0) == 1 and m.stride(1) == m.size(0) and m.size(0) % 8 == 0 and m.data_ptr() % 16 == 0:
        return m.t()
    return None


# ---- execution through the operator layer ----------------------------------------------------------------------------
def execute(g: Graph, feeds: Dict[int, torch.Tensor], device="cuda:0"):
    """Runs the op list with pimaicompiler_amd.ops; returns the graph outputs.  Constants are moved to `device`."""
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
