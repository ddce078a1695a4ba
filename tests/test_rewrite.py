"""The graph rewrites that feed the GEMV kernels (pimaicompiler_amd/rewrite.py): structure on the CPU, numerics on
the GPU against eager LibTorch on the original op list."""
import pytest
import torch

from pimaicompiler_amd import rewrite as R

DEV = "cuda:0"


def mlp_graph(seed=0, d_in=768, d_hidden=3072, d_out=768):
    """x -> linear(W1, b1) -> relu -> linear(W2, b2): the expert FFN of the MoE configuration."""
    g = torch.Generator().manual_seed(seed)
    c = {10: (0.02 * torch.randn(d_hidden, d_in, generator=g)).half(), 11: (0.02 * torch.randn(d_hidden, generator=g)).half(),
         12: (0.02 * torch.randn(d_out, d_hidden, generator=g)).half(), 13: (0.02 * torch.randn(d_out, generator=g)).half()}
    ops = [R.Op("aten::linear", [0, 10, 11], [1]), R.Op("aten::relu", [1], [2]), R.Op("aten::linear", [2, 12, 13], [3])]
    return R.Graph(ops, [0], [3], c, next_id=20), torch.randn(1, d_in, generator=g).half()


def joint_graph(seed=1):
    """RNNT joint: addmm over cat([f[1,1024], g[1,320]]) with a [512,1344] weight, then relu."""
    g = torch.Generator().manual_seed(seed)
    c = {10: (0.03 * torch.randn(512, 1344, generator=g)).half(), 11: (0.05 * torch.randn(512, generator=g)).half()}
    ops = [R.Op("prim::ListConstruct", [0, 1], [2], {"first_width": 1024}), R.Op("aten::cat", [2], [3], {"dim": -1}),
           R.Op("aten::linear", [3, 10, 11], [4]), R.Op("aten::relu", [4], [5])]
    return R.Graph(ops, [0, 1], [5], c, next_id=20), torch.randn(1, 1024, generator=g).half(), torch.randn(1, 320, generator=g).half()


def test_passes_produce_the_reference_structure():
    g, _ = mlp_graph()
    R.apply_reference_passes(g)
    # linear -> addmm; transposes around each addmm; the relu folded into the first addmm's act_type
    assert g.types() == ["aten::transpose", "aten::addmm", "aten::transpose", "aten::transpose", "aten::addmm", "aten::transpose"]
    a1, a2 = g.ops[1], g.ops[4]
    assert a1.attrs["act_type"] == "aten::relu" and a2.attrs["act_type"] == "none"
    # addmm(bias, W, T(x)): weight constant second, transposed data third (swap_addmm_inputs.cpp:64-67)
    assert a1.inputs[0] == 11 and a1.inputs[1] == 10 and a1.inputs[2] == g.ops[0].outputs[0] and g.ops[0].inputs == [0]
    assert g.ops[2].outputs == [2] and g.ops[3].inputs == [2]      # the relu's output id is now the transpose's output
    assert g.ops[5].outputs == [3] and g.outputs == [3]


def test_remove_cat_splits_the_weight_by_columns():
    g, f, gg = joint_graph()
    W, b = g.constants[10].clone(), g.constants[11].clone()
    R.convert_linear_to_addmm(g)
    R.remove_cat_for_addmm(g)
    assert g.types() == ["aten::addmm", "aten::addmm", "aten::relu"]
    first, second = g.ops[0], g.ops[1]
    assert first.inputs[:2] == [11, 0] and second.inputs[0] == first.outputs[0] and second.inputs[1] == 1
    assert torch.equal(g.constants[first.inputs[2]], W[:, :1024]) and torch.equal(g.constants[second.inputs[2]], W[:, 1024:])
    assert 10 not in g.constants and second.outputs == [4]


def test_product_over_a_cat_becomes_one_op():
    g, f, h = joint_graph()
    R.gemv_over_cat(g)
    assert g.types() == ["pimhip::gemv_cat2"]
    op = g.ops[0]
    assert op.inputs == [0, 1, 10, 11] and op.outputs == [5] and op.attrs == {"act_type": "aten::relu", "has_bias": True}
    R.apply_reference_passes(g)                       # nothing left for the reference's passes to split
    assert g.types() == ["pimhip::gemv_cat2"]
    # a cat that something else reads as well is left to the reference's way
    g, f, h = joint_graph()
    g.outputs.append(3)
    R.gemv_over_cat(g)
    assert g.types() == ["prim::ListConstruct", "aten::cat", "aten::linear", "aten::relu"]


def test_matmul_swap_and_fusion_guards():
    c = {10: torch.randn(8, 8).half(), 11: torch.randn(2, 8, 8).half()}
    g = R.Graph([R.Op("aten::matmul", [0, 10], [1]), R.Op("aten::matmul", [0, 11], [2]), R.Op("aten::matmul", [1, 2], [3])], [0], [3], c, 20)
    R.apply_reference_passes(g)
    assert g.types() == ["aten::transpose", "aten::matmul", "aten::transpose", "aten::matmul", "aten::matmul"]   # 2-D constant only
    # a relu whose producer has a second consumer is not fused (fuse_activation.cpp:29-33)
    c = {10: torch.randn(8, 8).half(), 11: torch.randn(8).half()}
    g = R.Graph([R.Op("aten::linear", [0, 10, 11], [1]), R.Op("aten::relu", [1], [2]), R.Op("aten::matmul", [1, 2], [3])], [0], [3], c, 20)
    R.apply_reference_passes(g)
    assert "aten::relu" in g.types() and g.ops[1].attrs["act_type"] == "none"


def test_lowering_removes_every_transpose():
    g, _ = mlp_graph()
    R.lower_to_hot_path(R.apply_reference_passes(g))
    assert g.types() == ["pimhip::gemv", "pimhip::gemv"]
    assert g.ops[0].inputs == [0, 10, 11] and g.ops[0].attrs == {"act_type": "aten::relu", "has_bias": True}
    assert g.ops[1].inputs == [2, 12, 13] and g.ops[1].outputs == [3]
    g, _, _ = joint_graph()
    R.lower_to_hot_path(R.apply_reference_passes(g))
    assert g.types() == ["pimhip::gemv", "pimhip::gemv"] and g.ops[1].attrs["act_type"] == "aten::relu"
    assert g.ops[1].inputs[2] == g.ops[0].outputs[0]     # the first product is the second one's bias


@pytest.mark.gpu
def test_rewritten_graphs_compute_what_eager_libtorch_computes(ops):
    # expert FFN
    g0, x = mlp_graph()
    c = g0.constants
    want = torch.nn.functional.linear(torch.relu(torch.nn.functional.linear(x.float(), c[10].float(), c[11].float())).half().float(),
                                      c[12].float(), c[13].float())
    for stage in ("original", "reference", "lowered"):
        g, _ = mlp_graph()
        if stage != "original":
            R.apply_reference_passes(g)
        if stage == "lowered":
            R.lower_to_hot_path(g)
        (y,) = R.execute(g, {0: x}, DEV)
        assert list(y.shape) == [1, 768], stage
        assert float((y.float().cpu() - want).abs().max()) <= 2e-3, stage
    # RNNT joint
    g0, f, gg = joint_graph()
    c = g0.constants
    want = torch.relu(torch.nn.functional.linear(torch.cat([f, gg], -1).float(), c[10].float(), c[11].float()))
    for stage in ("original", "reference", "lowered"):
        g, _, _ = joint_graph()
        if stage != "original":
            R.apply_reference_passes(g)
        if stage == "lowered":
            R.lower_to_hot_path(g)
        (y,) = R.execute(g, {0: f, 1: gg}, DEV)
        assert list(y.shape) == [1, 512], stage
        # two roundings (the split product is rounded to fp16 in between): 2 x 2e-3
        assert float((y.float().cpu() - want).abs().max()) <= 4e-3, stage
    # the same layer as one launch that reads f and g where they lie: one rounding
    g, _, _ = joint_graph()
    R.gemv_over_cat(g)
    (y,) = R.execute(g, {0: f, 1: gg}, DEV)
    assert list(y.shape) == [1, 512] and float((y.float().cpu() - want).abs().max()) <= 2e-3


def attention_projection_graph(seed=3, d=512, n=4, constant_weights=True):
    """The structure the reference's multi-stream pass looks for (multi_stream_execution.h:24-41): one start op, n
    branches ending in matmul -> add, joined by a ListConstruct.  With constant 2-D weights the branches are
    slice(x) -> matmul(., W_i) and the front-end passes turn each product into the MV order; otherwise the weights are
    slices of one stacked tensor, transposed on the way, as in the reference's Switch Transformer graph."""
    g = torch.Generator().manual_seed(seed)
    c, join_in = {}, []
    if constant_weights:
        ops, inputs = [R.Op("aten::contiguous", [0], [1])], [0]
        feeds = {0: torch.randn(n, d, generator=g).half()}
    else:
        ops, inputs = [R.Op("aten::contiguous", [0], [1])], [0, 5]
        feeds = {0: (0.03 * torch.randn(n, d, d, generator=g)).half(), 5: torch.randn(1, d, generator=g).half()}
    for i in range(n):
        c[200 + i] = (0.1 * torch.randn(1, d, generator=g)).half()
        if constant_weights:
            c[100 + i] = (0.03 * torch.randn(d, d, generator=g)).half()
            ops += [R.Op("aten::slice", [1], [10 + i], {"dim": 0, "start": i, "end": i + 1}),
                    R.Op("aten::matmul", [10 + i, 100 + i], [20 + i])]
        else:
            ops += [R.Op("aten::slice", [1], [10 + i], {"dim": 0, "start": i, "end": i + 1}),
                    R.Op("aten::transpose", [10 + i], [50 + i], {"dim0": -2, "dim1": -1}),
                    R.Op("aten::matmul", [5, 50 + i], [20 + i])]
        ops.append(R.Op("aten::add", [20 + i, 200 + i], [30 + i]))
        join_in.append(30 + i)
    ops.append(R.Op("prim::ListConstruct", join_in, [40]))
    return R.Graph(ops, inputs, [40], c, next_id=300), feeds


def test_multi_stream_pass_collects_the_sibling_products():
    g, _ = attention_projection_graph()
    R.apply_reference_passes(g)
    R.lower_to_hot_path(g)
    assert g.types().count("pimhip::gemv") == 4
    R.multi_stream_execution(g)
    # start, the four slices moved up behind it, ONE multi_stream op holding the four products, then the adds and the join
    assert g.types() == ["aten::contiguous"] + ["aten::slice"] * 4 + ["multi_stream"] + ["aten::add"] * 4 + ["prim::ListConstruct"]
    ms = g.ops[5]
    assert [m.type for m in ms.attrs["layers"]] == ["pimhip::gemv"] * 4 and ms.outputs == [20, 21, 22, 23]
    # the Switch Transformer shape of it: the products keep their type, their slices and transposes move up
    g, _ = attention_projection_graph(constant_weights=False)
    R.apply_reference_passes(g)
    R.lower_to_hot_path(g)
    R.multi_stream_execution(g)
    assert g.types() == ["aten::contiguous"] + ["aten::slice", "aten::transpose"] * 4 + ["multi_stream"] + ["aten::add"] * 4 + ["prim::ListConstruct"]
    assert [m.type for m in g.ops[9].attrs["layers"]] == ["aten::matmul"] * 4


def test_multi_stream_pass_leaves_dependent_or_startless_products_alone():
    # a chain (the second product consumes the first) joined with its own input: nothing to run side by side
    c = {10: torch.randn(8, 8).half(), 11: torch.randn(8, 8).half()}
    g = R.Graph([R.Op("aten::relu", [0], [1]), R.Op("aten::matmul", [1, 10], [2]), R.Op("aten::matmul", [2, 11], [3]),
                 R.Op("prim::ListConstruct", [2, 3], [4])], [0], [4], c, 20)
    before = g.types()
    R.multi_stream_execution(g)
    assert g.types() == before
    # two products on two different graph inputs: no common start
    g = R.Graph([R.Op("aten::matmul", [0, 10], [2]), R.Op("aten::matmul", [1, 11], [3]), R.Op("prim::ListConstruct", [2, 3], [4])],
                [0, 1], [4], c, 20)
    R.multi_stream_execution(g)
    assert g.types() == ["aten::matmul", "aten::matmul", "prim::ListConstruct"]


@pytest.mark.gpu
def test_multi_stream_graph_matches_the_original_op_list(ops):
    # stacked, sliced, transposed weights: x . W_i^T + b_i
    g, feeds = attention_projection_graph(constant_weights=False)
    want = [feeds[5].float() @ feeds[0][i].float().t() + g.constants[200 + i].float() for i in range(4)]
    (plain,) = R.execute(g, feeds, DEV)
    R.apply_reference_passes(g)
    R.lower_to_hot_path(g)
    R.multi_stream_execution(g)
    assert "multi_stream" in g.types()
    (outs,) = R.execute(g, feeds, DEV)
    for o, p0, w in zip(outs, plain, want):
        assert float((o.float().cpu().reshape(-1) - w.reshape(-1)).abs().max()) <= 4e-3
        assert torch.equal(o.reshape(-1), p0.reshape(-1))
    # constant 2-D weights: SwapMatmulInputs puts the constant first without transposing it
    # (swap_matmul_inputs.cpp:74-78), so the rewritten graph computes (W_i . x^T)^T = x . W_i^T; the grouped launch must
    # give what the reference's rewritten graph gives op by op
    g, feeds = attention_projection_graph()
    R.apply_reference_passes(g)
    (ref,) = R.execute(g, feeds, DEV)
    R.lower_to_hot_path(g)
    R.multi_stream_execution(g)
    (outs,) = R.execute(g, feeds, DEV)
    x = feeds[0]
    for i, (o, r) in enumerate(zip(outs, ref)):
        w = x[i:i + 1].float() @ g.constants[100 + i].float().t() + g.constants[200 + i].float()
        assert list(o.shape) == [1, 512] and float((o.float().cpu() - w).abs().max()) <= 4e-3
        assert float((o.float() - r.float()).abs().max()) <= 2e-3


# ---- the decoder's per-token chain into one op ----------------------------------------------------------------------
def decoder_graph(seed=11, H=256, S=9, vocab=500, query_from_layer0=False, in0=None):
    """One token of a GNMT-style decoder as the interpreter sees it: four seq_len-1 cells, layers 1..3 on cat(previous
    output, context), residual adds around layers 2 and 3, the attention bmm, the classifier.  With `query_from_layer0`
    the attention weights are computed from layer 0's output (as in GNMT), otherwise they are a graph input."""
    from pimaicompiler_amd import workloads
    g = torch.Generator().manual_seed(seed)
    in0 = H if in0 is None else in0
    c, ops = {}, []
    X, ATT, ENC, KEYS = 0, 1, 2, 3
    for k in range(4):
        prm = workloads.lstm_inputs(seed + 10 + k, in0 if k == 0 else 2 * H, H, 1, False, 1)[0]
        for j, t in enumerate(prm):
            c[100 + 4 * k + j] = t
    c[200], c[201] = (0.05 * torch.randn(vocab, H, generator=g)).half(), (0.01 * torch.randn(vocab, generator=g)).half()
    y, hn, cn, lst, cat, res = (lambda k: 300 + k), (lambda k: 310 + k), (lambda k: 320 + k), (lambda k: 330 + k), (lambda k: 340 + k), (lambda k: 350 + k)
    CTX = 40
    ops.append(R.Op("aten::lstm", [X, 10, 20, 100, 101, 102, 103], [y(0), hn(0), cn(0)]))
    if query_from_layer0:
        ops.append(R.Op("aten::bmm", [y(0), KEYS], [41]))          # scores [1, 1, S] from layer 0's output
        ops.append(R.Op("aten::bmm", [41, ENC], [CTX]))
    else:
        ops.append(R.Op("aten::bmm", [ATT, ENC], [CTX]))
    prev = y(0)
    for k in range(1, 4):
        ops += [R.Op("prim::ListConstruct", [prev, CTX], [lst(k)]), R.Op("aten::cat", [lst(k)], [cat(k)], {"dim": 2}),
                R.Op("aten::lstm", [cat(k), 10 + k, 20 + k] + [100 + 4 * k + j for j in range(4)], [y(k), hn(k), cn(k)])]
        if k >= 2:
            ops.append(R.Op("aten::add", [y(k), prev], [res(k)]))
            prev = res(k)
        else:
            prev = y(k)
    ops.append(R.Op("aten::linear", [prev, 200, 201], [400]))
    inputs = [X, ENC] + ([KEYS] if query_from_layer0 else [ATT]) + [10 + k for k in range(4)] + [20 + k for k in range(4)]
    outputs = [400] + [hn(k) for k in range(4)] + [cn(k) for k in range(4)]
    feeds = {X: torch.randn(1, 1, in0, generator=g).half(), ENC: torch.randn(1, S, H, generator=g).half()}
    if query_from_layer0:
        feeds[KEYS] = (0.05 * torch.randn(1, H, S, generator=g)).half()
    else:
        feeds[ATT] = torch.softmax(torch.randn(1, 1, S, generator=g), -1).half()
    for k in range(4):
        feeds[10 + k] = (0.3 * torch.randn(1, 1, H, generator=g)).half()
        feeds[20 + k] = (0.3 * torch.randn(1, 1, H, generator=g)).half()
    return R.Graph(ops, inputs, outputs, c, next_id=500), feeds


def test_decoder_chain_becomes_one_op():
    g, _ = decoder_graph()
    R.fuse_decoder_step(g)
    assert g.types() == ["pimhip::decoder_step"]
    op = g.ops[0]
    assert op.attrs["num_layers"] == 4 and op.attrs["first_takes_context"] is False and op.attrs["first_residual_layer"] == 2
    assert op.attrs["context"] == "bmm" and op.attrs["classifier"] == (200, 201)
    assert op.inputs == [0, 1, 2, 10, 11, 12, 13, 20, 21, 22, 23]
    assert op.outputs == [300, 301, 352, 353, 310, 311, 312, 313, 320, 321, 322, 323, 400]
    assert op.attrs["params"] == list(range(100, 116))


def test_decoder_chain_starts_after_the_cell_the_attention_reads():
    """In GNMT the attention weights come from layer 0's output: layer 0 and the scores stay operators, the rest of the
    token (context bmm, three cells, two adds, classifier) is one op whose first cell takes cat(y0, ctx)."""
    g, _ = decoder_graph(query_from_layer0=True)
    R.fuse_decoder_step(g)
    assert g.types() == ["aten::lstm", "aten::bmm", "pimhip::decoder_step"]
    op = g.ops[2]
    assert op.attrs["num_layers"] == 3 and op.attrs["first_takes_context"] is True and op.attrs["first_residual_layer"] == 1
    assert op.attrs["context"] == "bmm" and op.inputs[:3] == [300, 41, 2]


def test_decoder_chain_guards():
    # a pre-residual y with a second consumer cannot be dropped: the chain ends before that cell's add
    g, _ = decoder_graph()
    g.ops.append(R.Op("aten::relu", [302], [450]))
    g.outputs.append(450)
    R.fuse_decoder_step(g)
    fused = [o for o in g.ops if o.type == "pimhip::decoder_step"]
    assert len(fused) == 1 and fused[0].attrs["num_layers"] == 3 and fused[0].attrs["classifier"] is None
    assert fused[0].attrs["first_residual_layer"] == 3                    # layers 0..2, none of them with a residual add
    assert [o.type for o in g.ops].count("aten::lstm") == 1 and "aten::linear" in g.types()
    # the context is used elsewhere too: it stays an operator and is handed to the fused op
    g, _ = decoder_graph()
    g.outputs.append(40)
    R.fuse_decoder_step(g)
    assert g.types() == ["aten::bmm", "pimhip::decoder_step"] and g.ops[1].attrs["context"] == "given" and g.ops[1].inputs[:2] == [0, 40]
    # weights that are not constants: nothing to fuse
    g, _ = decoder_graph()
    w = g.constants.pop(104)
    g.inputs.append(104)
    R.fuse_decoder_step(g)
    fused = [o for o in g.ops if o.type == "pimhip::decoder_step"]
    assert len(fused) == 1 and fused[0].attrs["num_layers"] == 2 and fused[0].inputs[0] == 301   # only layers 2 and 3
    assert w is not None
    # a single cell is left alone
    g, _ = decoder_graph()
    g.ops = g.ops[:1]
    g.outputs = [300]
    R.fuse_decoder_step(g)
    assert g.types() == ["aten::lstm"]
    # a cell whose initial state is computed from the cells below it (layer 2 starts from layer 1's hn): the fused op reads
    # every h0 / c0 before any cell runs, so the chain ends in front of that cell and nothing reads a tensor nobody makes
    g, _ = decoder_graph()
    cell2 = [o for o in g.ops if o.type == "aten::lstm"][2]
    cell2.inputs[1] = 311
    R.fuse_decoder_step(g)
    fused = [o for o in g.ops if o.type == "pimhip::decoder_step"]
    # (two steps of two cells: the second starts at that cell and reads the hn the first one produces)
    assert [f.attrs["num_layers"] for f in fused] == [2, 2] and fused[0].attrs["classifier"] is None
    assert 311 in fused[0].outputs and 311 in fused[1].inputs and fused[1].attrs["classifier"] == (200, 201)
    assert "aten::lstm" not in g.types()
    produced = set(g.inputs) | set(g.constants)
    for o in g.ops:
        assert all(t in produced for t in o.inputs), o
        produced.update(o.outputs)
    # a classifier-shaped linear whose weight is a constant without a value (not loaded yet) is not taken, and does not
    # make the pass fail
    g, _ = decoder_graph()
    g.constants[200] = None
    R.fuse_decoder_step(g)
    assert g.types() == ["pimhip::decoder_step", "aten::linear"] and g.ops[0].attrs["classifier"] is None


@pytest.mark.gpu
@pytest.mark.parametrize("query_from_layer0", [False, True])
def test_fused_decoder_graph_matches_the_operator_list_and_libtorch(ops, query_from_layer0):
    H, S = 256, 9
    g0, feeds = decoder_graph(H=H, S=S, query_from_layer0=query_from_layer0)
    want_ops = [t.float().cpu() for t in R.execute(g0, feeds, DEV)]
    g1, _ = decoder_graph(H=H, S=S, query_from_layer0=query_from_layer0)
    R.fuse_decoder_step(g1)
    assert "pimhip::decoder_step" in g1.types()
    for rep in range(2):                      # the second call reuses the op's plan (and, told so, the sentence's projection)
        got = [t.float().cpu() for t in R.execute(g1, feeds, DEV, same_sentence=rep > 0)]
        assert [list(t.shape) for t in got] == [list(t.shape) for t in want_ops]
        for a, b in zip(got, want_ops):
            assert float((a - b).abs().max()) <= 5e-3
    # LibTorch CPU on the same op list
    c = g0.constants
    f = {k: v for k, v in feeds.items()}
    cell = lambda k, inp: torch.lstm(inp, (f[10 + k], f[20 + k]), [c[100 + 4 * k + j] for j in range(4)], True, 1, 0.0, False, False, False)  # noqa: E731
    y0, hn0, cn0 = cell(0, f[0])
    att = torch.bmm(y0.float(), f[3].float()).half() if query_from_layer0 else f[1]
    ctx = torch.bmm(att.float(), f[2].float()).half()
    y1, hn1, cn1 = cell(1, torch.cat([y0, ctx], 2))
    y2, hn2, cn2 = cell(2, torch.cat([y1, ctx], 2))
    r2 = y2 + y1
    y3, hn3, cn3 = cell(3, torch.cat([r2, ctx], 2))
    r3 = y3 + r2
    logits = torch.nn.functional.linear(r3.float(), c[200].float(), c[201].float())
    for a, b in zip(got, [logits, hn0, hn1, hn2, hn3, cn0, cn1, cn2, cn3]):
        assert float((a - b.float()).abs().max()) <= 5e-3


# ---- consecutive sequence layers into one multi-layer op --------------------------------------------------------------
def encoder_graph(seed=21, H=128, T=12, residual_from=4, constant_state=False):
    """The GNMT encoder as the interpreter sees it: a bidirectional layer, then three one-direction layers, each an
    aten::lstm of its own reading the sequence before it (the first of them 2H wide); layers from `residual_from` on
    (2 in GNMT) with a residual sum around them."""
    from pimaicompiler_amd import workloads
    g = torch.Generator().manual_seed(seed)
    c, ops, feeds = {}, [], {}
    X = 0
    p0 = workloads.lstm_inputs(seed + 10, H, H, 1, True, T)[0]
    for j, t in enumerate(p0):
        c[100 + j] = t
    ops.append(R.Op("aten::lstm", [X, 10, 20] + [100 + j for j in range(8)], [300, 310, 320], {"bidirectional": True, "seq_len": T}))
    prev = 300
    for k in range(1, 4):
        prm = workloads.lstm_inputs(seed + 10 + k, 2 * H if k == 1 else H, H, 1, False, T)[0]
        for j, t in enumerate(prm):
            c[100 + 8 * k + j] = t
        ops.append(R.Op("aten::lstm", [prev, 10 + k, 20 + k] + [100 + 8 * k + j for j in range(4)], [300 + k, 310 + k, 320 + k], {"seq_len": T}))
        if k >= residual_from:
            ops.append(R.Op("aten::add", [300 + k, prev], [350 + k]))
            prev = 350 + k
        else:
            prev = 300 + k
    feeds[X] = torch.randn(T, 1, H, generator=g).half()
    feeds[10], feeds[20] = (0.3 * torch.randn(2, 1, H, generator=g)).half(), (0.3 * torch.randn(2, 1, H, generator=g)).half()
    inputs = [X, 10, 20]
    for k in range(1, 4):
        h, cc = (0.3 * torch.randn(1, 1, H, generator=g)).half(), (0.3 * torch.randn(1, 1, H, generator=g)).half()
        if constant_state:
            c[10 + k], c[20 + k] = h, cc
        else:
            feeds[10 + k], feeds[20 + k] = h, cc
            inputs += [10 + k, 20 + k]
    outputs = [prev, 312, 322, 313]
    return R.Graph(ops, inputs, outputs, c, next_id=500), feeds


def test_sequence_layers_become_one_multi_layer_op():
    g, _ = encoder_graph()
    R.fuse_lstm_stack(g)
    assert g.types() == ["aten::lstm", "prim::ListConstruct", "aten::cat", "prim::ListConstruct", "aten::cat", "aten::lstm",
                         "aten::slice", "aten::slice", "aten::slice"]
    fused = g.ops[5]
    assert fused.attrs["num_layers"] == 3 and fused.inputs[0] == 300 and fused.outputs[0] == 303
    assert fused.inputs[3:] == [108 + j for j in range(4)] + [116 + j for j in range(4)] + [124 + j for j in range(4)]
    assert g.ops[1].inputs == [11, 12, 13] and g.ops[3].inputs == [21, 22, 23]
    assert [(o.outputs[0], o.inputs[0] == fused.outputs[1 if o.outputs[0] < 320 else 2], o.attrs["start"]) for o in g.ops[6:]] == \
        [(312, True, 1), (322, True, 1), (313, True, 2)]
    # an initial state of constants is stacked at rewrite time
    g, _ = encoder_graph(constant_state=True)
    R.fuse_lstm_stack(g)
    assert g.types() == ["aten::lstm", "aten::lstm", "aten::slice", "aten::slice", "aten::slice"]
    h_all = g.constants[g.ops[1].inputs[1]]
    assert list(h_all.shape) == [3, 1, 128] and torch.equal(h_all[1:2], g.constants[12])


def test_sequence_layer_chain_guards():
    # residual sums (GNMT: around the two upper layers) go into the fused op
    g, _ = encoder_graph(residual_from=2)
    R.fuse_lstm_stack(g)
    assert g.types()[:5] == ["aten::lstm", "prim::ListConstruct", "aten::cat", "prim::ListConstruct", "aten::cat"]
    fused = g.ops[5]
    assert fused.type == "pimhip::lstm_stack" and fused.attrs["num_layers"] == 3 and fused.attrs["first_residual_layer"] == 1
    assert fused.inputs[0] == 300 and fused.outputs[0] == 353 and "aten::add" not in g.types()
    # ... unless the sum is not of the layer's own input, or y is read before the sum, or a plain layer follows
    g, _ = encoder_graph(residual_from=3)
    g.ops[4].inputs = [303, 301]                    # add(y3, y1): not a residual sum of layer 3
    R.fuse_lstm_stack(g)
    fused = [o for o in g.ops if o.attrs.get("num_layers", 1) > 1]
    assert len(fused) == 1 and fused[0].type == "aten::lstm" and fused[0].attrs["num_layers"] == 2 and "aten::add" in g.types()
    g, _ = encoder_graph(residual_from=3)
    g.ops.append(R.Op("aten::relu", [303], [450]))  # y3 itself is read
    g.outputs.append(450)
    R.fuse_lstm_stack(g)
    fused = [o for o in g.ops if o.attrs.get("num_layers", 1) > 1]
    assert len(fused) == 1 and fused[0].type == "aten::lstm" and fused[0].attrs["num_layers"] == 2 and "aten::add" in g.types()
    g, _ = encoder_graph(residual_from=2)
    g.ops = [o for o in g.ops if not (o.type == "aten::add" and o.outputs[0] == 353)]   # layer 3 plain above layer 2 with a sum
    g.ops[-1].inputs[0] = 352
    g.outputs[0] = 303
    R.fuse_lstm_stack(g)
    fused = [o for o in g.ops if o.attrs.get("num_layers", 1) > 1]
    assert len(fused) == 1 and fused[0].type == "pimhip::lstm_stack" and fused[0].attrs["num_layers"] == 2 and fused[0].outputs[0] == 352
    assert [o.type for o in g.ops].count("aten::lstm") == 2
    # a sequence in between that is a graph output stays a tensor of its own
    g, _ = encoder_graph()
    g.outputs.append(302)
    R.fuse_lstm_stack(g)
    fused = [o for o in g.ops if o.type == "aten::lstm" and o.attrs.get("num_layers", 1) > 1]
    assert len(fused) == 1 and fused[0].attrs["num_layers"] == 2 and fused[0].outputs[0] == 302
    # a final state that is read before the chain ends: the chain ends at that reader
    g, _ = encoder_graph()
    g.ops.insert(2, R.Op("aten::relu", [311], [450]))
    g.outputs.append(450)
    R.fuse_lstm_stack(g)
    fused = [o for o in g.ops if o.type == "aten::lstm" and o.attrs.get("num_layers", 1) > 1]
    assert len(fused) == 1 and fused[0].attrs["num_layers"] == 2 and fused[0].inputs[0] == 301 and fused[0].outputs[0] == 303
    # weights that are graph inputs, single-step cells and bidirectional layers are not taken
    g, _ = encoder_graph()
    g.constants.pop(117)
    g.inputs.append(117)
    R.fuse_lstm_stack(g)
    assert all(o.attrs.get("num_layers", 1) == 1 for o in g.ops)
    g, _ = decoder_graph()
    before = g.types()
    R.fuse_lstm_stack(g)
    assert g.types() == before


@pytest.mark.gpu
@pytest.mark.parametrize("H,T,residual_from", [(128, 12, 4), (1024, 24, 4), (128, 12, 2), (1024, 50, 2), (256, 20, 3)])
def test_fused_sequence_layers_match_the_operator_list_and_libtorch(ops, H, T, residual_from):
    g0, feeds = encoder_graph(H=H, T=T, residual_from=residual_from)
    want_ops = [t.float().cpu() for t in R.execute(g0, feeds, DEV)]
    g1, _ = encoder_graph(H=H, T=T, residual_from=residual_from)
    R.fuse_lstm_stack(g1)
    assert [o.attrs.get("num_layers", 1) for o in g1.ops if o.type in ("aten::lstm", "pimhip::lstm_stack")] == [1, 3]
    got = [t.float().cpu() for t in R.execute(g1, feeds, DEV)]
    assert [list(t.shape) for t in got] == [list(t.shape) for t in want_ops]
    for a, b in zip(got, want_ops):
        assert float((a - b).abs().max()) <= 5e-3
    # LibTorch CPU on the original op list
    c, f = g0.constants, feeds
    y, _, _ = torch.lstm(f[0], (f[10], f[20]), [c[100 + j] for j in range(8)], True, 1, 0.0, False, True, False)
    finals = {}
    for k in range(1, 4):
        yk, hn, cn = torch.lstm(y, (f[10 + k], f[20 + k]), [c[100 + 8 * k + j] for j in range(4)], True, 1, 0.0, False, False, False)
        finals[310 + k], finals[320 + k] = hn, cn
        y = yk + y if k >= residual_from else yk
    for a, b in zip(got, [y, finals[312], finals[322], finals[313]]):
        assert list(a.shape) == list(b.shape) and float((a - b.float()).abs().max()) <= 5e-3
