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
