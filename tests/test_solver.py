"""Solver-side host logic on the CPU: graph tracing, solver-graph construction and the
schedule ILP, with synthetic operator costs instead of GPU measurements."""
import math

import numpy as np
import pytest
import torch
import torch.nn as nn

from monet_amd.graph import ComputeNode, Graph, Input, Param
from monet_amd.solver import CPU_GCD_MULTIPLIER, Model
from monet_amd.solver_info import BwdNode, FwdNode, IntNode, SolverInfo


class SmallNet(nn.Module):
    def __init__(self):
        super().__init__()
        self.c1 = nn.Conv2d(3, 8, 3, padding=1, bias=False)
        self.b1 = nn.BatchNorm2d(8)
        self.r = nn.ReLU(inplace=True)
        self.mp = nn.MaxPool2d(3, 2, 1)
        self.c2 = nn.Conv2d(8, 8, 3, padding=1, bias=True)
        self.b2 = nn.BatchNorm2d(8)
        self.ap = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Linear(8, 5)

    def forward(self, x):
        x = self.mp(self.r(self.b1(self.c1(x))))
        y = self.b2(self.c2(x))
        y += x
        y = self.r(y)
        return self.fc(torch.flatten(self.ap(y), 1))


def synthetic_cost(si):
    """Costs proportional to output size: ms = MB, workspace 0; one entry per variant."""
    def fn(n, op, bwd_op):
        mb = abs(np.prod(n.shape)) * 4 * si.bs / 1e6
        conv = si.select_conv_algo and n.op == "aten::_convolution"
        if conv:
            nf = op.n_fwd_algos()
            nb = op.n_bwd_ip_algos() if bwd_op == "ip_grad" else op.n_bwd_wt_algos()
            return ([0.0] * nf, [0.1 * c for c in range(nb)], []), \
                   ([mb] * nf, [mb * (1.0 - 0.1 * c) for c in range(nb)], [])
        if si.do_inplace and hasattr(op, 'inplace'):
            return ([0.0, 0.0], [0.0], []), ([0.1 * mb, 0.1 * mb], [0.1 * mb], [])
        if n.op in ("aten::batch_norm", "monet::batch_norm_relu", "monet::batch_norm_add_relu"):
            return ([0.0], [0.0], [0.0]), ([0.2 * mb], [0.3 * mb], [0.1 * mb])
        # implementations that keep an intermediate are a bit slower
        extra = 0.02 * mb if "Binary" in type(op).__name__ or "Indices" in type(op).__name__ else 0
        return ([0.0], [0.0], []), ([0.1 * mb + extra], [0.1 * mb + extra], [])
    return fn


def build(mode, bs=16):
    torch.manual_seed(0)
    g = Graph.create(SmallNet(), (3, 16, 16))
    si = SolverInfo(bs, "small", mode)
    si.extract(g, cost_fn=synthetic_cost(si))
    return g, si


def test_graph_trace():
    g = Graph.create(SmallNet(), (3, 16, 16))
    kinds = [n.op for n in g.nodes if isinstance(n, ComputeNode)]
    assert kinds == ["aten::_convolution", "aten::batch_norm", "aten::relu_", "aten::max_pool2d",
                     "aten::_convolution", "aten::batch_norm", "aten::add_", "aten::relu_",
                     "aten::adaptive_avg_pool2d", "aten::flatten", "aten::linear"]
    assert isinstance(g.nodes[0], Input) and g.nodes[0].shape == [-1, 3, 16, 16]
    conv1 = next(n for n in g.nodes if isinstance(n, ComputeNode))
    assert conv1.shape == [-1, 8, 16, 16] and conv1.has_backward
    # the data input carries no gradient, the weight does
    assert conv1.dependencies[0][1] is False and conv1.dependencies[1][1] is True
    assert len(conv1.args) == 13 and conv1.args[3].value == [1, 1]
    assert g._outputs == [len(g.nodes) - 1]


def test_solver_graph_structure():
    g, si = build("inplace_conv_multiway_newnode")
    fwd = [n for n in si.nodes.values() if isinstance(n, FwdNode) and not isinstance(n, IntNode)]
    ints = [n for n in si.nodes.values() if isinstance(n, IntNode)]
    bwd = [n for n in si.nodes.values() if isinstance(n, BwdNode)]
    assert len(fwd) == 11 + 1          # operators + loss
    assert len(ints) == 3              # two ReLU masks, one pool index tensor
    assert len(bwd) == 11 + 2 + 1      # + param_grad nodes of 2 convs and the linear layer
    assert si.select_conv_algo and si.do_inplace and si.compute_newnode
    assert si.mode == "conv_multiway_newnode"
    # intermediate sizes: packed bits / nibbles, per sample, times batch
    relu_int = si.nodes[si.nodes[2].intermediates[0][1]]
    assert relu_int.mem == 16 * (8 * 16 * 16) // 8
    pool_int = si.nodes[si.nodes[si.graph_to_solver[19]].intermediates[0][1]]
    assert pool_int.mem == 16 * (8 * 8 * 8) // 2
    # ReLU backward: three implementations with input / output / intermediate dependencies
    rb = si.nodes[si.fwd_to_bwd[2]]
    assert [d[0] for d in rb.dep_list_fwd] == [1, 2, si.nodes[2].intermediates[0][1]]
    # conv: the parameter-gradient node needs the layer input, the input-gradient node does not
    cb = si.fwd_to_bwd[si.graph_to_solver[20]]
    assert si.nodes[cb].bwd_op == "ip_grad" and si.nodes[cb - 1].bwd_op == "param_grad"
    assert si.nodes[cb - 1].dep_list_fwd[0] == [si.graph_to_solver[19]]
    assert si.nodes[cb].dep_list_fwd[0] == []
    # in-place candidates: the ReLUs and the residual add (and the ReLU intermediates)
    ops = sorted(si.nodes[v].op for v in si.inplace_list)
    assert ops.count("aten::relu_") == 2 and "aten::add_" in ops


def peak_of(si, sol):
    """Memory (KB) of the forward pass under a solution: stored + live tensors, coarse check."""
    V = si.loss + 1
    return sum(sol.s[1][i] * si.nodes[i].mem for i in range(V)) / 1024


@pytest.mark.parametrize("mode", ["normal", "multiway_newnode", "inplace_conv_multiway_newnode"])
def test_ilp_unconstrained_stores_and_never_recomputes(mode):
    g, si = build(mode)
    sol = Model(si, budget=1.0, time_limit=120, mip_rel_gap=0.0).solve()
    V, T = si.loss + 1, len(si.nodes) - si.loss
    assert sol.r.shape == (T, V) and sol.s.shape == (T + 1, V) and sol.m.shape == (T, 3)
    non_int = [i for i in range(V) if not isinstance(si.nodes[i], IntNode)]
    assert all(sol.r[0][i] == 1 for i in non_int)
    # memory is free, so nothing that costs time is recomputed
    cost = np.array([max(si.nodes[i].workspace_compute, default=0) for i in range(V)])
    assert (sol.r[1:] * cost).sum() == 0
    assert (sol.m.sum(axis=1) >= 1).all()
    if "conv" in mode:
        # every backward conv step picked exactly one variant, the cheapest one
        for i, k in si.conv_list.items():
            if i > si.loss:
                t = i + 1 - V
                # (directions differ in how many variants they have; the model rounds costs,
                # so two variants can tie)
                cost_i = [math.ceil(v * CPU_GCD_MULTIPLIER) for v in si.nodes[i].workspace_compute]
                assert sol.rf[t, k].sum() == 1
                assert cost_i[int(np.argmax(sol.rf[t, k]))] == min(cost_i)


def test_ilp_budget_forces_cheaper_storage_or_recomputation():
    g, si = build("inplace_conv_multiway_newnode", bs=64)
    free = Model(si, budget=1.0, time_limit=120, mip_rel_gap=0.0).solve()
    # walk the budget (MB) down to the last feasible one
    feasible = None
    for mb in [4, 2.4, 2.2, 2.0, 1.8, 1.7, 1.6]:
        try:
            sol = Model(si, budget=mb / 1024.0, time_limit=120, mip_rel_gap=0.0).solve()
            feasible = (mb, sol)
        except ValueError:
            break
    assert feasible is not None
    mb, tight = feasible
    assert mb < 2.0 and tight.runtime_expected > free.runtime_expected
    # a tight budget recomputes something or keeps compact intermediates instead of activations
    V = si.loss + 1
    ints = [i for i in range(V) if isinstance(si.nodes[i], IntNode)]
    assert tight.r[1:].sum() > 0 or tight.s[:, ints].sum() > 0 or tight.ip.sum() > 0
    assert tight.s[1:].sum() <= free.s[1:].sum() or tight.runtime_expected > free.runtime_expected


def test_ilp_infeasible_budget_raises():
    g, si = build("normal")
    with pytest.raises(ValueError):
        Model(si, budget=1e-6, time_limit=60).solve()


# ---------------------------------------------------------------- compiled plans
from monet_amd.schedule import Schedule  # noqa: E402
from plan_memory import replay  # noqa: E402


@pytest.mark.parametrize("mode", ["normal", "multiway_newnode", "inplace_conv_multiway_newnode"])
def test_compiled_plan_is_consistent_and_within_budget(mode):
    """Every solution must compile (all operands present when an instruction needs them) and
    the bytes the executor would hold must stay within what the ILP was given."""
    g, si = build(mode, bs=64)
    seen = 0
    for mb in [4, 2.4, 2.2, 2.0, 1.8, 1.7, 1.6]:
        try:
            sol = Model(si, budget=mb / 1024.0, time_limit=120, mip_rel_gap=0.0).solve()
        except ValueError:
            break
        sched = Schedule(g, si)
        sched.init_schedule(sol, si.mode)
        peak, _ = replay(sched, 64)
        assert peak <= mb * 2**20 * 1.001, (mode, mb, peak / 2**20)
        seen += 1
    assert seen >= 5


def test_recompute_window_is_a_restriction_of_the_exact_model():
    """The windowed model must stay feasible where the exact one is and can only cost more."""
    g, si = build("multiway_newnode", bs=64)
    for mb in (2.4, 2.0, 1.7):
        exact = Model(si, budget=mb / 1024.0, time_limit=120, mip_rel_gap=0.0).solve()
        windowed = Model(si, budget=mb / 1024.0, time_limit=120, mip_rel_gap=0.0,
                         recompute_window=4).solve()
        assert windowed.runtime_expected >= exact.runtime_expected
        sched = Schedule(g, si)
        sched.init_schedule(windowed, si.mode)
        peak, _ = replay(sched, 64)
        assert peak <= mb * 2**20 * 1.001
        # nothing further than the window below the step's own operator is recomputed
        V = si.loss + 1
        for t in range(1, windowed.r.shape[0]):
            f = si.bwd_to_fwd[V + t - 1]
            assert windowed.r[t][:max(0, f - 4)].sum() == 0


def test_peak_minimisation_finds_the_floor():
    g, si = build("multiway_newnode", bs=64)
    floor = Model(si, budget=None, time_limit=120, mip_rel_gap=0.0).solve()
    gb = floor.runtime_expected  # objective = peak in GB (+ a negligible run-time tie-break)
    assert 1.6 / 1024 < gb < 1.7 / 1024


def test_tight_budget_fallback_returns_a_schedule_within_the_real_budget(monkeypatch):
    """If the direct solve ends without a fitting incumbent, the tightening-target fallback
    must still return a schedule whose replayed peak is within the REAL budget."""
    from monet_amd import solver as S
    g, si = build("multiway_newnode", bs=64)
    mb = 1.8
    real_solve = S.Model.solve
    calls = {"n": 0}

    def first_call_fails(self, out_file=None):
        calls["n"] += 1
        if calls["n"] == 1:
            self.last_excess = 0.05 * self.budget
            raise ValueError("Model infeasible: the cheapest schedule found needs more")
        return real_solve(self, out_file)

    monkeypatch.setattr(S.Model, "solve", first_call_fails)
    sol = S.solve_within_budget(si, mb / 1024.0, time_limit=300, mip_rel_gap=0.0)
    assert calls["n"] >= 2
    sched = Schedule(g, si)
    sched.init_schedule(sol, si.mode)
    peak, _ = replay(sched, 64)
    assert peak <= mb * 2**20 * 1.001
    # and a budget below the floor is still reported as infeasible
    with pytest.raises(ValueError):
        S.solve_within_budget(si, 1.0 / 1024.0, time_limit=60, mip_rel_gap=0.0, rounds=2)


def test_model_definitions_trace_to_the_expected_operators():
    """The two benchmark networks, traced on the CPU: operator counts of the torchvision
    ResNet-50 topology and of the U-Net, and the solver graph sizes that follow."""
    from collections import Counter
    from monet_amd.models import build_model
    model, shape, name = build_model("torchvision.models.resnet50()")
    assert name == "resnet50" and shape == (3, 224, 224)
    assert sum(p.numel() for p in model.parameters()) == 25557032
    g = Graph.create(model, shape)
    from collections import Counter
    ops = Counter(n.op for n in g.nodes if isinstance(n, ComputeNode))
    assert ops == {"aten::_convolution": 53, "aten::batch_norm": 53, "aten::relu_": 49,
                   "aten::add_": 16, "aten::max_pool2d": 1, "aten::adaptive_avg_pool2d": 1,
                   "aten::flatten": 1, "aten::linear": 1}
    si = SolverInfo(184, name, "inplace_conv_multiway_newnode")
    si.extract(g, cost_fn=synthetic_cost(si))
    assert si.loss == 225 and len(si.nodes) == 455
    assert len(si.conv_list) == 53 * 3 and len(si.inplace_list) == (49 + 16) + 49

    unet, ushape, uname = build_model("unet")
    assert uname == "unet" and ushape == (3, 416, 608)
    gu = Graph.create(unet, ushape)
    uops = Counter(n.op for n in gu.nodes if isinstance(n, ComputeNode))
    assert uops == {"aten::_convolution": 19, "aten::batch_norm": 18, "aten::relu_": 18,
                    "aten::max_pool2d": 4, "aten::adaptive_avg_pool2d": 4, "aten::cat": 4}


def test_batch_norm_relu_fusion_pass():
    """BatchNorm nodes whose only reader is a ReLU merge with it; others stay."""
    g = Graph.create(SmallNet(), (3, 16, 16))
    f = Graph.create(SmallNet(), (3, 16, 16), fuse_bn_relu=True)
    kinds = [n.op for n in f.nodes if isinstance(n, ComputeNode)]
    # b1 -> relu fuses; b2 feeds the residual add, so it stays a plain BatchNorm, and the add
    # fuses with the ReLU behind it
    assert kinds == ["aten::_convolution", "monet::batch_norm_relu", "aten::max_pool2d",
                     "aten::_convolution", "aten::batch_norm", "monet::add_relu",
                     "aten::adaptive_avg_pool2d", "aten::flatten", "aten::linear"]
    assert len(f.nodes) == len(g.nodes) - 2 and f._outputs == [len(f.nodes) - 1]
    pool = next(n for n in f.nodes if isinstance(n, ComputeNode) and n.op == "aten::max_pool2d")
    fused = f.nodes[pool.args[0].index]
    assert fused.op == "monet::batch_norm_relu" and len(fused.args) == 9  # the BatchNorm's arguments
    si = SolverInfo(16, "small", "fused_inplace_conv_multiway_newnode")
    si.extract(f, cost_fn=synthetic_cost(si))
    assert si.fuse_bn_relu and si.mode == "conv_multiway_newnode"
    sol = Model(si, budget=1.0, time_limit=60, mip_rel_gap=0.0).solve()
    Schedule(f, si).init_schedule(sol, si.mode)


def test_batch_norm_add_relu_fusion_pass():
    """Second fusion level: the BatchNorm in front of a residual add + ReLU joins them."""
    f1 = Graph.create(SmallNet(), (3, 16, 16), fuse_bn_relu=1)
    f2 = Graph.create(SmallNet(), (3, 16, 16), fuse_bn_relu=2)
    kinds = [n.op for n in f2.nodes if isinstance(n, ComputeNode)]
    assert kinds == ["aten::_convolution", "monet::batch_norm_relu", "aten::max_pool2d",
                     "aten::_convolution", "monet::batch_norm_add_relu",
                     "aten::adaptive_avg_pool2d", "aten::flatten", "aten::linear"]
    assert len(f2.nodes) == len(f1.nodes) - 1 and f2._outputs == [len(f2.nodes) - 1]
    triple = next(n for n in f2.nodes if isinstance(n, ComputeNode) and
                  n.op == "monet::batch_norm_add_relu")
    # the BatchNorm's nine arguments, then the add's second operand and factor
    assert len(triple.args) == 11
    assert f2.nodes[triple.args[0].index].op == "aten::_convolution"
    assert f2.nodes[triple.args[9].index].op == "aten::max_pool2d"
    assert isinstance(triple.args[10], ComputeNode.V) and triple.args[10].value == 1
    assert [d for d, _ in triple.dependencies][:5] == [a.index for a in triple.args[:5]]
    si = SolverInfo(16, "small", "fused2_inplace_conv_multiway_newnode")
    si.extract(f2, cost_fn=synthetic_cost(si))
    assert si.fuse_bn_relu == 2 and si.mode == "conv_multiway_newnode"
    sol = Model(si, budget=1.0, time_limit=60, mip_rel_gap=0.0).solve()
    Schedule(f2, si).init_schedule(sol, si.mode)
    # ResNet-50: every block's last BatchNorm joins its add + ReLU (16), the downsample
    # BatchNorms (second operand of the add) stay
    from monet_amd.models import build_model
    model, shape, _ = build_model("resnet50")
    g = Graph.create(model, shape, fuse_bn_relu=2)
    from collections import Counter
    ops = Counter(n.op for n in g.nodes if isinstance(n, ComputeNode))
    assert ops["monet::batch_norm_add_relu"] == 16 and ops["monet::add_relu"] == 0
    assert ops["aten::batch_norm"] == 4 and ops["monet::batch_norm_relu"] == 33


def test_solver_sizes_follow_the_element_size_of_the_profiled_tensors():
    """A model profiled on bf16 tensors budgets 2 bytes per element for activations,
    parameters and gradients; compact intermediates (1 bit / 4 bits per element) stay as
    they are (the reference fixes 4 bytes, monet/solver_info.py:10)."""
    g = Graph.create(SmallNet(), (3, 16, 16))

    def sizes(first_arg):
        si = SolverInfo(16, "small", "multiway_newnode")
        si.extract(g, first_arg, cost_fn=synthetic_cost(si))
        return si
    f32 = sizes(torch.zeros(1))
    b16 = sizes(torch.zeros(1, dtype=torch.bfloat16))
    assert f32.elem_bytes == 4 and b16.elem_bytes == 2
    for i in f32.nodes:
        a, b = f32.nodes[i], b16.nodes[i]
        if isinstance(a, IntNode):
            assert a.mem == b.mem and a.mem > 0
        else:
            assert a.mem == 2 * b.mem
        assert a.fixed_mem == 2 * b.fixed_mem


class TinyNet(nn.Module):
    """Four operators: small enough to enumerate every schedule."""
    def __init__(self):
        super().__init__()
        self.c1 = nn.Conv2d(3, 6, 3, padding=1, bias=False)
        self.r = nn.ReLU()
        self.mp = nn.MaxPool2d(2, 2)
        self.fc = nn.Linear(6 * 4 * 4, 5)

    def forward(self, x):
        return self.fc(torch.flatten(self.mp(self.r(self.c1(x))), 1))


@pytest.mark.parametrize("mode", ["normal", "multiway"])
def test_ilp_optimum_equals_the_enumerated_optimum_on_a_tiny_graph(mode):
    """The restated ILP (with its reductions) against the reference's formulation evaluated on
    every schedule of a 6-node graph: same optimal run time at every budget from generous to the
    floor, and infeasible at the same budgets."""
    from brute_force_schedule import optimum
    torch.manual_seed(0)
    g = Graph.create(TinyNet(), (3, 8, 8))
    si = SolverInfo(64, "tiny", mode)

    def cost(n, op, bwd_op):   # uneven costs, so that what is recomputed matters
        mb = abs(np.prod(n.shape)) * 4 * si.bs / 1e6
        k = 1.0 + 0.37 * (len(n.op) % 5)
        # implementations that get by with less stored data are slower
        name = type(op).__name__
        k *= 1.25 if name.startswith(("OutputAct", "BinaryAct", "IndicesAct")) else 1.0
        return ([0.0], [0.0], []), ([k * mb], [0.7 * k * mb], [])
    si.extract(g, cost_fn=cost)
    V = si.loss + 1
    assert V <= 7
    seen_feasible = seen_infeasible = 0
    costs = []
    # (KB) generous, around the point where storing everything stops fitting, just above and just
    # below the floor of 341 KB
    for kb in (4096, 365, 342, 335):
        gb = kb / 1024.0 / 1024.0
        exact = optimum(si, gb)
        try:
            sol = Model(si, budget=gb, time_limit=120, mip_rel_gap=0.0).solve()
        except ValueError:
            sol = None
        if exact is None:
            assert sol is None, (mode, kb)
            seen_infeasible += 1
        else:
            assert sol is not None, (mode, kb)
            assert abs(sol.runtime_expected - exact) <= 1e-6 * max(1.0, exact), (mode, kb, sol.runtime_expected, exact)
            seen_feasible += 1
            costs.append(exact)
    assert seen_feasible == 3 and seen_infeasible == 1
    assert costs[-1] > costs[0]       # a tight budget costs run time: the comparison is not trivial
    # a cutoff row at a known schedule's run time: the optimum is still found when it lies below
    # the cutoff, and nothing is found when the cutoff is below the optimum
    from monet_amd.solver import CPU_GCD_MULTIPLIER
    gb = 342 / 1024.0 / 1024.0
    best_ms = costs[-1] / CPU_GCD_MULTIPLIER
    sol = Model(si, budget=gb, time_limit=120, mip_rel_gap=0.0, cutoff_ms=best_ms * 1.0001).solve()
    assert abs(sol.runtime_expected - costs[-1]) <= 1e-6 * max(1.0, costs[-1])
    with pytest.raises(ValueError):
        Model(si, budget=gb, time_limit=120, mip_rel_gap=0.0, cutoff_ms=best_ms * 0.99).solve()
