"""Executor parity on the GPU: a model run through a solved schedule must give the
output and parameter gradients stock autograd gives, at a generous budget (nothing
recomputed) and at tight ones (recomputation, compact intermediates, in-place)."""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

pytestmark = pytest.mark.gpu


class SmallNet(nn.Module):
    def __init__(self):
        super().__init__()
        self.c1 = nn.Conv2d(3, 16, 3, padding=1, bias=False)
        self.b1 = nn.BatchNorm2d(16)
        self.r = nn.ReLU(inplace=True)
        self.mp = nn.MaxPool2d(3, 2, 1)
        self.c2 = nn.Conv2d(16, 16, 3, padding=1, bias=True)
        self.b2 = nn.BatchNorm2d(16)
        self.c3 = nn.Conv2d(16, 16, 1, bias=False)
        self.b3 = nn.BatchNorm2d(16)
        self.ap = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Linear(16, 5)

    def forward(self, x):
        x = self.mp(self.r(self.b1(self.c1(x))))
        y = self.r(self.b2(self.c2(x)))
        y = self.b3(self.c3(y))
        y += x
        y = self.r(y)
        return self.fc(torch.flatten(self.ap(y), 1))


def _solve(model, shape, bs, mode, budget_gb, cuda):
    from monet_amd.graph import Graph, fusion_level
    from monet_amd.solver import Model
    from monet_amd.solver_info import SolverInfo
    graph = Graph.create(copy.deepcopy(model).cpu(), shape, fuse_bn_relu=fusion_level(mode))
    x = torch.randn((bs,) + shape, device=cuda)
    si = SolverInfo(bs, "test", mode)
    si.extract(graph, x, *list(model.state_dict(keep_vars=True).values()))
    sol = Model(si, budget_gb, time_limit=120, mip_rel_gap=0.0).solve()
    return graph, si, sol


def _reference_grads(model, x, gout):
    ref = copy.deepcopy(model)
    y = ref(x)
    y.backward(gout)
    return y.detach(), {n: p.grad.clone() for n, p in ref.named_parameters()}, ref


def _rel(a, b, floor=1e-30):
    return float((a - b).abs().max() / b.abs().max().clamp_min(floor))


@pytest.mark.parametrize("mode", ["normal", "multiway_newnode", "conv_multiway_newnode",
                                  "inplace_conv_multiway_newnode",
                                  "fused_inplace_conv_multiway_newnode",
                                  "fused2_inplace_conv_multiway_newnode"])
def test_schedule_matches_autograd(cuda, mode, monkeypatch):
    from monet_amd.schedule import Schedule
    if mode == "normal":
        # without kernel selection by the solver a convolution times its variants on first use
        # and keeps the fastest (the reference's cuDNN benchmark mode); pinned here so that
        # every schedule below runs the same kernels
        from monet_amd.lm_ops import conv as conv_mod
        monkeypatch.setattr(conv_mod, "_autotune", lambda n_variants, run: conv_mod.DEFAULT_VARIANT)
    torch.manual_seed(0)
    bs, shape = 32, (3, 32, 32)
    model = SmallNet().to(cuda).train()
    graph, si, free = _solve(model, shape, bs, mode, 1.0, cuda)
    # budgets from generous down to the tightest feasible one
    peak_mb = None
    solutions = [("free", free)]
    from monet_amd.solver import Model
    for frac in (0.95, 0.9, 0.8, 0.65, 0.55, 0.5, 0.45):
        total = sum(n.mem for i, n in si.nodes.items() if i < si.loss) + si.nodes[si.loss].fixed_mem
        try:
            solutions.append(("%.2f" % frac,
                              Model(si, frac * total / 2**30, time_limit=120, mip_rel_gap=0.0).solve()))
        except ValueError:
            break
    assert len(solutions) >= 2
    x = torch.randn((bs,) + shape, device=cuda)
    gout = torch.randn(bs, 5, device=cuda)
    unconstrained = None   # output under the first ("free") solution
    for name, sol in solutions:
        print("case", mode, name, "recomputations", int(sol.r[1:].sum()), flush=True)
        m = copy.deepcopy(model)
        y_ref, g_ref, ref = _reference_grads(m, x, gout)
        sched = Schedule(graph, si)
        sched.init_schedule(sol, si.mode)
        # a bias in front of a BatchNorm has an exactly zero gradient: both sides then hold
        # rounding noise only, which a floor tied to the largest gradient lets through
        floor = 1e-2 * max(float(g.abs().max()) for g in g_ref.values())
        for step in range(2):  # a second step must not see state of the first
            for p in m.parameters():
                p.grad = None
            if step == 1:
                m.load_state_dict(model.state_dict())
            y = sched.forward(x, *list(m.state_dict(keep_vars=True).values()))
            assert _rel(y, y_ref) < 1e-5
            sched.backward(gout.clone())
            worst = 0.0
            for n, p in m.named_parameters():
                assert p.grad is not None, n
                worst = max(worst, _rel(p.grad, g_ref[n], floor))
            print("achieved", mode, name, "step", step, "largest gradient difference to stock fp32 "
                  "%.2e" % worst, flush=True)
            # two fp32 evaluations of a 10-operator network with batch statistics: summation
            # orders differ (achieved: a few 1e-6)
            assert worst < 5e-5, (mode, name, worst)
        # "normal" has one implementation per operator and no kernel variants: a tighter budget
        # only changes what is stored and what is computed again, from the same values with the
        # same reproducible forward kernels, so the output equals the unconstrained schedule's
        # bit for bit (gradients do not: backward convolutions add split reductions with atomics)
        if mode == "normal":
            if unconstrained is None:
                unconstrained = y.clone()
            else:
                assert torch.equal(y, unconstrained), (name, "output")
                print("achieved normal", name, "output bit-identical to the unconstrained schedule",
                      flush=True)
        # running statistics advanced exactly once per step, like the stock model's
        assert _rel(m.b1.running_mean, ref.b1.running_mean) < 1e-5
        assert _rel(m.b3.running_var, ref.b3.running_var) < 1e-5


def test_wrapper_trains_like_the_plain_model(cuda, tmp_path):
    import pickle
    from monet_amd.monet_wrapper import MONeTWrapper
    torch.manual_seed(1)
    bs, shape = 16, (3, 32, 32)
    model = SmallNet().to(cuda).train()
    graph, si, sol = _solve(model, shape, bs, "inplace_conv_multiway_newnode", 1.0, cuda)
    total = sum(n.mem for i, n in si.nodes.items() if i < si.loss) + si.nodes[si.loss].fixed_mem
    from monet_amd.solver import Model
    for frac in (0.5, 0.6, 0.7, 0.85):   # the tightest of these that is feasible
        try:
            sol = Model(si, frac * total / 2**30, time_limit=120, mip_rel_gap=0.0).solve()
            break
        except ValueError:
            continue
    path = tmp_path / "solution.pkl"
    with open(path, "wb") as f:
        pickle.dump([si, sol], f)
    plain = copy.deepcopy(model)
    wrapped = MONeTWrapper(copy.deepcopy(model), str(path), shape).to(cuda)
    wrapped.train()
    opt_a = torch.optim.SGD(plain.parameters(), lr=0.05, momentum=0.9)
    opt_b = torch.optim.SGD(wrapped.parameters(), lr=0.05, momentum=0.9)
    crit = nn.CrossEntropyLoss()
    for step in range(3):
        x = torch.randn((bs,) + shape, device=cuda)
        t = torch.randint(0, 5, (bs,), device=cuda)
        la = crit(plain(x), t)
        opt_a.zero_grad(); la.backward(); opt_a.step()
        lb = crit(wrapped(x), t)
        opt_b.zero_grad(); lb.backward(); opt_b.step()
        assert abs(float(la) - float(lb)) < 1e-4 * max(1.0, abs(float(la)))
    for (n, pa), pb in zip(plain.named_parameters(), wrapped.model.parameters()):
        assert _rel(pb, pa, 1e-2) < 1e-3, n


def test_bottleneck_resnet_against_float64(cuda):
    """A residual network under a tight schedule (recomputation, 1-bit masks, in-place ops,
    kernel-variant choice).  fp32 training of a deep randomly initialised network is
    ill-conditioned, so both the schedule and stock fp32 autograd are measured against
    float64 autograd: the schedule may not be further from it than stock fp32 is, within a
    factor that covers the run-to-run spread of such errors."""
    from monet_amd.models.resnet import Bottleneck, ResNet
    from monet_amd.schedule import Schedule
    from monet_amd.solver import Model
    torch.manual_seed(0)
    bs, shape = 16, (3, 64, 64)
    model = ResNet(Bottleneck, [2, 1, 1, 1], num_classes=10).to(cuda).train()
    graph, si, free = _solve(model, shape, bs, "inplace_conv_multiway_newnode", 1.0, cuda)
    total = sum(n.mem for i, n in si.nodes.items() if i < si.loss) + si.nodes[si.loss].fixed_mem
    sol = None
    for frac in (0.75, 0.9):
        print("solving at %.2f of the unconstrained footprint" % frac, flush=True)
        try:
            sol = Model(si, frac * total / 2**30, time_limit=40, mip_rel_gap=0.05,
                        recompute_window=12).solve()
            break
        except ValueError:
            continue
    assert sol is not None
    assert sol.r[1:].sum() > 0 or sol.ip.sum() > 0
    x = torch.randn((bs,) + shape, device=cuda)
    target = torch.randint(0, 10, (bs,), device=cuda)
    crit = nn.CrossEntropyLoss()

    def stock(m, xin):
        m.zero_grad()
        crit(m(xin), target).backward()
        return {n: p.grad.detach().double() for n, p in m.named_parameters()}

    g64 = stock(copy.deepcopy(model).double(), x.double())
    g32 = stock(copy.deepcopy(model), x)

    m = copy.deepcopy(model)
    sched = Schedule(graph, si)
    sched.init_schedule(sol, si.mode)
    y = sched.forward(x, *list(m.state_dict(keep_vars=True).values())).requires_grad_(True)
    crit(y, target).backward()
    sched.backward(y.grad)
    worst_ours = worst_stock = 0.0
    for n, p in m.named_parameters():
        scale = g64[n].abs().max().clamp_min(1e-12)
        worst_ours = max(worst_ours, float((p.grad.double() - g64[n]).abs().max() / scale))
        worst_stock = max(worst_stock, float((g32[n] - g64[n]).abs().max() / scale))
    print("largest relative error against float64: schedule %.3e, stock fp32 %.3e" % (
        worst_ours, worst_stock), flush=True)
    assert worst_ours <= 4 * worst_stock + 1e-5


def test_reserve_pool_leaves_one_cached_block(cuda):
    """`reserve_pool` (the reference's README.md:60-65 advice as a function): afterwards the
    allocator holds at least the requested bytes in its free list and nothing is allocated."""
    from monet_amd.monet_wrapper import reserve_pool
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    before = torch.cuda.memory_allocated()
    reserve_pool(256 << 20, cuda)
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.memory_reserved() - before >= 256 << 20
    torch.cuda.empty_cache()
