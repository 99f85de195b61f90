"""GPU tests of the glue operators (channel concatenation, the addmm form of the fully
connected layer, transpose) and of executor behaviour on graph shapes a ResNet does not
have: one gradient tensor shared by two pending gradients, an operand used twice, a grouped
convolution whose backward is split in two steps.  Reference: monet/lm_ops/cat.py:5-29,
linear.py:25-62, elementary.py:75-79, funcs.py:23-59, conv.py:70-90."""
import copy

import pytest
import torch
import torch.nn as nn

import monet_amd.lm_ops as lm_ops

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


# ---------------------------------------------------------------- operators on their own
@pytest.mark.parametrize("dim", [1, 0, 3])
def test_cat_forward_and_backward(cuda, dim):
    torch.manual_seed(0)
    shapes = [[2, 3, 5, 4], [2, 3, 5, 4], [2, 3, 5, 4]]
    for k, s in enumerate(shapes):
        s[dim] += k                                   # chunks of different length along `dim`
    parts = [torch.randn(s, device=cuda) for s in shapes]
    op = lm_ops.cat.Cat()
    y = op.forward(*parts, dim)
    leaves = [p.clone().requires_grad_(True) for p in parts]
    ref = torch.cat(leaves, dim=dim)
    assert torch.equal(y, ref.detach())
    g = torch.randn_like(y)
    ref.backward(g)
    grads = op.backward(g, [])
    assert len(grads) == len(parts)
    for got, leaf in zip(grads, leaves):
        assert got.is_contiguous() and torch.equal(got, leaf.grad)
    # one tensor: the identity both ways
    single = lm_ops.cat.Cat()
    assert single.forward(parts[0], dim) is parts[0]
    assert single.backward(g, []) is g


def test_addmm_backward_in_both_steps_and_at_once(cuda):
    torch.manual_seed(1)
    inp = torch.randn(7, 12, device=cuda, requires_grad=True)
    w = torch.randn(5, 12, device=cuda, requires_grad=True)
    b = torch.randn(5, device=cuda, requires_grad=True)
    op = lm_ops.linear.LowMemAddMM()
    y = op.forward(b, inp, w, 1, 1)                   # the operator transposes the weight itself
    ref = torch.addmm(b, inp, w.t())
    torch.testing.assert_close(y, ref.detach())
    g = torch.randn_like(y)
    ref.backward(g)
    op.algorithm = 0                                  # parameter gradients, input present
    db, di, dw = op.backward(g, [inp.detach(), w.detach()], nodel=True)
    assert di is None
    torch.testing.assert_close(dw, w.grad)
    torch.testing.assert_close(db, b.grad)
    op.algorithm = 10                                 # input gradient, input already dropped
    stored = [None, w.detach()]
    db, di, dw = op.backward(g, stored)
    assert db is None and dw is None and stored == []   # consumed
    torch.testing.assert_close(di, inp.grad)
    op.algorithm = 20                                 # both
    db, di, dw = op.backward(g, [inp.detach(), w.detach()])
    torch.testing.assert_close(di, inp.grad)
    torch.testing.assert_close(dw, w.grad)
    torch.testing.assert_close(db, b.grad)
    with pytest.raises(AssertionError):
        lm_ops.linear.LowMemAddMM().forward(b, inp, w, 2, 1)   # only beta = alpha = 1


def test_transpose_operator(cuda):
    x = torch.randn(6, 9, device=cuda)
    op = lm_ops.elementary.T()
    y = op.forward(x)
    assert torch.equal(y, x.t())
    g = torch.randn_like(y)
    assert torch.equal(op.backward(g, []), g.t())


# ---------------------------------------------------------------- through the executor
class SharedGradient(nn.Module):
    """x + relu(conv(x)): the add hands ONE gradient tensor to both operands, the ReLU
    backward overwrites its gradient in place while the other operand's is still pending."""

    def __init__(self):
        super().__init__()
        self.stem = nn.Conv2d(3, 8, 3, padding=1)
        self.conv = nn.Conv2d(8, 8, 3, padding=1)
        self.fc = nn.Linear(8, 4)

    def forward(self, x):
        x = self.stem(x)
        y = x + torch.relu(self.conv(x))
        return self.fc(torch.flatten(torch.nn.functional.adaptive_avg_pool2d(y, 1), 1))


class UsedTwice(nn.Module):
    """y + y and y + 0.5 * ... of one tensor: both gradient contributions must arrive."""

    def __init__(self):
        super().__init__()
        self.conv = nn.Conv2d(3, 8, 3, padding=1)
        self.bn = nn.BatchNorm2d(8)
        self.fc = nn.Linear(8, 4)

    def forward(self, x):
        y = self.bn(self.conv(x))
        z = torch.relu(y + y)
        z = torch.add(z, z, alpha=0.5)
        return self.fc(torch.flatten(torch.nn.functional.adaptive_avg_pool2d(z, 1), 1))


class Grouped(nn.Module):
    """A grouped (not depthwise) convolution and a depthwise one, each with a bias."""

    def __init__(self):
        super().__init__()
        self.stem = nn.Conv2d(3, 8, 3, padding=1)
        self.grouped = nn.Conv2d(8, 16, 3, padding=1, groups=2)
        self.depthwise = nn.Conv2d(16, 16, 3, padding=1, groups=16)
        self.fc = nn.Linear(16, 4)

    def forward(self, x):
        x = torch.relu(self.stem(x))
        x = torch.relu(self.grouped(x))
        x = torch.relu(self.depthwise(x))
        return self.fc(torch.flatten(torch.nn.functional.adaptive_avg_pool2d(x, 1), 1))


class CatAddmm(nn.Module):
    """A skip connection by concatenation (with the replicating "upsample" of the
    reference's UNet) and a fully connected layer written as addmm(bias, x, weight.t())."""

    def __init__(self):
        super().__init__()
        self.a = nn.Conv2d(3, 6, 3, padding=1)
        self.pool = nn.MaxPool2d(2)
        self.b = nn.Conv2d(6, 10, 3, padding=1)
        self.up = nn.AdaptiveAvgPool2d((16, 16))
        self.c = nn.Conv2d(16, 8, 3, padding=1)
        self.weight = nn.Parameter(torch.randn(4, 8) * 0.3)
        self.bias = nn.Parameter(torch.randn(4) * 0.1)

    def forward(self, x):
        x1 = torch.relu(self.a(x))
        x2 = torch.relu(self.b(self.pool(x1)))
        y = torch.relu(self.c(torch.cat([x1, self.up(x2)], dim=1)))
        feat = torch.flatten(torch.nn.functional.adaptive_avg_pool2d(y, 1), 1)
        return torch.addmm(self.bias, feat, self.weight.t())


@pytest.mark.parametrize("net", [SharedGradient, UsedTwice, Grouped, CatAddmm])
@pytest.mark.parametrize("mode", ["inplace_conv_multiway_newnode",
                                  "fused_inplace_conv_multiway_newnode"])
def test_schedule_on_other_graph_shapes(cuda, net, mode):
    from monet_amd.graph import Graph, fusion_level
    from monet_amd.schedule import Schedule
    from monet_amd.solver import Model
    from monet_amd.solver_info import SolverInfo
    torch.manual_seed(0)
    bs, shape = 8, (3, 16, 16)
    model = net().to(cuda).train()
    graph = Graph.create(copy.deepcopy(model).cpu(), shape, fuse_bn_relu=fusion_level(mode))
    ops = {n.op for n in graph.nodes if hasattr(n, "op")}
    if net is CatAddmm:
        assert "aten::cat" in ops and "aten::addmm" in ops
    x = torch.randn((bs,) + shape, device=cuda)
    si = SolverInfo(bs, "test", mode)
    si.extract(graph, x, *list(model.state_dict(keep_vars=True).values()))
    total = sum(n.mem for i, n in si.nodes.items() if i < si.loss) + si.nodes[si.loss].fixed_mem
    solutions = [Model(si, 1.0, time_limit=60, mip_rel_gap=0.0).solve()]
    for frac in (0.8, 0.6):
        try:
            solutions.append(Model(si, frac * total / 2**30, time_limit=60, mip_rel_gap=0.0).solve())
        except ValueError:
            break
    gout = torch.randn(bs, 4, device=cuda)
    ref = copy.deepcopy(model)
    y_ref = ref(x)
    y_ref.backward(gout)
    g_ref = {n: p.grad for n, p in ref.named_parameters()}
    floor = 1e-2 * max(float(g.abs().max()) for g in g_ref.values())
    for sol in solutions:
        m = copy.deepcopy(model)
        sched = Schedule(graph, si)
        sched.init_schedule(sol, si.mode)
        for step in range(2):
            for p in m.parameters():
                p.grad = None
            y = sched.forward(x, *list(m.state_dict(keep_vars=True).values()))
            assert _rel(y, y_ref.detach()) < 1e-5
            keep = gout.clone()
            sched.backward(gout)
            assert torch.equal(gout, keep), "the executor wrote into the caller's gradient"
            for n, p in m.named_parameters():
                assert p.grad is not None, n
                err = float((p.grad - g_ref[n]).abs().max() / g_ref[n].abs().max().clamp_min(floor))
                assert err < 1e-4, (net.__name__, mode, n, err)
