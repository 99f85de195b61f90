"""Executor of a solved schedule (reference: monet/schedule.py:14-311).

A solution says, for every timestep t (0 = the forward pass, t > 0 = backward
solver node loss+t), which forward operators to (re)compute, with which
implementation, kernel variant and in-place flag, which outputs to keep for
the next timestep, and which backward implementation to run.  The reference
interprets those tables on every training step, walking all graph nodes once
per timestep.  Here `init_schedule` replays that walk ONCE, symbolically, and
compiles it into a flat instruction list; a training step then only executes
the instructions, so the host cost per step is proportional to the operators
that actually run, and operator objects exist only for those.

Semantics kept from the reference:
  * a timestep starts from the tensors the previous one stored; an operator
    flagged for recomputation runs only if its output is absent or it has to
    produce an intermediate (schedule.py:156-158);
  * tensors are dropped as soon as no later operator of the step reads them,
    except those the step's backward needs (schedule.py:28-37, 188-191);
  * convolution and fully connected layers run their backward in two
    timesteps, parameter gradients first, then the input gradient without the
    stored input (schedule.py:220-246);
  * the state an operator's forward leaves in `params` travels to whichever
    instance runs its recomputation or its backward; operators that replay an
    autograd node run their backward on the forward's own instance
    (schedule.py:159-173, 247-251).
Beyond the reference: an intermediate the solution does not keep is freed at
the end of the timestep that produced it, and parameter gradients are handed
to `.grad` directly instead of through the autograd engine.
"""
import copy
import pickle
from collections import OrderedDict, defaultdict, namedtuple

import torch

from . import lm_ops
from .lm_ops import bn as bn_ops
from .graph import ComputeNode, Graph, is_batch_norm, two_step_backward
from .solver_info import BwdNode, IntNode, SolverInfo

ScheduleType = namedtuple('ScheduleType', 'recompute store_output store_intermediate')

# instruction opcodes
_FWD, _FREE, _FREE_INT, _BWD = 0, 1, 2, 3


def _storage_list(op):
    s = op.backward_storage
    if s is None:
        return []
    return s if isinstance(s, list) else [s]


class Schedule(Graph):
    def __init__(self, graph: Graph, info: SolverInfo):
        super().__init__()
        self.si = info
        self._nodes = graph.nodes
        self._outputs = graph._outputs
        self.solution = None
        self.lennodes = len(self._nodes)
        self.computeInstance = [k for k, n in enumerate(self._nodes)
                                if isinstance(n, ComputeNode) and n.op != "aten::t"]
        self._leaves = [k for k, n in enumerate(self._nodes) if not isinstance(n, ComputeNode)]

        # tensors whose last reader within a forward sweep is solver node j
        si = self.si
        self.deltensors = defaultdict(list)
        for j in si.nodes:
            if j >= si.loss:
                continue
            nxt = j + 1
            while isinstance(si.nodes[nxt], IntNode):
                nxt += 1
            for i in si.nodes[j].local_tensors:
                if i not in si.nodes[nxt].local_tensors and si.solver_to_graph[i] >= 0:
                    self.deltensors[j].append(si.solver_to_graph[i])

        self._plan = []        # per timestep: list of instructions
        self._ops0 = []        # batch-norm operators of the forward pass (state reset per step)
        self._regs = [None] * self.lennodes
        self._ints = [None] * self.lennodes
        self._state = [None] * self.lennodes
        self._bw = [None] * self.lennodes
        # storage address -> number of pending gradients (entries of _bw) that live in it
        self._shared = {}
        self._args = []

    # ------------------------------------------------------------ compile
    def _implementation(self, solution, t, j):
        """Index of the forward implementation of solver node j at timestep t: the one whose
        intermediate the solution computes there, else the first."""
        p = 0
        node = self.si.nodes[j]
        if self.si.compute_newnode and node.has_intermediates:
            for p_option, intid in node.intermediates:
                if solution.r[t][intid]:
                    assert solution.r[t][j], "an intermediate is computed without its operator"
                    p = p_option
        return p

    def _make_fwd_op(self, solution, t, k, j):
        si, n = self.si, self._nodes[k]
        op = lm_ops.list_ops(si.mode, n.op)[self._implementation(solution, t, j)]()
        if si.select_conv_algo and j in si.conv_list:
            for c in range(min(op.n_fwd_algos(), solution.rf.shape[2])):
                if solution.rf[t, si.conv_list[j], c]:
                    op.algorithm = c
                    break
        if n.is_depthwise:
            op.is_depthwise = True
        if si.do_inplace and j in si.inplace_list and solution.ip[t][j]:
            op.inplace = True
        return op

    def _make_bwd_op(self, solution, t):
        si = self.si
        bwd_t = si.loss + t
        b = si.nodes[bwd_t]
        n = self._nodes[si.solver_to_graph[si.bwd_to_fwd[bwd_t]]]
        p = 0
        for o in range(len(solution.m[t])):
            if solution.m[t][o] == 1:
                p = o
        op = lm_ops.list_ops(si.mode, n.op)[p]()
        if n.is_depthwise:
            op.is_depthwise = True
        if two_step_backward(n):
            algo = 0
            algo_type = 0 if b.bwd_op == "param_grad" else 1
            if si.select_conv_algo and bwd_t in si.conv_list:
                algo = -1
                for c in range(solution.rf.shape[2]):
                    if solution.rf[t, si.conv_list[bwd_t], c]:
                        algo = c
                        break
                if algo == -1:
                    raise RuntimeError("Algorithm not decided", t, bwd_t)
            op.algorithm = algo_type * 10 + algo
        return op

    def init_schedule(self, solution, mode=None):
        """Compile `solution` into per-timestep instruction lists."""
        self.solution = solution
        si = self.si
        T = len(si.nodes) - si.loss
        self._plan = [[] for _ in range(T)]
        self._fwd_schedule = [[] for _ in range(T)]
        self._ops0 = []
        g2s, s2g = si.graph_to_solver, si.solver_to_graph

        live = set()       # computed tensors present in the register file
        have_int = set()   # intermediates present
        for t in range(T):
            plan = self._plan[t]
            # ---- what the backward operator of this timestep needs
            bwd = None
            keep = []
            if t > 0:
                bwd_t = si.loss + t
                assert isinstance(si.nodes[bwd_t], BwdNode)
                b = si.nodes[bwd_t]
                k_b = s2g[si.bwd_to_fwd[bwd_t]]
                n_b = self._nodes[k_b]
                bop = self._make_bwd_op(solution, t)
                second = two_step_backward(n_b) and b.bwd_op == "ip_grad"
                spec = []  # (kind, index, may_be_absent): kind 0 register, 1 intermediate
                for storage in _storage_list(bop):
                    if isinstance(storage, lm_ops.InputStorage):
                        ids = [n_b.args[i].index for i in storage.ids]
                        for pos, i in enumerate(ids):
                            # the input-gradient half of a split backward runs without the input
                            spec.append((0, i, second and pos != len(ids) - 1))
                    elif isinstance(storage, lm_ops.OutputStorage):
                        spec.append((0, k_b, False))
                    elif isinstance(storage, lm_ops.IntermediateStorage):
                        spec.append((1, k_b, False))
                required = [i for kind, i, _ in spec if kind == 0]
                keep = [required[1]] if second else required
                bwd = (bop, k_b, n_b, spec, b)

            # ---- forward sweep of this timestep
            stored = set()
            for k in self.computeInstance:
                n = self._nodes[k]
                j = g2s[k]
                recompute = bool(solution.r[t][j])
                store_output = bool(solution.s[t + 1][j]) if t < T - 1 else False
                cls = lm_ops.list_ops(si.mode, n.op)[self._implementation(solution, t, j)]
                with_int = any(isinstance(s, lm_ops.IntermediateStorage) for s in _storage_list(cls))
                self._fwd_schedule[t].append(ScheduleType(recompute, store_output, with_int))
                if recompute and (k not in live or with_int):
                    op = self._make_fwd_op(solution, t, k, j)
                    for a in n.args:
                        if isinstance(a, ComputeNode.D) and isinstance(self._nodes[a.index], ComputeNode):
                            assert a.index in live, \
                                "timestep %d: %s (node %d) needs node %d, which is neither stored " \
                                "nor recomputed" % (t, n.op, k, a.index)
                    args = tuple((False, a.value) if isinstance(a, ComputeNode.V)
                                 else (True, (a.index, a.requires_grad)) for a in n.args)
                    is_bn = is_batch_norm(n.op)
                    if is_bn and t == 0:
                        self._ops0.append(op)
                    inplace_src = -1
                    if getattr(op, 'inplace', False):
                        inplace_src = n.args[0].index  # the tensor the kernel overwrites
                    plan.append((_FWD, op, k, args, with_int, is_bn and t > 0,
                                 hasattr(op, 'params'), isinstance(op, lm_ops.NativeOP), inplace_src))
                    live.add(k)
                    if with_int:
                        have_int.add(k)
                    if inplace_src >= 0:
                        live.discard(inplace_src)
                if store_output:
                    assert k in live, 'Storing a None tensor for graph node %d, solver node %d, ' \
                        'op %s at timestep %d' % (k, j, n.op, t)
                    stored.add(k)
                for kk in self.deltensors[j]:
                    if kk not in keep and kk in live:
                        live.discard(kk)
                        if kk not in stored:  # a stored tensor stays for the next timestep
                            plan.append((_FREE, kk))

            # ---- backward operator
            consumed_int = -1
            if bwd is not None:
                bop, k_b, n_b, spec, b = bwd
                for kind, i, optional in spec:
                    if kind == 1:
                        assert i in have_int, "Intermediate output not computed for node %d" % i
                        consumed_int = i
                    elif isinstance(self._nodes[i], ComputeNode) and not optional:
                        assert i in live, "Tensor dependency %d not computed or stored for node " \
                            "%d %s t=%d" % (i, k_b, n_b.op, t)
                drop = tuple(sorted(live - stored))
                last = not (two_step_backward(n_b) and b.bwd_op == "param_grad")
                # an operator that can add its first input's gradient to one that is already
                # there (convolution backward-data) is handed that tensor instead of a later add
                deps_b = tuple(n_b.dependencies)
                acc = bool(getattr(bop, 'accumulates_input_grad', False)) and len(deps_b) > 0 and \
                    bool(deps_b[0][1])
                plan.append((_BWD, bop, k_b, tuple(spec), drop, last, deps_b,
                             hasattr(bop, 'params'), isinstance(bop, lm_ops.NativeOP), acc))
                have_int.discard(consumed_int)
            else:
                # the forward pass: the model output stays until forward() has returned it
                out = self.lennodes - 1
                plan.append((_FREE,) + tuple(sorted(live - stored - {out})))
                self._free_output = out not in stored
            live = set(stored)

            # ---- intermediates the solution does not carry into the next timestep
            for k in sorted(have_int):
                j = g2s[k]
                carried = any(t < T - 1 and solution.s[t + 1][iid]
                              for _, iid in si.nodes[j].intermediates)
                if not carried:
                    plan.append((_FREE_INT, k))
                    have_int.discard(k)

    # ------------------------------------------------------------ execute
    def _run(self, plan):
        regs, ints, state, bw = self._regs, self._ints, self._state, self._bw
        for ins in plan:
            code = ins[0]
            if code == _FWD:
                _, op, k, argspec, with_int, restore, has_params, native, inplace_src = ins
                if restore:
                    op.params = state[k]
                args = [v if not is_t else regs[v[0]].requires_grad_(v[1]) for is_t, v in argspec]
                if with_int:
                    regs[k], ints[k] = op.forward(*args)
                    assert ints[k] is not None
                else:
                    regs[k] = op.forward(*args)
                del args
                if has_params:
                    state[k] = op.params
                if native:
                    state[k] = op
                if inplace_src >= 0:
                    regs[inplace_src] = None
            elif code == _FREE:
                for kk in ins[1:]:
                    regs[kk] = None
            elif code == _FREE_INT:
                ints[ins[1]] = None
            else:
                _, op, k, spec, drop, last, deps, has_params, native, acc = ins
                stored = []
                for kind, i, _ in spec:
                    if kind == 0:
                        stored.append(regs[i])
                    else:
                        stored.append(ints[i])
                        ints[i] = None
                for kk in drop:
                    regs[kk] = None
                if has_params:
                    op.params = state[k]
                if native:
                    op = state[k]
                    assert op is not None
                grad = bw[k]
                assert grad is not None, "Backward input not computed for graph node %d (%s)" % (
                    k, self._nodes[k].op)
                # Pending gradients may share storage (an add hands ONE tensor to both operands,
                # a view operator hands on a view).  Whoever writes into such storage - an
                # operator that overwrites its gradient, an accumulation - gets a private copy
                # while another pending gradient still lives there.
                shared = self._shared
                if last:
                    bw[k] = None
                    key = grad.untyped_storage().data_ptr()
                    others = shared.get(key, 1) - 1
                    if others > 0:
                        shared[key] = others
                        if op.overwrites_grad:
                            grad = grad.clone()
                    else:
                        shared.pop(key, None)
                target = None
                if acc:
                    ti = deps[0][0]
                    target = bw[ti]
                    if target is not None:
                        key = target.untyped_storage().data_ptr()
                        if shared.get(key, 1) > 1:
                            shared[key] -= 1
                            target = bw[ti] = target.clone()
                            shared[target.untyped_storage().data_ptr()] = 1
                if target is not None:
                    outs = op.backward(grad, stored, accumulate_into=target)
                else:
                    outs = op.backward(grad, stored)
                del grad, stored
                if not isinstance(outs, (list, tuple)):
                    outs = (outs,)
                assert len(outs) == len(deps), \
                    "Require the same number of grad outputs as forward inputs %s: %d vs %d" % (
                        self._nodes[k].op, len(outs), len(deps))
                for pos, ((i, r), o) in enumerate(zip(deps, outs)):
                    if r and o is not None:
                        if bw[i] is None:
                            bw[i] = o
                            key = o.untyped_storage().data_ptr()
                            shared[key] = shared.get(key, 0) + 1
                        elif pos == 0 and o is target:
                            pass  # the operator has added it to the pending gradient itself
                        else:
                            key = bw[i].untyped_storage().data_ptr()
                            if shared.get(key, 1) > 1:   # someone else still reads this storage
                                shared[key] -= 1
                                bw[i] = bw[i] + o
                                shared[bw[i].untyped_storage().data_ptr()] = 1
                            else:
                                bw[i] += o
                del outs, target

    def forward(self, *args):
        """Forward pass; `args` = (input, *parameters and buffers) in graph-node order."""
        assert len(args) == len(self._leaves), \
            "expected %d inputs and parameters, got %d" % (len(self._leaves), len(args))
        self._args = args
        for op in self._ops0:
            op.params = None  # fresh batch statistics every step
        regs = self._regs
        for k in self._leaves:
            regs[k] = args[k]
        self._run(self._plan[0])
        out = regs[self.lennodes - 1]
        assert out is not None
        if self._free_output:
            regs[self.lennodes - 1] = None
        return out

    def backward(self, delta_x):
        bw = self._bw
        self._shared.clear()
        for k in self._outputs:
            bw[k] = delta_x
            # the caller's tensor: never written in place (counted as if someone else held it)
            self._shared[delta_x.untyped_storage().data_ptr()] = 2
        for plan in self._plan[1:]:
            self._run(plan)
        # hand the accumulated gradients to the leaves
        for k in self._leaves:
            g, a = bw[k], self._args[k]
            bw[k] = None
            if g is None or not a.requires_grad:
                continue
            key = g.untyped_storage().data_ptr()
            if self._shared.get(key, 1) > 1:   # never hand one storage to two leaves
                self._shared[key] -= 1
                g = g.clone()
            if a.is_leaf:
                if a.grad is None:
                    a.grad = g if g.shape == a.shape else g.reshape(a.shape)
                else:
                    a.grad += g
            else:
                a.backward(g)
        for k in range(self.lennodes):
            self._regs[k] = self._ints[k] = self._state[k] = self._bw[k] = None
        self._args = []
        self._shared.clear()
        for op in self._ops0:
            op.params = None
        # once per step, without waiting for the device: did a BatchNorm kernel give up a wait
        # (its results are NaN then)?  Raises one step late.
        if delta_x.is_cuda:
            bn_ops.poll_waits(delta_x.device)


def disable_dropout(model):
    for m in model.modules():
        if isinstance(m, torch.nn.Dropout):
            m.p = 0.0


def load_solution(filename):
    from .solver import Solution  # noqa: F401  (the pickle refers to it)
    with open(filename, 'rb') as f:
        si, solution = pickle.load(f)
    return si, solution


# Traced graphs by (architecture, parameter shapes, plain attributes of every module, input
# shape, fusion level, training flags): tracing runs the model once on the CPU (tens of seconds
# for a UNet at full resolution), and a graph holds structure only, so wrappers of the same
# architecture share it.  The assumption is that the traced graph depends on nothing else; a
# model whose forward() branches on state the key does not see (a global, a tensor's value) must
# not be traced through this cache (`cache=False`).  The eight most recently used graphs are kept.
_graph_cache = OrderedDict()
_GRAPH_CACHE_SIZE = 8


def _plain_attributes(model):
    """(module path, attribute, repr) of every public attribute of a module that is a number, a
    string, None or a flat tuple / list of those: what repr(model) may leave out and forward()
    may read (UNet's target height and width, a flag)."""
    plain = (bool, int, float, str, type(None))
    out = []
    for path, mod in model.named_modules():
        for k, v in sorted(vars(mod).items()):
            if k.startswith("_") or k == "training":
                continue
            if isinstance(v, plain) or (isinstance(v, (tuple, list)) and
                                        all(isinstance(e, plain) for e in v)):
                out.append((path, k, repr(v)))
    return tuple(out)


def _traced_graph(model, input_shape, fuse_level, cache=True):
    def trace():
        m = copy.deepcopy(model)
        m.cpu()
        return Graph.create(m, input_shape, fuse_bn_relu=fuse_level)
    if not cache:
        return trace()
    key = (type(model).__module__, type(model).__qualname__, repr(model),
           tuple((k, tuple(v.shape)) for k, v in model.state_dict().items()),
           _plain_attributes(model), tuple(input_shape), int(fuse_level),
           tuple(bool(mod.training) for mod in model.modules()))
    if key in _graph_cache:
        _graph_cache.move_to_end(key)
    else:
        _graph_cache[key] = trace()
        while len(_graph_cache) > _GRAPH_CACHE_SIZE:
            _graph_cache.popitem(last=False)
    return _graph_cache[key]


def create_schedule(model, sol_file, input_shape=(3, 224, 224)):
    """Trace `model` (on the CPU), load (solver info, solution) from `sol_file` and
    return the compiled schedule (reference: monet/schedule.py:326-346)."""
    m = model
    if m._get_name() == 'MobileNetV2':
        m = torch.nn.Sequential(m.features, torch.nn.AdaptiveAvgPool2d((1, 1)),
                                torch.nn.Flatten(start_dim=1), m.classifier[0], m.classifier[1])
    solver_info, solution = load_solution(sol_file)
    graph = _traced_graph(m, input_shape, getattr(solver_info, "fuse_bn_relu", False))
    schedule = Schedule(graph, solver_info)
    schedule.init_schedule(solution, solver_info.mode)
    return schedule


def _timed_steps(step, warmup, iters):
    """Mean ms per call of `step` and the peak allocation (MB) over the timed calls."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        step()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters, torch.cuda.max_memory_allocated() / 2**20


def main(argv=None):
    """`python -m monet_amd.schedule MODEL BATCH_SIZE BUDGET MODE SOLVER --solution_file F
    (--check_runtime | --check_diff | --run_bs)` (reference: monet/schedule.py:348-517)."""
    import argparse

    from . import config
    from .models import build_model

    parser = argparse.ArgumentParser()
    parser.add_argument('model')
    parser.add_argument('bs', type=int)
    parser.add_argument('budget', type=float)
    parser.add_argument('mode')
    parser.add_argument('solver', nargs='?', default="HIGHS")
    parser.add_argument("--solution_file", type=str, required=True)
    parser.add_argument("--check_runtime", action="store_true",
                        help="time the schedule (and, with --original, stock autograd)")
    parser.add_argument("--original", action="store_true")
    parser.add_argument("--run_bs", action="store_true", help="one step, report peak memory")
    parser.add_argument("--check_diff", action="store_true",
                        help="compare output and gradients with stock autograd")
    parser.add_argument("--warmup", type=int, default=10)
    parser.add_argument("--iters", type=int, default=20)
    args = parser.parse_args(argv)

    config.budget = args.budget
    model, input_shape, model_name = build_model(args.model)
    if args.check_diff:
        disable_dropout(model)
    si, solution = load_solution(args.solution_file)
    graph = Graph.create(model, input_shape=input_shape,
                         fuse_bn_relu=getattr(si, "fuse_bn_relu", False))
    model.cuda()
    schedule = Schedule(graph, si)
    schedule.init_schedule(solution, si.mode)
    input_ = torch.randn((args.bs,) + tuple(input_shape)).cuda()
    state = lambda: list(model.state_dict(keep_vars=True).values())

    def monet_step():
        out = schedule.forward(input_, *state())
        schedule.backward(-torch.ones_like(out))
        for v in model.parameters():
            v.grad = None

    if args.check_runtime:
        ms, mb = _timed_steps(monet_step, args.warmup, args.iters)
        print("monet: %f ms avg, %8.2f MB" % (ms, mb))
        if args.original:
            def plain_step():
                model(input_).sum().backward()
                for v in model.parameters():
                    v.grad = None
            schedule = None
            torch.cuda.empty_cache()
            ms0, mb0 = _timed_steps(plain_step, args.warmup, args.iters)
            print("original: %f ms avg, %8.2f MB" % (ms0, mb0))
    elif args.check_diff:
        ref = copy.deepcopy(model)
        y0 = ref(input_)
        y0.sum().backward()
        y1 = schedule.forward(input_, *state())
        print('Forward mean absolute difference', float((y0 - y1).abs().mean()))
        schedule.backward(torch.ones_like(y1))
        worst = 0.0
        # parameters whose true gradient is zero (a bias in front of a BatchNorm) hold rounding
        # noise on both sides: measure against at least 1e-3 of the largest gradient
        floor = 1e-3 * max(float(q.grad.abs().max()) for q in ref.parameters())
        for (name, p), q in zip(model.named_parameters(), ref.parameters()):
            rel = float((p.grad - q.grad).abs().max() / q.grad.abs().max().clamp_min(floor))
            worst = max(worst, rel)
            print("%.3e %s %s" % (rel, name, tuple(p.shape)))
        print("largest relative gradient difference %.3e" % worst)
    elif args.run_bs:
        torch.cuda.reset_peak_memory_stats()
        from time import time
        t0 = time()
        monet_step()
        torch.cuda.synchronize()
        print("Ran batch %d with peak memory %8.2fM, %fs" % (
            args.bs, torch.cuda.max_memory_allocated() / 2**20, time() - t0))


if __name__ == '__main__':
    main()
