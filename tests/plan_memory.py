"""Byte-level replay of a compiled schedule: which tensors are alive after every
instruction, without running any kernel.  Used to check that what the executor
would hold agrees with what the ILP budgeted."""
import numpy as np

from monet_amd import schedule as S
from monet_amd.graph import ComputeNode


def _bytes(shape, bs):
    n = 4
    for d in shape:
        n *= bs if d == -1 else d
    return n


def replay(sched, bs):
    """Peak bytes over the step and per timestep: parameters + inputs + activations kept or
    in flight + intermediates + gradients (workspace excluded)."""
    nodes = sched._nodes
    size = [_bytes(n.shape, bs) for n in nodes]
    fixed = sum(size[k] for k in sched._leaves)
    regs, ints, bw = {}, {}, {}
    int_bytes = {}
    for j, node in sched.si.nodes.items():
        if j < sched.si.loss and node.has_intermediates:
            k = sched.si.solver_to_graph[j]
            int_bytes[k] = {p: sched.si.nodes[iid].mem for p, iid in node.intermediates}
    peaks = []
    for k in sched._outputs:
        bw[k] = size[k]
    for t, plan in enumerate(sched._plan):
        peak = 0
        for ins in plan:
            cur = fixed + sum(regs.values()) + sum(ints.values()) + sum(bw.values())
            if ins[0] == S._FWD:
                _, op, k, args, with_int, *_rest, inplace_src = ins
                for is_t, v in args:
                    if is_t and isinstance(nodes[v[0]], ComputeNode):
                        assert v[0] in regs, (t, k, v[0])
                extra = 0 if inplace_src >= 0 else size[k]
                if with_int:
                    impl = sched._implementation(sched.solution, t, sched.si.graph_to_solver[k])
                    ints[k] = int_bytes[k][impl]
                    extra += ints[k]
                peak = max(peak, cur + extra)
                if inplace_src >= 0:
                    regs.pop(inplace_src, None)
                regs[k] = size[k]
            elif ins[0] == S._FREE:
                for kk in ins[1:]:
                    regs.pop(kk, None)
            elif ins[0] == S._FREE_INT:
                ints.pop(ins[1], None)
            else:
                _, op, k, spec, drop, last, deps, *_rest2 = ins
                held = 0
                for kind, i, optional in spec:
                    if kind == 1:
                        held += ints.pop(i)
                    elif isinstance(nodes[i], ComputeNode) and not optional:
                        assert i in regs, (t, k, i)
                for kk in drop:
                    if kk in regs and any(kind == 0 and i == kk for kind, i, _ in spec):
                        held += regs[kk]
                    regs.pop(kk, None)
                assert k in bw, (t, k)
                outs = sum(size[i] for i, r in deps if r)
                cur = fixed + sum(regs.values()) + sum(ints.values()) + sum(bw.values()) + held
                peak = max(peak, cur + outs)
                if last:
                    bw.pop(k)
                for i, r in deps:
                    if r:
                        bw[i] = size[i]
        peaks.append(peak)
    return max(peaks), peaks
