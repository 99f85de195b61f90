"""Exact optimum of the checkpointing schedule problem on a tiny solver graph, by enumeration.

Test infrastructure: the reference's formulation (monet/cvxpy_solver.py:54-334) evaluated
directly on candidate schedules, with none of the reductions `monet_amd/solver.py` applies
to keep its ILP small (per-timestep frontiers, running sums carried by real variables, products
S*M only where a backward node has several implementations).  Modes without in-place operators
and without convolution variants (P == R, no IP, no RF).

The constraints of a timestep t only involve S[t], R[t], S[t+1] and M[t], and the objective is
a sum over timesteps, so the optimum is a shortest path over the stored sets:
    best[t][S_t] = min over feasible (R_t, S_t+1, p)  cost(t, R_t, p) + best[t+1][S_t+1]
with every (R_t, S_t+1, p) enumerated (2^V x 2^V x paths candidates per state).
"""
import numpy as np

from monet_amd.solver import Model
from monet_amd.solver_info import IntNode


def optimum(si, budget_gb):
    """(minimal objective in the ILP's cost units, or None if no schedule fits the budget)."""
    ref = Model(si, budget=budget_gb)       # unit conversions only: ram (KB), cpu (scaled ints)
    V = si.loss + 1
    T = len(si.nodes) - si.loss
    assert not si.do_inplace and not si.select_conv_algo and V <= 7
    budget = budget_gb * 1024 * 1024        # KB, as cvxpy_solver.py:56
    ram = [float(ref.ram[i]) for i in range(V)]
    full = 1 << V
    bit = lambda mask, i: (mask >> i) & 1
    int_nodes = [isinstance(si.nodes[i], IntNode) for i in range(V)]
    ff_edges = [(u, v) for (u, v, p) in si.edge_list if u < V and v < V]
    fb_edges = {}
    for (u, v, p) in si.edge_list:
        if u < V <= v:
            fb_edges.setdefault((v + 1 - V, p), []).append(u)
    parents = [(i, intid) for i in range(V) for (_, intid) in si.nodes[i].intermediates]

    ramsum = np.zeros(full)                 # bytes of a set of forward tensors
    for mask in range(1, full):
        low = mask & -mask
        ramsum[mask] = ramsum[mask ^ low] + ram[low.bit_length() - 1]
    below = [(1 << j) - 1 for j in range(V + 1)]          # bits < j
    local_mask = [sum(1 << i for i in si.nodes[j].local_tensors if i < V) for j in range(V)]

    def computable(S, R):
        """Dependencies among forward nodes (:162-164) and intermediates only with their parent
        (:170-176)."""
        for (u, v) in ff_edges:
            if bit(R, v) and not (bit(R, u) or bit(S, u)):
                return False
        for (i, intid) in parents:
            if bit(R, intid) and not bit(R, i):
                return False
        return True

    def step(t, S, R, S1, p):
        """Cost of timestep t with stored set S, computed set R (checked by `computable`), next
        stored set S1 (a subset of S | R, :155) and backward implementation p, or None if a
        constraint of cvxpy_solver.py:165-268 is violated."""
        b = V + t - 1
        node = si.nodes[b]
        for u in fb_edges.get((t, p), []):      # (:165-167)
            if not (bit(R, u) or bit(S1, u)):
                return None
        # memory (:189-268)
        gradm = (ref.local_memory(b) if t != 0 else 0) + ref.fixed_ram(b - 1)
        args_mask = sum(1 << a for a in set(node.args[p]) if a < V)
        for j in range(V):
            # read by implementation p, below j, and not stored for later (lm1 + lm2)
            keep = ramsum[args_mask & below[j] & ~S1]
            sm1 = ramsum[S & ~below[j]] + ramsum[S1 & below[j]]
            if gradm + sm1 + keep > budget:
                return None
            if bit(R, j):
                ws = ref.cmem(j)[0] if t == 0 else ref.cmem(j, recompute=True)[0]
                sm2 = ramsum[S & ~below[j + 1] & ~local_mask[j]] + ramsum[S1 & below[j] & ~local_mask[j]]
                if gradm + ws + ram[j] + ref.local_memory(j) + sm2 + keep > budget:
                    return None
        if t > 0:
            # lm3: everything implementation p reads; lm4: what stays stored and p does not read
            deps_mask = sum(1 << i for i in set(node.dep_list_fwd[p]) if i < V)
            m3 = ref.cmem(b)[p] + ref.local_memory(b) + ref.fixed_ram(b) + float(ref.ram[b])
            m3 += ramsum[args_mask] + ramsum[S1 & ~deps_mask]
            if m3 > budget:
                return None
        # objective (:289-296)
        cost = 0.0
        for i in range(V):
            if bit(R, i):
                cost += ref.cpu[i][0] if t == 0 else ref.cpu_recompute[i][0]
        if p < len(ref.cpu[b]):
            cost += ref.cpu[b][p]
        return cost

    inf = float("inf")
    best = np.full((T + 1, full), inf)
    best[T, :] = 0.0
    forward_all = sum(1 << i for i in range(V) if not int_nodes[i])
    for t in range(T - 1, -1, -1):
        paths = 1 if t == 0 else len(si.nodes[V + t - 1].args)
        states = [0] if t == 0 else range(full)     # S[0] = 0 (:122)
        for S in states:
            for R in range(full):
                if t == 0 and (R & forward_all) != forward_all:   # the forward pass computes everything (:125-127)
                    continue
                if not computable(S, R):
                    continue
                cand = S | R
                S1 = cand
                while True:                                       # all subsets of S | R
                    if best[t + 1, S1] < inf:
                        for p in range(paths):
                            c = step(t, S, R, S1, p)
                            if c is not None and c + best[t + 1, S1] < best[t, S]:
                                best[t, S] = c + best[t + 1, S1]
                    if S1 == 0:
                        break
                    S1 = (S1 - 1) & cand
    return None if best[0, 0] == inf else float(best[0, 0])
