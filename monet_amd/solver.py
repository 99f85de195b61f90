"""The schedule ILP (reference: monet/cvxpy_solver.py:54-334, restated from the
clearer monet/gurobi_solver.py:84-271) on scipy's HiGHS MILP solver, because
neither cvxpy nor CBC / Gurobi are available where this runs.

Binary variables, for timestep t (0 = forward pass, t > 0 = backward node
V+t-1) and forward solver node i:
  R[t,i]   i is (re)computed at t            P[t,i]  its output is kept after computing
  S[t,i]   i is in memory entering t         M[t,p]  backward implementation p runs at t
  SM[p][t,i] = S[t+1,i] * M[t,p]             IP[t,i] i runs in place
  RF[c][t,k] convolution k uses kernel variant c at t
The constraints and the three memory bounds per (t, i) are the reference's.
Two exact reductions keep the model small enough for HiGHS:
  * forward nodes that no backward step at or after t can use are never
    computed or kept at t (R = S = 0 beyond a per-timestep frontier);
  * SM is only a variable where the backward node has more than one
    implementation; with a single one it is S itself.
"""
import math
import pickle
from time import time

import numpy as np
from scipy import sparse
from scipy.optimize import Bounds, LinearConstraint, milp

from .solver_info import BwdNode, IntNode, SolverInfo

CPU_GCD_MULTIPLIER = 100
MEM_GCD_MULTIPLIER = 1
GB_TO_KB = 1024 * 1024
Y = 3  # implementation slots per operator
EXCESS_PRICE = 1000.0        # objective for exceeding the budget by 100%, in total run times
EXCESS_TOLERANCE = 1e-6      # accepted excess, as a fraction of the budget


class Solution:
    def __init__(self, r, s, m, rf, ip, p, solve_time, fwd_init, bwd_init, runtime_expected):
        self.r = r
        self.s = s
        self.m = m
        self.rf = rf
        self.ip = ip
        self.p = p
        self.solve_time = solve_time
        self.fwd_init = fwd_init
        self.bwd_init = bwd_init
        self.runtime_expected = runtime_expected


class _Builder:
    """Accumulates variables, linear rows lo <= a.x <= hi and the objective."""

    def __init__(self):
        self.nvars = 0
        self.rows, self.cols, self.vals = [], [], []
        self.lo, self.hi = [], []
        self.cost = {}
        self.continuous = []  # non-negative real variables (the rest are binary)

    def var(self, continuous=False):
        self.nvars += 1
        if continuous:
            self.continuous.append(self.nvars - 1)
        return self.nvars - 1

    def add(self, terms, lo=-np.inf, hi=np.inf, const=0.0):
        """Row sum(coef * x[var]) + const within [lo, hi]; terms = [(var, coef)];
        var None is a constant 1."""
        acc = {}
        for v, c in terms:
            if c == 0:
                continue
            if v is None:
                const += c
            else:
                acc[v] = acc.get(v, 0.0) + c
        if not acc:
            if not (lo - 1e-9 <= const <= hi + 1e-9):
                raise ValueError("Infeasible: a constraint without variables is violated "
                                 "(%g not in [%g, %g])" % (const, lo, hi))
            return
        r = len(self.lo)
        for v, c in acc.items():
            self.rows.append(r)
            self.cols.append(v)
            self.vals.append(c)
        self.lo.append(lo - const)
        self.hi.append(hi - const)

    def minimise(self, terms):
        for v, c in terms:
            if v is not None and c != 0:
                self.cost[v] = self.cost.get(v, 0.0) + c


class Model:
    def __init__(self, si: SolverInfo, budget, time_limit=86400, solver="HIGHS", ablation=False,
                 mip_rel_gap=0.01, verbose=False, presolve=True, recompute_window=None,
                 excess_price=EXCESS_PRICE, accept_up_to=None, cutoff_ms=None):
        self.si = si
        # run time of a schedule already known (ms): a row keeps the search below it, so the solver
        # only has to prove that schedule optimal or beat it
        self.cutoff_ms = cutoff_ms
        self.budget = budget
        self.time_limit = time_limit
        self.solver = solver
        self.ablation = ablation
        self.mip_rel_gap = mip_rel_gap
        self.verbose = verbose
        self.presolve = presolve
        self.recompute_window = recompute_window
        self.excess_price = excess_price
        # a schedule is accepted if its peak is within this many GB (default: the budget)
        self.accept_up_to = budget if accept_up_to is None else accept_up_to
        n = si.nodes
        self.ram = np.array([math.ceil(n[i].mem * MEM_GCD_MULTIPLIER / 1024) for i in n])  # KB
        scale = lambda vals: [math.ceil(v * CPU_GCD_MULTIPLIER) for v in vals]
        self.cpu = {i: scale(n[i].workspace_compute) for i in n}
        self.cpu_recompute = {i: scale(n[i].recompute_workspace_compute) for i in n}
        self.cpu_inplace = {i: scale(n[i].inplace_workspace_compute) for i in n}

    def cmem(self, j, recompute=False, inplace=False):
        node = self.si.nodes[j]
        vals = node.inplace_workspace_mem if inplace else (
            node.recompute_workspace_mem if recompute else node.workspace_mem)
        return [math.ceil(v * MEM_GCD_MULTIPLIER * 1024) for v in vals]  # MB -> KB

    def local_memory(self, j):
        return math.ceil(self.si.nodes[j].local_memory * MEM_GCD_MULTIPLIER / 1024)

    def fixed_ram(self, j):
        return math.ceil(self.si.nodes[j].fixed_mem * MEM_GCD_MULTIPLIER / 1024)

    # ------------------------------------------------------------------ build
    def _frontier(self, V, T):
        """lim[t]: largest forward node any backward step at or after t can use."""
        si = self.si
        lim = [V - 1] * T
        for t in range(1, T):
            b = si.nodes[V + t - 1]
            f = si.bwd_to_fwd[V + t - 1]
            top = f + len(si.nodes[f].intermediates)
            for deps in b.dep_list_fwd:
                top = max([top] + [d for d in deps if d < V])
            lim[t] = top
        for t in range(T - 2, 0, -1):
            lim[t] = max(lim[t], lim[t + 1])
        return lim

    def solve(self, out_file=None):
        si = self.si
        ram = self.ram
        # budget None: minimise the peak memory itself (in GB, through a real variable) and
        # break ties by run time; useful to find out how far a model can be squeezed
        # With a budget, what the peak exceeds it by is a second real variable that the
        # objective prices above any possible gain in run time, and a solution that still
        # exceeds the budget is reported as infeasible.  (A hard bound would be the obvious
        # statement, but HiGHS 1.8 presolve then declares feasible models infeasible.)
        find_floor = self.budget is None
        V = si.loss + 1
        T = len(si.nodes) - si.loss
        lim = self._frontier(V, T)
        B = _Builder()
        ONE = None  # the constant-1 pseudo variable
        peak = [(B.var(continuous=True), -float(GB_TO_KB * MEM_GCD_MULTIPLIER))]
        budget = 0.0
        excess = None
        if not find_floor:
            excess = B.var(continuous=True)
            B.add([(peak[0][0], 1.0), (excess, -1.0)], hi=float(self.budget))

        paths = [1] + [len(si.nodes[V + t - 1].args) for t in range(1, T)]
        # Optional restriction: a backward step may only recompute forward nodes at most
        # `recompute_window` positions before its own operator.  A tensor below the window
        # cannot be produced, so it is either kept until the window reaches it or dropped right
        # after the forward pass (dropping later never helps): its S is one variable until then.
        lo_at = [0] * T
        if self.recompute_window is not None:
            lo_at = [0] + [max(0, si.bwd_to_fwd[V + t - 1] - self.recompute_window)
                           for t in range(1, T)]

        def active(t, i):
            return lo_at[t] <= i <= lim[t]

        R = [[B.var() if active(t, i) else -1 for i in range(V)] for t in range(T)]
        # S[t][i], t = 0..T; S[0] = 0; S[t+1][i] exists for i <= lim[t]
        S = [[-1] * V]
        for t in range(T):
            S.append([(B.var() if active(t, i) else S[t][i]) if i <= lim[t] else -1
                      for i in range(V)])
        if si.do_inplace:
            P = [[B.var() if active(t, i) else -1 for i in range(V)] for t in range(T)]
            IP = [[B.var() if (i in si.inplace_list and active(t, i)) else -1 for i in range(V)]
                  for t in range(T)]
        else:
            P = R
            IP = [[-1] * V for _ in range(T)]
        M = [[-2] + [-1] * (Y - 1)] + [[B.var() if p < paths[t] else -1 for p in range(Y)]
                                      for t in range(1, T)]  # -2: the constant 1 (M[0,0])
        # the product S[t+1,i] * M[t,p] is only ever needed for the forward tensors i that
        # implementation p of the backward step reads (see the memory rows below)
        SM = [[[-1] * V for _ in range(T)] for _ in range(Y)]
        for t in range(T):
            for p in range(paths[t]):
                for i in (a for a in si.nodes[V + t - 1].args[p] if a < V):
                    if S[t + 1][i] != -1:
                        SM[p][t][i] = S[t + 1][i] if paths[t] == 1 else B.var()
        RF = {}
        n_algos = si.num_conv_algos if si.select_conv_algo else 0
        for i, k in (si.conv_list.items() if si.select_conv_algo else []):
            for c in range(n_algos):
                ok = c < len(self.cpu[i]) and self.cpu[i][c] >= 0
                for t in range(T):
                    if not ok:
                        continue
                    if i < si.loss:
                        if R[t][i] != -1:
                            RF[c, t, k] = B.var()
                    elif t == i + 1 - V:
                        RF[c, t, k] = B.var()

        def term(v, coef=1.0):
            """(var, coef) with -1 = absent (0) and -2 = constant 1."""
            if v == -1:
                return (ONE, 0.0)
            if v == -2:
                return (ONE, coef)
            return (v, coef)

        # ---- structural constraints
        for t in range(T):
            for i in range(V):
                if si.do_inplace and R[t][i] != -1:
                    B.add([term(P[t][i]), term(R[t][i], -1)], hi=0)
                    if IP[t][i] != -1:
                        B.add([term(IP[t][i]), term(R[t][i], -1)], hi=0)
                if S[t + 1][i] != -1:  # stored next only if stored or produced now
                    B.add([term(S[t + 1][i]), term(S[t][i], -1), term(P[t][i], -1)], hi=0)
        if si.do_inplace:
            for v, u in si.inplace_list.items():
                if isinstance(si.nodes[v], IntNode):
                    continue
                for t in range(T):
                    if IP[t][v] == -1:
                        continue
                    B.add([term(P[t][u]), term(R[t][u], -1), term(IP[t][v], 2)], lo=0)
                    B.add([term(P[t][u]), term(IP[t][v], 2)], hi=2)
                    B.add([term(S[t + 1][u]), term(IP[t][v], 2)], hi=2)
        for i in range(V):  # the forward pass computes everything but optional intermediates
            if not isinstance(si.nodes[i], IntNode):
                B.add([term(R[0][i])], lo=1, hi=1)
        for t in range(1, T):
            B.add([term(M[t][p]) for p in range(Y)], lo=1, hi=1)  # exactly one implementation
        for p in range(Y):
            for t in range(T):
                if paths[t] == 1:
                    continue
                for i in range(V):
                    sm = SM[p][t][i]
                    if sm == -1:
                        continue
                    B.add([term(sm), term(M[t][p], -1), term(S[t + 1][i], -1)], lo=-1)
                    B.add([term(sm), term(M[t][p], -1)], hi=0)
                    B.add([term(sm), term(S[t + 1][i], -1)], hi=0)
        if self.ablation:
            for t in range(1, T):
                for i in range(V):
                    if R[t][i] != -1:
                        B.add([term(R[t][i])], hi=0)
            if si.do_inplace:
                for v in si.inplace_list:
                    for t in range(T):
                        if IP[t][v] != -1:
                            B.add([term(IP[t][v]), term(R[t][v], -1)], lo=0, hi=0)
        for (u, v, p) in si.edge_list:
            if u < V and v < V:
                for t in range(T):
                    if R[t][v] != -1:
                        B.add([term(R[t][v]), term(R[t][u], -1), term(S[t][u], -1)], hi=0)
            elif u < V <= v:
                t = v + 1 - V
                B.add([term(M[t][p]), term(P[t][u], -1), term(S[t + 1][u], -1)], hi=0)
        for i in range(V):
            for (_, intid) in si.nodes[i].intermediates:
                for t in range(T):
                    if R[t][intid] == -1:
                        continue
                    B.add([term(R[t][intid]), term(R[t][i], -1)], hi=0)
                    if si.do_inplace and i in si.inplace_list:
                        B.add([term(IP[t][intid]), term(IP[t][i], -1), term(R[t][intid], -1)], lo=-1)
                        B.add([term(IP[t][intid]), term(IP[t][i], -1)], hi=0)
        if si.select_conv_algo:
            for i, k in si.conv_list.items():
                if i < si.loss:
                    for t in range(T):
                        if R[t][i] != -1:
                            B.add([term(RF.get((c, t, k), -1)) for c in range(n_algos)] +
                                  [term(R[t][i], -1)], lo=0)
                else:
                    t = i + 1 - V
                    B.add([term(RF.get((c, t, k), -1)) for c in range(n_algos)], lo=1)

        # ---- memory constraints
        gradm = [(self.local_memory(V + t - 1) if t else 0) + self.fixed_ram(V + t - 2)
                 for t in range(T)]
        keep = [[[] for _ in range(T)] for _ in range(Y)]  # keep[p][t] = [i < j in args_p(t)]
        args_at = [[set(a for a in path if a < V) for path in si.nodes[V + t - 1].args]
                   for t in range(T)]
        # W[t] = sum_{i>=j} S[t,i] ram_i + sum_{i<j} S[t+1,i] ram_i, carried from j to j+1 as a
        # real variable so that every memory row stays short
        W = [None] * T
        for j in range(V):
            local_j = self.local_memory(j)
            ws_first = self.cmem(j)
            ws_again = self.cmem(j, recompute=True)
            ws_inpl = self.cmem(j, inplace=True)
            sm2_zero = si.nodes[j].local_tensors
            for t in range(T):
                jmax = (lim[t - 1] if t else V - 1) + 1  # rows beyond repeat the row at jmax
                if j > jmax:
                    continue
                same = j > 0 and S[t][j - 1] == S[t + 1][j - 1]
                if not same:
                    w = B.var(continuous=True)
                    if j == 0:
                        B.add([(w, -1.0)] + [term(S[t][i], float(ram[i])) for i in range(V)],
                              lo=0, hi=0)
                    else:
                        B.add([(w, -1.0), (W[t], 1.0), term(S[t][j - 1], -float(ram[j - 1])),
                               term(S[t + 1][j - 1], float(ram[j - 1]))], lo=0, hi=0)
                    W[t] = w
                common = [(ONE, gradm[t]), (W[t], 1.0)]
                for p in range(paths[t]):
                    kp = keep[p][t]
                    if kp:
                        common.append(term(M[t][p], float(sum(ram[i] for i in kp))))
                        common.extend(term(SM[p][t][i], -float(ram[i])) for i in kp)
                if not (same and all(j - 1 not in a for a in args_at[t])):
                    B.add(common + peak, hi=budget)  # else: the row written for j - 1
                if R[t][j] == -1:
                    continue
                m2 = list(common)
                ws = ws_first if t == 0 else ws_again
                if si.select_conv_algo and j in si.conv_list:
                    k = si.conv_list[j]
                    m2.extend(term(RF.get((c, t, k), -1), float(ws[c])) for c in range(len(ws)))
                elif si.do_inplace and j in si.inplace_list:
                    m2.append(term(IP[t][j], float(ws_inpl[0] - ws[0])))
                    m2.append(term(R[t][j], float(ws[0])))
                else:
                    m2.append(term(R[t][j], float(ws[0])))
                m2.append(term(R[t][j], float(ram[j] + local_j)))
                m2.append(term(S[t][j], -float(ram[j])))
                m2.extend(term(S[t][i] if i > j else S[t + 1][i], -float(ram[i]))
                          for i in sm2_zero if i != j and i < V)
                B.add(m2 + peak, hi=budget)
            for t in range(T):
                for p in range(paths[t]):
                    if j in args_at[t][p]:
                        keep[p][t].append(j)
        for t in range(1, T):
            b = V + t - 1
            node = si.nodes[b]
            row = [(ONE, self.local_memory(b) + self.fixed_ram(b) + float(ram[b]))]
            wmem = self.cmem(b)
            if si.select_conv_algo and b in si.conv_list:
                k = si.conv_list[b]
                row.extend(term(RF.get((c, t, k), -1), float(wmem[c])) for c in range(len(wmem)))
            else:
                row.extend(term(M[t][p], float(wmem[p])) for p in range(paths[t]))
            for p in range(paths[t]):
                row.append(term(M[t][p], float(sum(ram[i] for i in keep[p][t]))))
                # sum over i not read by p of S[t+1,i] * M[t,p], using sum_p M[t,p] = 1
                row.extend(term(SM[p][t][i], -float(ram[i])) for i in node.dep_list_fwd[p] if i < V)
            row.extend(term(S[t + 1][i], float(ram[i])) for i in range(V))
            B.add(row + peak, hi=budget)

        # ---- objective
        obj = []
        conv = si.conv_list if si.select_conv_algo else {}
        for i in range(V):
            if i in conv:
                continue
            obj.append(term(R[0][i], self.cpu[i][0]))
            obj.extend(term(R[t][i], self.cpu_recompute[i][0]) for t in range(1, T))
        conv_node = {k: i for i, k in conv.items()}
        for (c, t, k), v in RF.items():
            obj.append((v, self.cpu[conv_node[k]][c]))
        if si.do_inplace:
            for i in si.inplace_list:
                obj.extend(term(IP[t][i], self.cpu_inplace[i][0] - self.cpu[i][0])
                           for t in range(T))
        for t in range(T):
            b = V + t - 1
            if b in conv:
                continue
            obj.extend(term(M[t][p], self.cpu[b][p]) for p in range(Y)
                       if p < len(self.cpu[b]) and M[t][p] != -1)
        const_cost = sum(c for v, c in obj if v is None)
        if find_floor:
            total = sum(abs(c) for v, c in obj) + 1.0
            # run time only breaks ties: all of it weighs 1e-4 of the activations' size
            tie = 1e-4 * float(sum(ram[:V])) / (GB_TO_KB * MEM_GCD_MULTIPLIER)
            obj = [(v, c / total * tie) for v, c in obj] + [(peak[0][0], 1.0)]
            const_cost = 0.0
        else:
            total = sum(abs(c) for v, c in obj) + 1.0
            if self.cutoff_ms is not None:
                B.add([(v, c) for v, c in obj if v is not None],
                      hi=self.cutoff_ms * CPU_GCD_MULTIPLIER - const_cost)
            obj = obj + [(excess, self.excess_price * total / float(self.budget))]
        B.minimise(obj)

        # ---- solve
        n = B.nvars
        A = sparse.csr_matrix((B.vals, (B.rows, B.cols)), shape=(len(B.lo), n))
        cvec = np.zeros(n)
        for v, c in B.cost.items():
            cvec[v] = c
        if self.verbose:
            print(f"[solver] {n - len(B.continuous)} binaries, {len(B.continuous)} reals, {A.shape[0]} rows, {A.nnz} non-zeros")
        t0 = time()
        integrality, upper = np.ones(n), np.ones(n)
        integrality[B.continuous] = 0
        upper[B.continuous] = np.inf
        res = milp(cvec, constraints=LinearConstraint(A, np.array(B.lo), np.array(B.hi)),
                   integrality=integrality, bounds=Bounds(0, upper),
                   options={"time_limit": float(self.time_limit), "mip_rel_gap": self.mip_rel_gap,
                            "disp": bool(self.verbose), "presolve": bool(self.presolve)})
        solve_time = time() - t0
        if res.x is None:
            raise ValueError("Model infeasible" if res.status == 2 else
                             f"no schedule found: {res.message}")
        self.last_excess = float(res.x[excess]) if excess is not None else 0.0
        # how far the incumbent may be from the optimum (large when the time limit ended the search)
        self.last_gap = float(getattr(res, "mip_gap", float("nan")))
        if excess is not None and \
                self.budget + res.x[excess] > self.accept_up_to * (1.0 + EXCESS_TOLERANCE):
            raise ValueError("Model infeasible: the cheapest schedule found needs %.3f GB, budget "
                             "%.3f GB" % (self.budget + res.x[excess], self.budget))
        x = np.around(res.x)

        def val(v):
            return 0.0 if v == -1 else (1.0 if v == -2 else x[v])

        # 0/1 tables as bytes: a ResNet-50 solution stays a few hundred KB on disk
        table = lambda rows: np.array(rows, dtype=np.uint8)
        r = table([[val(R[t][i]) for i in range(V)] for t in range(T)])
        pp = table([[val(P[t][i]) for i in range(V)] for t in range(T)])
        s = table([[val(S[t][i]) for i in range(V)] for t in range(T + 1)])
        m = table([[val(M[t][p]) for p in range(Y)] for t in range(T)])
        ip = table([[val(IP[t][i]) for i in range(V)] for t in range(T)])
        rf = np.zeros((T, len(conv), max(n_algos, 1)), dtype=np.uint8)
        for (c, t, k), v in RF.items():
            rf[t, k, c] = x[v]
        run_time = float(res.fun + const_cost)
        if excess is not None:  # without what an accepted overshoot of the target was charged
            run_time -= float(cvec[excess] * res.x[excess])
        solution = Solution(r, s, m, rf, ip, pp, solve_time, float("nan"), float("nan"), run_time)
        solution.mip_gap = self.last_gap
        if out_file is not None:
            with open(out_file, 'wb') as f:
                pickle.dump([si, solution], f)
        return solution


def solve_within_budget(si, budget, time_limit=86400, solver="HIGHS", ablation=False,
                        out_file=None, rounds=6, **options):
    """Model(si, budget).solve(), with a fallback for tight budgets.  HiGHS can spend its whole
    time limit without an incumbent when every schedule it tries overshoots a tight budget at
    the (deliberately prohibitive) default price.  The fallback solves the same model against
    a slightly LOWER target with a MODERATE price on the overshoot - any schedule is then an
    acceptable incumbent and the price steers the search - and tightens the target until a
    schedule fits the real budget.  What comes out fits the budget; it need not be optimal."""
    # the plain model gets the larger share: an incumbent it returns at its time limit is
    # accepted as it is, however far from the optimum (the achieved gap is reported)
    first = max(30.0, 0.6 * time_limit) if rounds else time_limit
    per_solve = max(30.0, (time_limit - first) / max(rounds, 1))
    try:
        return Model(si, budget, first, solver, ablation, **options).solve(out_file=out_file)
    except ValueError as e:
        if "cheapest schedule found" not in str(e) or not rounds:
            raise
        first_error = e
    target, price = float(budget), 4.0
    for _ in range(rounds):
        m = Model(si, target, per_solve, solver, ablation, excess_price=price,
                  accept_up_to=budget, **options)
        try:
            return m.solve(out_file=out_file)  # fits the real budget (it may overshoot the target)
        except ValueError as e:
            if "cheapest schedule found" not in str(e):
                raise
        # aim lower by what was missing and make overshooting dearer
        target = max(0.5 * budget, target - 1.5 * (target + m.last_excess - budget))
        price *= 3.0
    raise first_error


def solution_file_name(model_name, bs, mode, budget):
    return "solution_%s_%d_%s_%.2f.pkl" % (model_name, bs, mode, budget)


def main(argv=None):
    """`python -m monet_amd.solver MODEL BATCH_SIZE BUDGET MODE SOLVER [--time_limit S]`
    (reference: monet/cvxpy_solver.py:336-384).  Profiling needs the GPU, solving does not:
    `--profile_only` stops after writing the profiled solver info to --data_dir, `--si_file`
    solves from such a file on a machine without a GPU."""
    import argparse

    import torch

    from .graph import Graph, fusion_level
    from .models import build_model

    parser = argparse.ArgumentParser()
    parser.add_argument('model')
    parser.add_argument('bs', type=int)
    parser.add_argument('budget', type=float, help="memory budget in GB")
    parser.add_argument('mode')
    parser.add_argument('solver', nargs='?', default="HIGHS")
    parser.add_argument("--ablation", action="store_true", help="no recomputation")
    parser.add_argument("--time_limit", default=86400, type=int, help="solver time limit, seconds")
    parser.add_argument("--gap", default=0.01, type=float, help="relative optimality gap")
    parser.add_argument("--window", default=None, type=int,
                        help="only recompute forward nodes this close below the running "
                             "backward step (smaller model, possibly costlier schedule)")
    parser.add_argument("--data_dir", default="data", help="where profiles and solutions go")
    parser.add_argument("--si_file", default="", help="profiled solver info to solve from")
    parser.add_argument("--profile_only", action="store_true")
    parser.add_argument("--rounds", default=6, type=int,
                        help="tightening-target rounds to fall back on when the direct solve ends "
                             "without a fitting schedule (0: one solve with the whole time limit)")
    parser.add_argument("--reserve_mb", default=0.0, type=float,
                        help="MiB of the budget to leave to what the schedule does not hold "
                             "(optimizer state, loss tensors, allocator rounding): the model is "
                             "solved against BUDGET minus this, the file keeps BUDGET in its name")
    parser.add_argument("--cutoff_ms", default=None, type=float,
                        help="run time of a known schedule: only look for schedules at most this slow")
    parser.add_argument("--verbose", action="store_true")
    args = parser.parse_args(argv)

    from pathlib import Path
    Path(args.data_dir).mkdir(parents=True, exist_ok=True)
    if args.si_file:
        with open(args.si_file, 'rb') as f:
            si = pickle.load(f)
        model_name = si.model_name
    else:
        model, input_shape, model_name = build_model(args.model)
        graph = Graph.create(model, input_shape=input_shape, fuse_bn_relu=fusion_level(args.mode))
        model.cuda()
        input_ = torch.randn([args.bs, *input_shape]).cuda()
        si = SolverInfo(args.bs, model_name=model_name, mode=args.mode, data_dir=args.data_dir)
        si.extract(graph, input_, *list(model.state_dict(keep_vars=True).values()))
        print("profiled %d solver nodes -> %s" % (len(si.nodes), args.data_dir))
        if args.profile_only:
            return None
    print("Memory budget", args.budget, "GB; batch size", si.bs, "; model", model_name,
          "; mode", args.mode)
    out = Path(args.data_dir) / solution_file_name(model_name, si.bs, args.mode, args.budget)
    solution = solve_within_budget(si, args.budget - args.reserve_mb / 1024.0, args.time_limit,
                                   args.solver, args.ablation,
                                   out_file=str(out), rounds=args.rounds, mip_rel_gap=args.gap,
                                   verbose=args.verbose,
                                   recompute_window=args.window, cutoff_ms=args.cutoff_ms)
    gap = getattr(solution, "mip_gap", float("nan"))
    print("solved in %.1f s, expected run time %.2f ms, gap %.2f %% -> %s" % (
        solution.solve_time, solution.runtime_expected / CPU_GCD_MULTIPLIER, 100.0 * gap, out))
    if gap == gap and gap > max(0.05, 10.0 * args.gap):
        print("warning: the search ended at its time limit %.0f %% above the best bound; "
              "a longer --time_limit (or --rounds 0) may find a cheaper schedule" % (100.0 * gap))
    return solution


if __name__ == '__main__':
    # run the module under its real name, so that pickles refer to monet_amd.solver.Solution
    from monet_amd.solver import main as _main
    _main()
