"""Solver view of a training step (reference: monet/solver_info.py).

`SolverInfo.extract(graph, input, *params)` turns the operator graph into the
node list the schedule solver works on:

  0 .. loss-1      forward nodes in execution order; an operator that can keep
                   a compact intermediate (ReLU mask, pool indices) is followed
                   by one `IntNode` per such implementation
  loss             the loss node
  loss+1 .. size-1 backward nodes in reverse forward order; convolution and
                   fully connected layers get two (`param_grad`, then `ip_grad`)

and annotates every node with tensor sizes, the tensors that must stay alive
around it, and - by running each operator implementation and kernel variant on
the GPU (monet_amd.meminfo) - its workspace (MB) and run time (ms).

The mode string follows the reference (solver_info.py:96-100): an optional
`inplace_` prefix enables in-place selection, `conv` enables per-convolution
kernel-variant selection, `newnode` enables the intermediate-keeping
implementations, `multiway` the output-keeping ones.
"""
import pickle
import sys
from collections import defaultdict
from pathlib import Path

import numpy as np

from . import lm_ops
from .graph import ComputeNode, Graph, Input, Param, fusion_level, is_batch_norm, two_step_backward

MEMORY_MULTIPLIER = 4  # bytes per element of an fp32 tensor: the reference's constant
#                        (solver_info.py:10); SolverInfo.elem_bytes holds the size in use


class SolverNode:
    def __init__(self):
        self.input_shapes = []
        self.output_shapes = []
        self.local_tensors = set()  # tensors alive while this node is (re)computed
        self.local_memory = -1      # their bytes
        self.mem = -1               # bytes of this node's output
        self.workspace_mem = []     # MB beyond inputs and outputs, per implementation / variant
        self.fixed_mem = -1         # inputs + parameters (+ parameter gradients so far)
        self.workspace_compute = []  # ms, per implementation / variant
        self.last_used = -1
        self.recompute_workspace_mem = []
        self.recompute_workspace_compute = []
        self.inplace_workspace_mem = []
        self.inplace_workspace_compute = []


class BwdNode(SolverNode):
    def __init__(self, fwd_node, fwd_id, num_bwd, bwd_op="ip_grad"):
        super().__init__()
        self.fwd_node = fwd_node
        self.fwd_id = fwd_id
        self.bwd_op = bwd_op
        self.stored = []  # parameters whose gradients this node produces
        self.num_bwd = num_bwd
        self.dep_list_fwd = [[] for _ in range(num_bwd)]
        self.dep_list_bwd = [[] for _ in range(num_bwd)]
        self.args = [[] for _ in range(num_bwd)]
        self.has_intermediates = False

    def __repr__(self):
        if two_step_backward(self.fwd_node):
            return '<BwdNode %s %s>' % (self.fwd_node, self.bwd_op)
        return '<BwdNode %s>' % self.fwd_node.op

    def make_args(self):
        self.op = self.fwd_node.op + "_" + self.bwd_op
        for p in range(self.num_bwd):
            self.args[p] = self.dep_list_fwd[p] + self.dep_list_bwd[p]


class FwdNode(SolverNode):
    def __init__(self, node):
        super().__init__()
        self.gnode = node
        self.op = node.op
        self.inbound_nodes = []
        self.args = [[]]
        self.has_intermediates = False
        self.intermediates = []  # (implementation index, solver id of the IntNode)

    def make_args(self):
        self.args = [self.inbound_nodes]

    def __repr__(self):
        return '%s' % self.gnode


class IntNode(FwdNode):
    def __init__(self, node, solver_parent_id, op_idx):
        super().__init__(node)
        self.solver_parent_id = solver_parent_id
        self.op_idx = op_idx

    def __repr__(self):
        return 'Int::%s' % self.gnode


def _nbytes(shape, bs, elem_bytes=MEMORY_MULTIPLIER):
    n = int(np.prod(shape)) if len(shape) else 1
    n = n * elem_bytes
    return -n * bs if n < 0 else n


class SolverInfo:
    def __init__(self, bs, model_name, mode, data_dir=None):
        self.nodes = {}
        self.newnodes = []
        self.loss = 0
        self.edge_list = []
        self.fwd_to_bwd = {}
        self.bwd_to_fwd = {}
        self.solver_to_graph = []
        self.graph_to_solver = {}

        self.bs = bs
        # bytes per element of the activations, parameters and gradients the sizes are
        # computed for: 4 (fp32) unless `extract` is given tensors of another floating type
        self.elem_bytes = MEMORY_MULTIPLIER
        self.model_name = model_name
        self.mode = mode
        self.data_path = "%s_%d_%s" % (model_name, bs, mode)
        self.data_dir = None if data_dir is None else str(data_dir)

        self.select_conv_algo = "conv" in mode
        self.do_inplace = "inplace" in mode
        self.compute_newnode = "newnode" in mode
        # "fused_": the graph was traced with BatchNorm+ReLU pairs as single operators
        # "fused2_": also BatchNorm + add + ReLU triples (the end of a residual block)
        self.fuse_bn_relu = fusion_level(mode)
        # the registry knows nothing of these prefixes
        self.mode = mode.replace("fused2_", "").replace("fused_", "").replace("inplace_", "")

    # ------------------------------------------------------------------ build
    def extract(self, graph: Graph, *args, cost_fn=None):
        """Build the solver graph and profile it.  `args` = (input, *parameters),
        indexed like the graph's nodes.  `cost_fn(n, op, bwd_op)` may replace the
        GPU measurement; it returns (meminfo triple, computeinfo triple)."""
        if args and hasattr(args[0], "is_floating_point") and args[0].is_floating_point():
            self.elem_bytes = int(args[0].element_size())   # bf16 / fp16 models: 2
        for i, n in enumerate(graph.nodes):
            if not (isinstance(n, ComputeNode) and n.has_backward):
                continue
            self.solver_to_graph.append(i)
            self.graph_to_solver[i] = len(self.solver_to_graph) - 1
            sid = len(self.nodes)
            node = FwdNode(n)
            node.inbound_nodes = [self.graph_to_solver[dep] for dep, grad in n.dependencies
                                  if isinstance(graph.nodes[dep], ComputeNode)]
            self.nodes[sid] = node
            for idx, op in enumerate(lm_ops.list_ops(self.mode, n.op)):
                storage = op.backward_storage
                for st in (storage if isinstance(storage, list) else [storage]):
                    if isinstance(st, lm_ops.IntermediateStorage):
                        ni = ComputeNode([st.size(n.shape)], -1, "int::" + op.__name__, [], False)
                        self.solver_to_graph.append(-1)
                        iid = len(self.nodes)
                        inode = IntNode(ni, sid, idx)
                        inode.inbound_nodes = [sid]
                        self.nodes[iid] = inode
                        self.newnodes.append(iid)
                        node.has_intermediates = True
                        node.intermediates.append((idx, iid))

        self.loss = len(self.nodes)
        nloss = ComputeNode(self.nodes[self.loss - 1].gnode.shape, -2, "loss::loss", [], False)
        self.nodes[self.loss] = FwdNode(nloss)
        self.nodes[self.loss].inbound_nodes = [self.loss - 1]
        self.extract_deps(graph)
        self.get_mem()
        self.get_local_memory()
        self.get_fixed_memory(graph)
        self.get_conv_info()
        self.get_inplace_info()
        self.get_workspace_cost(graph, *args, cost_fn=cost_fn)
        self.size = len(self.nodes)
        if self.data_dir is not None:
            with open(Path(self.data_dir) / ("si_" + self.data_path + ".pkl"), 'wb') as f:
                pickle.dump(self, f)

    def _impls(self, op):
        return lm_ops.list_ops(self.mode, op)

    def extract_deps(self, graph):
        # backward nodes, in reverse forward order
        for i in sorted(self.nodes, reverse=True):
            if i > self.loss or not self.nodes[i].gnode.has_backward:
                continue
            num_bwd = len(self._impls(self.nodes[i].op))
            if two_step_backward(self.nodes[i].gnode):
                self.bwd_to_fwd[len(self.nodes)] = i
                self.nodes[len(self.nodes)] = BwdNode(self.nodes[i].gnode, i, num_bwd, "param_grad")
                self.fwd_to_bwd[i] = len(self.nodes)  # points at the input-gradient node
                self.bwd_to_fwd[len(self.nodes)] = i
                self.nodes[len(self.nodes)] = BwdNode(self.nodes[i].gnode, i, num_bwd, "ip_grad")
            else:
                self.fwd_to_bwd[i] = len(self.nodes)
                self.bwd_to_fwd[len(self.nodes)] = i
                self.nodes[len(self.nodes)] = BwdNode(self.nodes[i].gnode, i, num_bwd)
        self.fwd_to_bwd[self.loss] = self.loss

        for i in list(self.nodes):
            node = self.nodes[i]
            if isinstance(node, BwdNode) or not node.gnode.has_backward:
                continue
            # the gradient of i's inputs needs the gradient of i
            for ni in node.inbound_nodes:
                prev = self.nodes[ni]
                for p in range(len(self._impls(prev.op))):
                    self.nodes[self.fwd_to_bwd[ni]].dep_list_bwd[p].append(self.fwd_to_bwd[i])
                    if two_step_backward(prev.gnode):
                        self.nodes[self.fwd_to_bwd[ni] - 1].dep_list_bwd[p].append(self.fwd_to_bwd[i])
            ops = self._impls(node.op)
            num_bwd = len(ops)
            if two_step_backward(node.gnode):
                assert len(node.inbound_nodes) <= 1
                if len(node.inbound_nodes) == 1:
                    for p in range(num_bwd):  # the parameter gradient needs the layer's input
                        self.nodes[self.fwd_to_bwd[i] - 1].dep_list_fwd[p].append(node.inbound_nodes[0])
            else:
                for p in range(num_bwd):
                    deps = ops[p].backward_storage
                    needed = []
                    for dep in (deps if isinstance(deps, list) else [deps]):
                        if isinstance(dep, lm_ops.InputStorage):
                            for k in dep.ids:
                                a = node.gnode.args[k]
                                if isinstance(a, ComputeNode.D) and \
                                        isinstance(graph.nodes[a.index], ComputeNode):
                                    needed.append(self.graph_to_solver[a.index])
                        if isinstance(dep, lm_ops.OutputStorage):
                            needed.append(i)
                        if isinstance(dep, lm_ops.IntermediateStorage):
                            mine = [iid for (p_opt, iid) in node.intermediates if p_opt == p]
                            assert mine, "implementation keeps an intermediate but has no IntNode"
                            needed.extend(mine)
                    self.nodes[self.fwd_to_bwd[i]].dep_list_fwd[p] = needed
            if i == self.loss - 1:  # the last operator's backward starts from the loss
                for p in range(num_bwd):
                    self.nodes[self.fwd_to_bwd[i]].dep_list_fwd[p].append(self.loss)
                    if two_step_backward(node.gnode):
                        self.nodes[self.fwd_to_bwd[i] - 1].dep_list_fwd[p].append(self.loss)

        for i in range(self.loss + 1):
            self.nodes[i].make_args()
        for i in range(self.loss + 1, len(self.nodes)):
            b = self.nodes[i]
            b.make_args()
            stored, output_shapes = [], []
            for dep, rgrad in b.fwd_node.dependencies:
                nin = graph.nodes[dep]
                if isinstance(nin, Param):
                    if rgrad:
                        stored.append(nin)
                elif isinstance(nin, (ComputeNode, Input)):
                    if rgrad:
                        output_shapes.append(list(nin.shape))
                else:
                    sys.exit("Unknown node encountered")
            if two_step_backward(b.fwd_node):
                if b.bwd_op == "ip_grad":
                    stored = []
                else:
                    output_shapes = []
            b.output_shapes = output_shapes
            b.stored = stored

        self.edge_list = [(u, v, k) for v in self.nodes
                          for k, vdeps in enumerate(self.nodes[v].args) for u in vdeps]

    def _eb(self):
        return getattr(self, "elem_bytes", MEMORY_MULTIPLIER)   # (older profile files lack it)

    def get_mem(self):
        for i, node in self.nodes.items():
            if isinstance(node, BwdNode):
                node.mem = sum(_nbytes(s, self.bs, self._eb()) for s in node.output_shapes)
            else:
                node.mem = _nbytes(list(node.gnode.shape), self.bs, self._eb())
                if "int::" in node.op:
                    # an intermediate's "shape" already is its size in bytes (per sample when
                    # the batch is symbolic)
                    node.mem = int(node.mem / self._eb())

    def get_local_memory(self):
        present = -1
        for v in self.nodes:
            for u in self.nodes[v].args[0]:
                if v > self.loss and u < self.loss:
                    continue  # forward tensors are not part of a backward node's working set
                self.nodes[v].local_tensors.add(u)
                self.nodes[u].last_used = v
                if u != present:
                    for ni in range(u + 1, v):
                        self.nodes[ni].local_tensors.add(u)
            present = v
        for node in self.nodes.values():
            node.local_memory = sum(self.nodes[u].mem for u in node.local_tensors)

    def get_fixed_memory(self, graph):
        fixed = 0
        for i in range(self.loss):
            for a in self.nodes[i].gnode.args:
                if isinstance(a, ComputeNode.D) and isinstance(graph.nodes[a.index], (Param, Input)):
                    fixed += _nbytes(list(graph.nodes[a.index].shape), self.bs, self._eb())
        self.nodes[0].fixed_mem = fixed
        for i in self.nodes:
            if i == 0:
                continue
            self.nodes[i].fixed_mem = self.nodes[i - 1].fixed_mem
            if i <= self.loss:
                continue
            for prm in self.nodes[i].stored:  # parameter gradients accumulate through the backward
                self.nodes[i].fixed_mem += _nbytes(list(prm.shape), self.bs, self._eb())

    def get_conv_info(self):
        self.conv_list = {}
        convop = self._impls('aten::_convolution')[0]
        self.num_conv_algos = 1
        if self.select_conv_algo:
            self.num_conv_algos = max(convop.n_fwd_algos(), convop.n_bwd_ip_algos(),
                                      convop.n_bwd_wt_algos())
            for i, node in self.nodes.items():
                g = node.fwd_node if isinstance(node, BwdNode) else node.gnode
                if "convolution" in node.op and not g.is_depthwise:
                    self.conv_list[i] = len(self.conv_list)

    def get_inplace_info(self):
        """inplace_list[v] = u: operator v may overwrite its input u, because v is u's last
        reader in the forward pass.  u is always v's FIRST tensor argument, the one the
        in-place kernels write (the reference takes the last argument whose last reader is v,
        solver_info.py:444-456, which for `a += b` can name b while a is overwritten)."""
        self.inplace_list = {}
        if not self.do_inplace:
            return
        for v in range(self.loss):
            node = self.nodes[v]
            if isinstance(node, IntNode):
                continue
            if not hasattr(self._impls(node.op)[0], 'inplace'):
                continue
            first = node.gnode.args[0]
            if not isinstance(first, ComputeNode.D) or first.index not in self.graph_to_solver:
                continue
            u = self.graph_to_solver[first.index]
            if self.nodes[u].last_used == v:
                self.inplace_list[v] = u
                for _, intmd in node.intermediates:
                    self.inplace_list[intmd] = u

    # ---------------------------------------------------------------- profile
    def _cost_file(self):
        return None if self.data_dir is None else Path(self.data_dir) / ("cost_" + self.data_path + ".pkl")

    def get_workspace_cost(self, graph, *args, cost_fn=None):
        fields = ("workspace_mem", "workspace_compute", "recompute_workspace_mem",
                  "recompute_workspace_compute", "inplace_workspace_mem", "inplace_workspace_compute")
        cost = self._cost_file()
        if cost is not None and cost.is_file():
            with open(cost, 'rb') as f:
                tables = pickle.load(f)
            assert len(tables[0]) == len(self.nodes) and len(tables[1]) == len(self.nodes)
            for i in self.nodes:
                for name, table in zip(fields, tables):
                    setattr(self.nodes[i], name, table[i])
            return

        if cost_fn is None:
            from .meminfo import computeinfo, meminfo

            def cost_fn(n, op, bwd_op):
                common = (n, op, graph, self.bs, bwd_op, self.select_conv_algo, self.do_inplace)
                return meminfo(*common, *args), computeinfo(*common, *args)

        for i in sorted(self.nodes.keys(), reverse=True):
            node = self.nodes[i]
            if isinstance(node, BwdNode):
                b, n = node, node.fwd_node
                fwd = self.nodes[self.bwd_to_fwd[i]]
                for op_impl in self._impls(n.op):
                    (fmem, bmem, fmem_re), (ftime, btime, ftime_re) = cost_fn(n, op_impl(), b.bwd_op)
                    if self.select_conv_algo and self.bwd_to_fwd[i] in self.conv_list:
                        b.workspace_mem.extend(bmem)
                        b.workspace_compute.extend(btime)
                        if b.bwd_op != "ip_grad":
                            fwd.workspace_mem.extend(fmem)
                            fwd.workspace_compute.extend(ftime)
                    elif self.do_inplace and self.bwd_to_fwd[i] in self.inplace_list:
                        b.workspace_mem.append(bmem[0])
                        b.workspace_compute.append(btime[0])
                        fwd.workspace_mem.append(fmem[0])
                        fwd.workspace_compute.append(ftime[0])
                        fwd.inplace_workspace_mem.append(fmem[1])
                        fwd.inplace_workspace_compute.append(ftime[1])
                    else:
                        b.workspace_mem.append(bmem[0])
                        b.workspace_compute.append(btime[0])
                        if not (two_step_backward(n) and b.bwd_op == "ip_grad"):
                            if is_batch_norm(n.op):
                                fwd.recompute_workspace_mem.append(fmem_re[0])
                                fwd.recompute_workspace_compute.append(ftime_re[0])
                            fwd.workspace_mem.append(fmem[0])
                            fwd.workspace_compute.append(ftime[0])
            elif "int::" in node.op:
                parent = self.nodes[node.solver_parent_id]
                p = node.op_idx
                node.workspace_mem.append(parent.workspace_mem[p])
                node.workspace_compute.append(parent.workspace_compute[p] - parent.workspace_compute[0])
                if self.do_inplace and node.solver_parent_id in self.inplace_list:
                    node.inplace_workspace_mem.append(parent.inplace_workspace_mem[p])
                    node.inplace_workspace_compute.append(
                        parent.inplace_workspace_compute[p] - parent.inplace_workspace_compute[0])
            elif "loss::" in node.op:  # the loss is taken to be free
                node.workspace_compute.append(0)
                node.workspace_mem.append(0)

        for node in self.nodes.values():
            if len(node.recompute_workspace_mem) == 0:
                node.recompute_workspace_mem = node.workspace_mem
                node.recompute_workspace_compute = node.workspace_compute
            if len(node.inplace_workspace_mem) == 0:
                node.inplace_workspace_mem = node.workspace_mem
                node.inplace_workspace_compute = node.workspace_compute
        if cost is not None:
            tables = [{i: getattr(self.nodes[i], name) for i in self.nodes} for name in fields]
            with open(cost, 'wb') as f:
                pickle.dump(tables, f)
