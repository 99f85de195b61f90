"""Flat operator graph of a model's forward pass (reference: monet/graph.py).

`Graph.create(model, input_shape)` JIT-traces the model on the CPU and records,
in execution order, one node per graph input (`Input`), per parameter / buffer
(`Param`) and per aten operator (`ComputeNode`).  A compute node's arguments
are either constants (`ComputeNode.V`) or references to earlier nodes
(`ComputeNode.D(index, requires_grad)`).  The batch dimension is symbolic: the
trace runs at batch TRACE_BATCH and every dimension of that size is recorded
as -1, like the reference does (monet/graph.py:104,171).

Differences from the reference that current PyTorch forces:
  * connectivity to the data input is computed by reachability over the trace
    (the reference matches the substring "input" in value names, graph.py:124-133);
  * operators that neither depend on the data input nor feed anything (the
    in-place update of BatchNorm's `num_batches_tracked`) are left out;
  * constants are read with `toIValue()`, which also covers int lists.
"""
from functools import lru_cache

import torch

TRACE_BATCH = 23


class Node:
    def __init__(self, shape):
        self.shape = shape


class Input(Node):
    def __repr__(self):
        return '<Input %s>' % str(list(self.shape))


class Param(Node):
    def __repr__(self):
        return '<Param %s>' % str(list(self.shape))


class ComputeNode(Node):
    class Arg:
        pass

    class V(Arg):
        """A constant argument."""

        def __init__(self, v):
            self.value = v

        def __repr__(self):
            return '<V %s>' % str(self.value)

    class D(Arg):
        """A tensor argument: the output of graph node `index`."""

        def __init__(self, index, requires_grad=False):
            self.index = index
            self.requires_grad = requires_grad

        def __repr__(self):
            return '<D %d %d>' % (self.index, self.requires_grad)

    def __init__(self, shape, nodeid, op, args, has_backward, is_depthwise=False):
        super().__init__(shape)
        self._op = op
        self._args = args
        self.id = nodeid
        self._has_backward = has_backward
        self._is_depthwise = is_depthwise

    @property
    def op(self):
        return self._op

    @property
    def args(self):
        return self._args

    @property
    def has_backward(self):
        return self._has_backward

    @property
    def is_depthwise(self):
        return self._is_depthwise

    @property
    @lru_cache(maxsize=None)
    def dependencies(self):
        """[(node index, requires_grad)] of the tensor arguments, in order."""
        return [(a.index, a.requires_grad) for a in self._args if isinstance(a, self.D)]

    def __repr__(self):
        return '<Op %s %s>' % (str(self._op), str(list(self.shape)))


FUSED_BN_RELU = "monet::batch_norm_relu"
FUSED_ADD_RELU = "monet::add_relu"
FUSED_BN_ADD_RELU = "monet::batch_norm_add_relu"
_FUSABLE = {"aten::batch_norm": FUSED_BN_RELU, "aten::add_": FUSED_ADD_RELU, "aten::add": FUSED_ADD_RELU}


def fusion_level(mode):
    """Fusion level named by a mode string: "fused2_..." = 2 (pairs and BatchNorm + add + ReLU
    triples), "fused_..." = 1 (pairs), anything else 0."""
    return 2 if "fused2_" in mode else (1 if "fused" in mode else 0)


def is_batch_norm(op_name):
    """BatchNorm, alone or fused with the ReLU behind it: operators whose first forward of a
    step computes statistics that recomputations and the backward must reuse."""
    return op_name in ("aten::batch_norm", FUSED_BN_RELU, FUSED_BN_ADD_RELU)


def two_step_backward(node):
    """Operators whose backward is split into a parameter-gradient step and an
    input-gradient step (non-depthwise convolution and the fully connected
    layer in either of its traced forms)."""
    return (node.op == "aten::_convolution" and not node.is_depthwise) or \
        node.op in ("aten::addmm", "aten::linear")


class Graph:
    def __init__(self):
        self._nodes = []
        self._outputs = []

    @property
    def nodes(self):
        return self._nodes

    def _add(self, node):
        self._nodes.append(node)
        return len(self._nodes) - 1

    def fuse_batch_norm_relu(self):
        """New graph in which every BatchNorm or residual add whose only reader is a ReLU forms
        ONE node with it (`monet::batch_norm_relu` / `monet::add_relu`, with the arguments of the
        first operator).  The reference has no such pass; a fused pair makes one pass over the
        activation where the two operators make two."""
        nodes = self._nodes
        readers = [0] * len(nodes)
        for n in nodes:
            if isinstance(n, ComputeNode):
                for a in n.args:
                    if isinstance(a, ComputeNode.D):
                        readers[a.index] += 1
        for o in self._outputs:
            readers[o] += 1
        fused_into = {}  # index of the ReLU node -> index of its BatchNorm
        for j, n in enumerate(nodes):
            if isinstance(n, ComputeNode) and n.op in ("aten::relu", "aten::relu_"):
                src = [a.index for a in n.args if isinstance(a, ComputeNode.D)]
                if len(src) == 1 and isinstance(nodes[src[0]], ComputeNode) and \
                        nodes[src[0]].op in _FUSABLE and readers[src[0]] == 1 and \
                        self._add_is_fusable(nodes[src[0]]):
                    fused_into[j] = src[0]
        g = Graph()
        new_index = {}
        for k, n in enumerate(nodes):
            if k in fused_into:
                new_index[k] = new_index[fused_into[k]]
                continue
            if isinstance(n, ComputeNode):
                args = [ComputeNode.D(new_index[a.index], a.requires_grad)
                        if isinstance(a, ComputeNode.D) else a for a in n.args]
                op = _FUSABLE[n.op] if k in fused_into.values() else n.op
                new_index[k] = g._add(ComputeNode(n.shape, len(g._nodes), op, args, n.has_backward,
                                                  n.is_depthwise))
            else:
                new_index[k] = g._add(n)
        g._outputs = [new_index[o] for o in self._outputs]
        return g

    def fuse_batch_norm_add_relu(self):
        """Second fusion level, on a graph that went through `fuse_batch_norm_relu`: a fused
        add + ReLU whose FIRST operand is a plain BatchNorm that nothing else reads (the end of
        a residual block) becomes one `monet::batch_norm_add_relu` node with the BatchNorm's
        arguments followed by the add's other operand and factor.  The node takes the add's
        place in the order (the other operand may be computed after the BatchNorm's input)."""
        nodes = self._nodes
        readers = [0] * len(nodes)
        for n in nodes:
            if isinstance(n, ComputeNode):
                for a in n.args:
                    if isinstance(a, ComputeNode.D):
                        readers[a.index] += 1
        for o in self._outputs:
            readers[o] += 1
        absorbed = {}  # index of the add+ReLU node -> index of the BatchNorm it absorbs
        for j, n in enumerate(nodes):
            if not (isinstance(n, ComputeNode) and n.op == FUSED_ADD_RELU):
                continue
            first = n.args[0]
            if not isinstance(first, ComputeNode.D) or readers[first.index] != 1:
                continue
            bn = nodes[first.index]
            if isinstance(bn, ComputeNode) and bn.op == "aten::batch_norm" and \
                    list(bn.shape) == list(n.shape) and len(n.args) == 3 and \
                    isinstance(n.args[2], ComputeNode.V):
                absorbed[j] = first.index
        gone = set(absorbed.values())
        g = Graph()
        new_index = {}

        def moved(a):
            return ComputeNode.D(new_index[a.index], a.requires_grad) \
                if isinstance(a, ComputeNode.D) else a

        for k, n in enumerate(nodes):
            if k in gone:
                continue
            if k in absorbed:
                bn = nodes[absorbed[k]]
                args = [moved(a) for a in bn.args] + [moved(a) for a in n.args[1:]]
                new_index[k] = g._add(ComputeNode(n.shape, len(g._nodes), FUSED_BN_ADD_RELU, args,
                                                  n.has_backward))
            elif isinstance(n, ComputeNode):
                new_index[k] = g._add(ComputeNode(n.shape, len(g._nodes), n.op,
                                                  [moved(a) for a in n.args], n.has_backward,
                                                  n.is_depthwise))
            else:
                new_index[k] = g._add(n)
        g._outputs = [new_index[o] for o in self._outputs]
        return g

    def _add_is_fusable(self, n):
        """An add fuses only if both operands are activations of the output's shape (no
        broadcasting, no parameter operand)."""
        if n.op == "aten::batch_norm":
            return True
        ops = [a for a in n.args if isinstance(a, ComputeNode.D)]
        return len(ops) == 2 and all(isinstance(self._nodes[a.index], ComputeNode) and
                                     list(self._nodes[a.index].shape) == list(n.shape) for a in ops)

    @classmethod
    def create(cls, model, input_shape=(3, 224, 224), fuse_bn_relu=False):
        """`fuse_bn_relu`: 0 / False = the operators as traced; 1 / True = BatchNorm + ReLU and
        add + ReLU pairs as single nodes; 2 = also BatchNorm + add + ReLU triples."""
        g = cls._trace(model, input_shape)
        if fuse_bn_relu:
            g = g.fuse_batch_norm_relu()
            if int(fuse_bn_relu) >= 2:
                g = g.fuse_batch_norm_add_relu()
        return g

    @classmethod
    def _trace(cls, model, input_shape):
        example = (torch.ones((TRACE_BATCH,) + tuple(input_shape)),)
        trace, _ = torch.jit._get_trace_graph(model, example, _force_outplace=False,
                                              _return_inputs_states=False)
        torch._C._jit_pass_constant_propagation(trace)
        torch._C._jit_pass_inline(trace)
        torch._C._jit_pass_dce(trace)
        torch._C._jit_pass_lint(trace)
        params = torch.jit._unique_state_dict(model)
        graph_inputs = list(trace.inputs())
        assert len(graph_inputs) == len(example) + len(params)

        g = cls()
        node_of = {}  # trace value id -> graph node index
        shapes = [list(a.shape) for a in example] + [list(p.shape) for p in params.values()]
        for k, value in enumerate(graph_inputs):
            if k < len(example):
                node_of[value.unique()] = g._add(Input([-1] + shapes[k][1:]))
            else:
                node_of[value.unique()] = g._add(Param(shapes[k]))

        # values that depend on the data input
        tracked = {graph_inputs[k].unique() for k in range(len(example))}
        for n in trace.nodes():
            if n.kind() != "aten::size" and any(i.unique() in tracked for i in n.inputs()):
                for o in n.outputs():
                    tracked.add(o.unique())

        const, lists = {}, {}
        for n in trace.nodes():
            kind = n.kind()
            assert kind != 'prim::GetAttr'
            if kind == 'prim::Constant':
                const[n.output().unique()] = n.output().toIValue()
            elif kind in ('prim::ListConstruct', 'prim::TupleConstruct'):
                lists[n.output().unique()] = [i.unique() for i in n.inputs()]
            elif kind.startswith('aten::'):
                out = n.output()
                connected = out.unique() in tracked
                if not connected and len(out.uses()) == 0:
                    continue  # side effect on a buffer (e.g. num_batches_tracked += 1)
                args = []
                for i in n.inputs():
                    for iu in lists.get(i.unique(), [i.unique()]):
                        if iu in const:
                            args.append(ComputeNode.V(const[iu]))
                        elif iu in node_of:
                            src = g._nodes[node_of[iu]]
                            if iu not in tracked and isinstance(src, ComputeNode):
                                # a parameter reshaped before use (e.g. weight.t() for addmm):
                                # refer to the parameter itself
                                for ii in i.node().inputs():
                                    assert isinstance(g._nodes[node_of[ii.unique()]], (Input, Param))
                                    args.append(ComputeNode.D(node_of[ii.unique()],
                                                              ii.requires_grad()))
                            else:
                                grad = True if isinstance(src, ComputeNode) and iu in tracked \
                                    else bool(i.requires_grad())
                                args.append(ComputeNode.D(node_of[iu], grad))
                        else:
                            raise ValueError('Nodes %s disconnected' % repr(i))
                is_depthwise = False
                if kind == "aten::_convolution":
                    assert isinstance(args[8], ComputeNode.V)
                    groups = args[8].value
                    is_depthwise = groups > 1 and groups == g._nodes[args[0].index].shape[1]
                shape = [s if s != TRACE_BATCH else -1 for s in out.type().sizes()]
                nodeid = len(g._nodes)
                node_of[out.unique()] = g._add(
                    ComputeNode(shape, nodeid, kind, args, connected, is_depthwise))
            else:
                print('Unknown OP', kind, n)

        for o in trace.outputs():
            if o.node().kind().startswith('aten::'):
                g._outputs.append(node_of[o.unique()])
            elif o.node().kind() == 'prim::TupleConstruct':
                for i in o.node().inputs():
                    g._outputs.append(node_of[i.unique()])
        return g
