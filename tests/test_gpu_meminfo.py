"""Workspace / run-time accounting on the GPU: what the profiler reports for an operator must
be what its kernels really allocate, because the schedule solver budgets with these numbers."""
import ctypes

import pytest
import torch
import torch.nn as nn

pytestmark = pytest.mark.gpu


def _conv_graph(cin, cout, k, stride, pad, hw):
    from monet_amd.graph import ComputeNode, Graph
    net = nn.Sequential(nn.Conv2d(cin, cin, 1, bias=False), nn.Conv2d(cin, cout, k, stride, pad, bias=False))
    g = Graph.create(net, (cin, hw, hw))
    node = [n for n in g.nodes if isinstance(n, ComputeNode)][1]
    return net, g, node


def test_conv_workspace_is_what_the_library_asks_for(cuda):
    from monet_amd import _lib, lm_ops
    from monet_amd.lm_ops.conv import conv_geometry
    from monet_amd.meminfo import computeinfo, meminfo
    bs, cin, cout, hw = 32, 64, 128, 28
    net, g, node = _conv_graph(cin, cout, 3, 1, 1, hw)
    net.to(cuda)
    params = [None] + list(net.state_dict(keep_vars=True).values())
    op_cls = lm_ops.list_ops("conv_multiway_newnode", "aten::_convolution")[0]
    geo = conv_geometry((bs, cin, hw, hw), (cout, cin, 3, 3), 1, 1, 1, 1)

    def asked(direction, variant, geo=geo):
        n = ctypes.c_size_t(0)
        try:
            _lib.call("mn_conv_ws_bytes", geo, direction, variant, _lib.F32, ctypes.byref(n))
        except _lib.MonetHipError as e:
            if e.status != _lib.MN_EUNSUPPORTED:
                raise
            # a variant that does not take the shape (the three-slice one on a 3x3 filter): the
            # operator runs variant 0 in its place
            return asked(direction, 0, geo)
        return n.value

    for bwd_op, direction, count in (("param_grad", _lib.CONV_BWD_WEIGHT, op_cls.n_bwd_wt_algos()),
                                     ("ip_grad", _lib.CONV_BWD_DATA, op_cls.n_bwd_ip_algos())):
        fmem, bmem, _ = meminfo(node, op_cls(), g, bs, bwd_op, True, False, *params)
        assert len(fmem) == op_cls.n_fwd_algos() and len(bmem) == count
        for v in range(op_cls.n_fwd_algos()):
            want = asked(_lib.CONV_FWD, v)
            assert abs(fmem[v] * 2**20 - want) <= 1024, ("forward", v, fmem[v] * 2**20, want)
        for v in range(count):
            want = asked(direction, v)
            # the backward frees its stored inputs as it goes; it never holds more than the
            # workspace beyond its outputs
            assert bmem[v] * 2**20 <= want + 1024, (bwd_op, v, bmem[v] * 2**20, want)
        ftime, btime, _ = computeinfo(node, op_cls(), g, bs, bwd_op, True, False, *params)
        assert len(ftime) == op_cls.n_fwd_algos() and len(btime) == count
        # (a variant that refuses the shape - the three-slice one here - records -1 s, as
        # monet/meminfo.py:52-55 does for a failing cuDNN algorithm)
        assert all(0 < t < 50 or t == -1000 for t in list(ftime) + list(btime))
        assert all(0 < t < 50 for t in list(ftime)[:4] + list(btime)[:3])
    # the repacked-weight variants ask for the padded weight size, variant 0 for nothing
    assert asked(_lib.CONV_FWD, 0) == 0 and asked(_lib.CONV_BWD_DATA, 0) == 0
    assert asked(_lib.CONV_FWD, 1) == 9 * cin * 128 * 4
    assert asked(_lib.CONV_BWD_DATA, 1) == 9 * cout * 128 * 4
    # the three-slice variant of a 1x1 convolution: three bf16 copies of the weights, output
    # channels padded to 256
    one = conv_geometry((bs, cin, hw, hw), (cout, cin, 1, 1), 1, 0, 1, 1)
    assert asked(_lib.CONV_FWD, 4, one) == 3 * 256 * cin * 2
    assert asked(_lib.CONV_BWD_DATA, 4, one) == 3 * 256 * cout * 2


def test_intermediate_sizes_match_the_tensors_the_ops_return(cuda):
    from monet_amd import lm_ops
    x = torch.randn(8, 16, 30, 30, device=cuda)
    relu = lm_ops.list_ops("multiway_newnode", "aten::relu")[2]()
    y, mask = relu.forward(x)
    assert mask.numel() * mask.element_size() == relu.backward_storage.size(list(x.shape))
    pool = lm_ops.list_ops("multiway_newnode", "aten::max_pool2d")[1]()
    out, idx = pool.forward(x, [3, 3], [2, 2], [1, 1], [1, 1], False)
    assert idx.numel() * idx.element_size() == pool.backward_storage.size(list(out.shape))
