"""Host-side logic of the operator library that needs no GPU: the registry,
storage descriptors and the accounting sizes the solver reads."""
import pytest
import torch

import monet_amd.lm_ops as lm_ops
from monet_amd.lm_ops import InputStorage, IntermediateStorage, OutputStorage


def names(mode, op):
    return [c.__name__ for c in lm_ops.list_ops(mode, op)]


def test_registration_order_is_the_implementation_index():
    m = "conv_multiway_newnode"
    assert names(m, "aten::relu") == ["InputActReLU", "OutputActReLU", "BinaryActReLU"]
    assert names(m, "aten::relu_") == ["InputActReLU", "OutputActReLU", "BinaryActReLU"]
    assert names(m, "aten::batch_norm") == ["InputActBatchNorm", "OutputActBatchNorm"]
    assert names(m, "aten::max_pool2d") == ["SimpleMaxPool2D", "IndicesActMaxPool2D"]
    assert names("normal", "aten::relu") == ["InputActReLU"]
    assert names("conv_normal", "aten::relu") == ["OutputActReLU"]
    assert names("multiway", "aten::relu") == ["InputActReLU", "OutputActReLU"]
    assert names("newnode", "aten::relu") == ["InputActReLU", "BinaryActReLU"]
    assert names("newnode", "aten::max_pool2d") == ["SimpleMaxPool2D", "IndicesActMaxPool2D"]
    assert names("normal", "aten::batch_norm") == ["InputActBatchNorm"]
    for mode in ["normal", "multiway", "newnode", "multiway_newnode", "conv_multiway_newnode",
                 "conv_normal"]:
        for op in ["aten::add", "aten::add_", "aten::adaptive_avg_pool2d", "aten::flatten",
                   "aten::cat", "aten::t", "aten::addmm", "aten::linear", "aten::softmax"]:
            assert len(lm_ops.list_ops(mode, op)) == 1, (mode, op)
    # no op offers more implementations than the solver has slots for
    assert max(len(v) for by in lm_ops.registry.values() for v in by.values()) <= 3


def test_storage_descriptors():
    assert lm_ops.relu.InputActReLU.backward_storage.ids == (0,)
    assert isinstance(lm_ops.relu.OutputActReLU.backward_storage, OutputStorage)
    assert isinstance(lm_ops.relu.BinaryActReLU.backward_storage, IntermediateStorage)
    bs = lm_ops.bn.OutputActBatchNorm.backward_storage
    assert isinstance(bs, list) and bs[0].ids == (1, 2, 3, 4) and isinstance(bs[1], OutputStorage)
    assert lm_ops.bn.InputActBatchNorm.backward_storage.ids == (0, 1, 2, 3, 4)
    assert lm_ops.pool.SimpleMaxPool2D.backward_storage.ids == (0,)
    assert lm_ops.linear.LowMemAddMM.backward_storage.ids == (1, 2)


def test_intermediate_sizes_match_the_packed_formats():
    relu_size = lm_ops.relu.BinaryActReLU.backward_storage.size
    pool_size = lm_ops.pool.IndicesActMaxPool2D.backward_storage.size
    assert relu_size([184, 256, 56, 56]) == 18464768
    assert relu_size([3, 3]) == 2
    assert pool_size([184, 64, 56, 56]) == 18464768
    assert pool_size([1, 1, 3, 3]) == 5
    # the solver evaluates sizes on a per-sample shape with batch -1 and later multiplies by
    # -batch; floor division of the negative count must round away from zero
    assert -184 * relu_size([-1, 256, 56, 56]) >= 18464768
    assert -184 * pool_size([-1, 64, 56, 56]) >= 18464768


def test_ops_refuse_cpu_tensors():
    from monet_amd.lm_ops import pack
    with pytest.raises(RuntimeError, match="GPU tensor"):
        pack.pack(torch.zeros(8, dtype=torch.bool))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        lm_ops.relu.BinaryActReLU().forward(torch.zeros(8))
    with pytest.raises(RuntimeError, match="GPU tensor"):
        lm_ops.relu.InputActReLU().backward(torch.zeros(8), [torch.zeros(8)])
    with pytest.raises(RuntimeError, match="GPU tensor"):
        lm_ops.pool.IndicesActMaxPool2D().forward(torch.zeros(1, 1, 4, 4), 2, 2, 0, 1, False)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        lm_ops.bn.bn_forward_train(torch.zeros(2, 2, 2, 2), None, None, None, None, 0.1, 1e-5)


def test_adaptive_avg_pool_replication_path_equals_the_pooling_operator():
    """Outputs that are a power-of-two multiple of the input (the reference UNet's upsampling,
    unet_parts.py:45-56) take a copy / gather path; values and gradients must equal those of
    aten's adaptive pooling, and other sizes must keep using it."""
    torch.manual_seed(0)
    rep = lm_ops.funcs.AdaptiveAvgPool2D._replicates
    assert rep((1, 2, 26, 38), (52, 76)) and rep((1, 2, 3, 4), (12, 4))
    assert not rep((1, 2, 5, 7), (15, 21))      # factor 3: not exact in single precision
    assert not rep((1, 2, 6, 6), (4, 9)) and not rep((1, 2, 6, 6), (6, 6)) and not rep((1, 2, 6, 6), (1, 1))
    for in_hw, out_hw in (((5, 7), (10, 14)), ((3, 4), (12, 4)), ((5, 7), (15, 21)), ((6, 6), (4, 9))):
        x = torch.randn(2, 3, *in_hw, dtype=torch.float64)
        op = lm_ops.funcs.AdaptiveAvgPool2D()
        y = op.forward(x, list(out_hw))
        xr = x.clone().requires_grad_(True)
        ref = torch.nn.functional.adaptive_avg_pool2d(xr, list(out_hw))
        assert torch.equal(y, ref.detach())
        g = torch.randn_like(y)
        ref.backward(g)
        torch.testing.assert_close(op.backward(g, []), xr.grad, rtol=1e-12, atol=1e-12)
