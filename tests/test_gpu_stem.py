"""ResNet stem block (conv7x7/s2 -> BatchNorm -> ReLU -> maxpool3x3/s2) forward + backward
through the operator classes in the two storage combinations a schedule can legally pick
(configuration: N=8, 3x224x224, Kaiming-normal weights, seed 0).

Truth is stock autograd on the CPU in float64.  A float64 forward and an fp32 forward can
resolve a near-tie inside a pooling window, or a ReLU input within rounding of zero,
differently, which re-routes single gradient elements; that is a property of the precision,
not of the kernels.  So the DECISIONS (ReLU sign, pooling argmax) are taken from the GPU
forward - after checking that they agree with the float64 ones almost everywhere - and all
ARITHMETIC of the expected gradients is float64."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import monet_amd.lm_ops as lm_ops
from oracle import lm_oracle as O

pytestmark = pytest.mark.gpu


def rel(got, exp):
    exp = torch.as_tensor(exp).double()
    return float((got.double().cpu() - exp).abs().max() / exp.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("combo", ["output_act_bn+mask_relu+index_pool",
                                   "input_act_bn+inplace_relu+simple_pool"])
def test_stem_block(cuda, combo):
    torch.manual_seed(0)
    x = torch.randn(8, 3, 224, 224)
    w = torch.empty(64, 3, 7, 7)
    torch.nn.init.kaiming_normal_(w, mode='fan_out', nonlinearity='relu')
    dy = torch.randn(8, 64, 56, 56)

    # ---- float64 forward on the CPU
    x64 = x.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True)
    g64 = torch.ones(64, dtype=torch.float64, requires_grad=True)
    b64 = torch.zeros(64, dtype=torch.float64, requires_grad=True)
    rm64, rv64 = torch.zeros(64, dtype=torch.float64), torch.ones(64, dtype=torch.float64)
    c64 = F.conv2d(x64, w64, None, 2, 3)
    y64 = F.batch_norm(c64, rm64, rv64, g64, b64, True, 0.1, 1e-5)
    z64, zi64 = F.max_pool2d(F.relu(y64), 3, 2, 1, return_indices=True)

    # ---- GPU forward through the operator classes
    tx = x.to(cuda).requires_grad_(True)
    tw = w.to(cuda).requires_grad_(True)
    gamma = torch.ones(64, device=cuda, requires_grad=True)
    beta = torch.zeros(64, device=cuda, requires_grad=True)
    rm, rv = torch.zeros(64, device=cuda), torch.ones(64, device=cuda)
    conv = lm_ops.conv.SpecificAlgoConvolution()
    conv.algorithm = 0
    c = conv.forward(tx, tw, None, [2, 2], [3, 3], [1, 1], False, [0, 0], 1)
    if combo.startswith("output_act_bn"):
        bn, relu, pool = (lm_ops.bn.OutputActBatchNorm(), lm_ops.relu.BinaryActReLU(),
                          lm_ops.pool.IndicesActMaxPool2D())
        y = bn.forward(c, gamma, beta, rm, rv, True, 0.1, 1e-5)
        a, mask = relu.forward(y)
        z, idx = pool.forward(a, [3, 3], [2, 2], [1, 1], [1, 1], False)
        sign = torch.from_numpy(O.unpack_bits(mask.cpu().numpy(), a.numel())).view(a.shape)
        idx_packed = idx.cpu().numpy()
        g_a = pool.backward(dy.to(cuda), [idx])
        g_y = relu.backward(g_a, [mask])
        g_c, dg, db, _, _ = bn.backward(g_y, [gamma, beta, rm, rv, y])
    else:
        bn, relu, pool = (lm_ops.bn.InputActBatchNorm(), lm_ops.relu.OutputActReLU(),
                          lm_ops.pool.SimpleMaxPool2D())
        relu.inplace = True
        y = bn.forward(c, gamma, beta, rm, rv, True, 0.1, 1e-5)
        a = relu.forward(y)
        assert a.data_ptr() == y.data_ptr()   # BN's output is gone: only the input form is legal
        z = pool.forward(a, [3, 3], [2, 2], [1, 1], [1, 1], False)
        sign = a.cpu() > 0
        idx_packed = O.maxpool_fwd_idx(a.cpu().numpy(), 3, 2, 1)[1]
        g_a = pool.backward(dy.to(cuda), [a])
        g_y = relu.backward(g_a, [a])
        g_c, dg, db, _, _ = bn.backward(g_y, [c, gamma, beta, rm, rv])
    conv.algorithm = 20
    dx, dw = conv.backward(g_c, [tx.detach(), tw.detach()])

    # ---- forward values and decisions
    assert rel(z, z64.detach()) < 1e-5
    # the batch means are ~0.003 standard deviations of the data (100k samples per channel), so the
    # running mean is held to 1e-6 of what it is a mean OF (momentum * the data's spread) rather
    # than to 1e-5 of its own near-zero value
    spread = 0.1 * float(c64.detach().std())
    assert float((rm.double().cpu() - rm64).abs().max()) < 1e-6 * spread and rel(rv, rv64) < 1e-5
    assert float((sign != (y64.detach() > 0)).double().mean()) < 1e-5
    idx_gpu = O.unpack_nibbles(idx_packed, z64.numel()).reshape(z64.shape)
    h, wc = zi64.numpy() // 112, zi64.numpy() % 112
    ph = np.arange(56)[None, None, :, None]
    pw = np.arange(56)[None, None, None, :]
    idx_ref = (h - (2 * ph - 1)) * 3 + (wc - (2 * pw - 1))
    assert float((idx_gpu != idx_ref).mean()) < 1e-4

    # ---- expected gradients: GPU decisions, float64 arithmetic
    g_a64 = torch.from_numpy(O.maxpool_bwd_idx(dy.numpy(), idx_packed, (8, 64, 112, 112), 3, 2, 1))
    y64.backward(g_a64.double() * sign.double())
    # within 1e-5 of each tensor's scale (achieved: 1e-7 to 1e-6)
    achieved = {"dgamma": rel(dg, g64.grad), "dbeta": rel(db, b64.grad), "dw": rel(dw, w64.grad),
                "dx": rel(dx, x64.grad)}
    print("achieved stem block (%s): " % combo + ", ".join("%s %.2e" % kv for kv in achieved.items()))
    assert all(v < 1e-5 for v in achieved.values()), achieved
