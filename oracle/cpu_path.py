"""The stock PyTorch CPU operators that the reference's operator library
delegates its arithmetic to (F.batch_norm, relu, max_pool2d and their autograd
backward): the "reference CPU path" for the bandwidth-bound operators.

TEST INFRASTRUCTURE ONLY: used as a second checker in tests and as the timed
CPU baseline of bench.py; the product never imports it.  The reference's
low-memory operators have no CPU implementation of their own
(examples/imagenet.py:150-151 asserts a GPU), so these library routines - the
same ones tests/test_oracle.py pins oracle/lm_oracle.py against - stand in.
"""
import torch
import torch.nn.functional as F


def bn_backward(dy, x, gamma, save_mean, save_invstd, eps=1e-5):
    """(dx, dgamma, dbeta) of training-mode BatchNorm on CPU tensors."""
    return torch.ops.aten.native_batch_norm_backward(
        dy, x, gamma, None, None, save_mean, save_invstd, True, eps, [True, True, True])


def bn_forward(x, gamma, beta, eps=1e-5):
    """(y, save_mean, save_invstd) of training-mode BatchNorm."""
    return torch.ops.aten.native_batch_norm(x, gamma, beta, None, None, True, 0.1, eps)


def relu_backward(dy, y):
    return torch.ops.aten.threshold_backward(dy, y, 0)


def maxpool_forward(x, k, s, p):
    return F.max_pool2d(x, k, s, p, return_indices=True)


def maxpool_backward(dy, x, k, s, p, indices):
    return torch.ops.aten.max_pool2d_with_indices_backward(
        dy, x, [k, k], [s, s], [p, p], [1, 1], False, indices)


def conv_forward(x, w, stride, pad):
    return F.conv2d(x, w, None, stride, pad)


def conv_backward(dy, x, w, stride, pad, output_mask):
    """(dx, dw, dbias) of a 2-D convolution, only the ones `output_mask` asks for."""
    return torch.ops.aten.convolution_backward(
        dy, x, w, None, [stride, stride], [pad, pad], [1, 1], False, [0, 0], 1, output_mask)


def stem_block(batch):
    """The first block of ResNet-50 (models of torchvision: 7x7/2 convolution to 64 channels,
    BatchNorm, ReLU, 3x3/2 max-pool) and a seeded batch of 3 x 224 x 224 images."""
    torch.manual_seed(0)
    block = torch.nn.Sequential(
        torch.nn.Conv2d(3, 64, 7, 2, 3, bias=False), torch.nn.BatchNorm2d(64), torch.nn.ReLU(inplace=True),
        torch.nn.MaxPool2d(3, 2, 1)).train()
    return block, torch.randn(batch, 3, 224, 224, requires_grad=True)


def stem_step(block, x):
    """One forward + backward of the stem block (gradients of the input and the parameters)."""
    block.zero_grad(set_to_none=True)
    x.grad = None
    block(x).sum().backward()
