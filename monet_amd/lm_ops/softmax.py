"""Softmax operator (reference: monet/lm_ops/softmax.py:7-23) and the fused
softmax-cross-entropy gradient used by the training harness."""
import torch

from .. import _lib
from .base import OP, OutputStorage, implements


def _view3(t, dim):
    dim = dim % t.dim()
    outer = 1
    for d in t.shape[:dim]:
        outer *= d
    inner = 1
    for d in t.shape[dim + 1:]:
        inner *= d
    return outer, t.shape[dim], inner


def softmax_forward(x, dim):
    _lib.require_gpu_tensor(x, "input", torch.float32)
    xc = x if x.is_contiguous() else x.contiguous()
    y = torch.empty_like(xc)
    outer, d, inner = _view3(xc, dim)
    _lib.call("mn_softmax_fwd_f32", _lib.ptr(xc), _lib.ptr(y), outer, d, inner,
              _lib.stream_ptr(x.device))
    return y


def softmax_backward(grad, output, dim):
    _lib.require_gpu_tensor(grad, "grad_output", torch.float32)
    _lib.require_gpu_tensor(output, "output", torch.float32)
    g = grad if grad.is_contiguous() else grad.contiguous()
    y = output if output.is_contiguous() else output.contiguous()
    if g.shape != y.shape:
        raise RuntimeError("grad_output and output differ in shape")
    dx = torch.empty_like(y)
    outer, d, inner = _view3(y, dim)
    _lib.call("mn_softmax_bwd_f32", _lib.ptr(g), _lib.ptr(y), _lib.ptr(dx), outer, d, inner,
              _lib.stream_ptr(y.device))
    return dx


def cross_entropy_backward(logits, labels, scale=None):
    """d/dlogits of mean-reduced softmax cross-entropy over dim 1.

    `logits` is [N, C] or [N, C, d1, ...], `labels` int64 [N] / [N, d1, ...];
    `scale` defaults to 1 / labels.numel() (the 'mean' reduction).
    """
    _lib.require_gpu_tensor(logits, "logits", torch.float32)
    _lib.require_gpu_tensor(labels, "labels", torch.int64)
    lc = logits if logits.is_contiguous() else logits.contiguous()
    lab = labels if labels.is_contiguous() else labels.contiguous()
    outer, d, inner = _view3(lc, 1)
    if lab.numel() != outer * inner:
        raise RuntimeError("labels do not match the logits")
    if scale is None:
        scale = 1.0 / max(lab.numel(), 1)
    out = torch.empty_like(lc)
    _lib.call("mn_xent_bwd_f32", _lib.ptr(lc), _lib.ptr(lab), _lib.ptr(out), outer, d, inner,
              float(scale), _lib.stream_ptr(lc.device))
    return out


@implements(['aten::softmax'],
            ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode',
             'conv_normal'])
class Softmax(OP):
    params = None
    backward_storage = OutputStorage()

    def forward(self, input_, dim, dtype):
        with torch.no_grad():
            assert dtype is None
            self.params = input_.type(), dim
            return softmax_forward(input_, dim)

    def backward(self, grad_output, stores, nodel=False):
        with torch.no_grad():
            output = stores[0]
            if not nodel:
                del stores[0]
            _, dim = self.params
            return softmax_backward(grad_output, output, dim)
