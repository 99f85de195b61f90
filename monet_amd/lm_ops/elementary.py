"""Shape / elementwise glue operators that simply defer to PyTorch and keep
the autograd node of their own forward for the backward (reference:
monet/lm_ops/elementary.py:5-94).  No custom kernels here."""
import torch

from .base import OP, implements

_ALL = ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode', 'conv_normal']


class NativeOP(OP):
    """Runs `op` under autograd and replays its grad_fn in the backward.

    The executor recognises this class: the instance that ran the forward is
    the one whose `backward` must be called, because it owns `grad_fn`.
    """
    op = None
    grad_fn = None
    backward_storage = None

    def forward(self, input_, *args, **kwargs):
        with torch.enable_grad():
            r = self.op(input_.detach().requires_grad_(True), *args, **kwargs)
        assert r.grad_fn is not None
        self.grad_fn = r.grad_fn
        return r.detach()

    def backward(self, grad_output, stored, nodel=False):
        assert len(stored) == 0
        return self.grad_fn(grad_output)


def _native(names, fn):
    def deco(cls):
        cls.op = staticmethod(fn)
        return implements(names, _ALL)(cls)
    return deco


@_native(['aten::flatten'], lambda x, start_dim, end_dim: x.flatten(start_dim, end_dim))
class Flatten(NativeOP):
    pass


@_native(['aten::permute'], lambda x, order: x.permute(order))
class Permute(NativeOP):
    pass


@_native(['aten::transpose'], lambda x, d0, d1: torch.transpose(x, d0, d1))
class Transpose(NativeOP):
    pass


@_native(['aten::view'], lambda x, dims: x.view(dims))
class View(NativeOP):
    pass


@_native(['aten::div'], lambda x, divisor: torch.div(x, divisor))
class Div(NativeOP):
    pass


def _contiguous(x, memory_format):
    assert memory_format == 0
    return x.contiguous()


@_native(['aten::contiguous'], _contiguous)
class Contiguous(NativeOP):
    pass


@_native(['aten::mul'], lambda x, alpha: x * alpha)
class Mul(NativeOP):
    pass


@_native(['aten::t'], lambda x: x.t())
class T(NativeOP):
    pass


def _avg_pool2d(x, kernel_size, stride, padding, ceil_mode, count_include_pad, *rest):
    assert ceil_mode in (0, 1) and count_include_pad in (0, 1)
    return torch._C._nn.avg_pool2d(x, kernel_size, stride, padding, bool(ceil_mode),
                                   bool(count_include_pad), *rest)


@_native(['aten::avg_pool2d'], _avg_pool2d)
class AvgPool2D(NativeOP):
    pass


@_native(['aten::dropout'],
         lambda x, p, training=False: torch.nn.functional.dropout(x, p, bool(training)))
class Dropout(NativeOP):
    pass


@implements(['aten::unsqueeze'], _ALL)
class Unsqueeze(OP):
    def forward(self, x, dim):
        assert not x.requires_grad
        return torch.unsqueeze(x, dim)
