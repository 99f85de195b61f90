"""Fully connected layer (reference: monet/lm_ops/linear.py:25-62).

The backward is split like the convolution's: `algorithm // 10` selects
0 -> parameter gradients (dw, db), 1 -> input gradient, 2 -> both, so the
executor can run them in two timesteps and drop the input in between.
`aten::addmm(bias, input, weight^T)` is what old tracers emit for nn.Linear;
current ones emit `aten::linear(input, weight, bias)`; both are registered.
"""
import torch

from .base import OP, InputStorage, implements

_ALL = ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode', 'conv_normal']


def _linear_backward(kind, grad, input_, weight, need):
    di = dw = db = None
    g2 = grad.reshape(-1, grad.shape[-1])
    if kind in (0, 2) and input_ is not None:
        if need[1]:
            dw = g2.t().mm(input_.reshape(-1, input_.shape[-1]))
        if need[2]:
            db = g2.sum(0)
    if kind in (1, 2) and weight is not None and need[0]:
        di = grad.matmul(weight)
    return di, dw, db


@implements(['aten::addmm'], _ALL)
class LowMemAddMM(OP):
    backward_storage = InputStorage(1, 2)
    params = None
    algorithm = -1

    def forward(self, bias, input_, weight, beta, alpha):
        self.params = [input_.requires_grad, weight.requires_grad,
                       bias is not None and bias.requires_grad]
        assert alpha == 1 and beta == 1
        with torch.no_grad():
            return torch.addmm(bias, input_, weight.t(), beta=beta, alpha=alpha)

    def backward(self, output_grad, stores, nodel=False):
        with torch.no_grad():
            input_, weight = stores[0], stores[1]
            if not nodel:
                del stores[1]
                del stores[0]
            di, dw, db = _linear_backward(self.algorithm // 10, output_grad, input_, weight,
                                          self.params)
            return db, di, dw


@implements(['aten::linear'], _ALL)
class LowMemLinear(OP):
    backward_storage = InputStorage(0, 1)
    params = None
    algorithm = -1

    def forward(self, input_, weight, bias=None):
        self.params = [input_.requires_grad, weight.requires_grad,
                       bias is not None and bias.requires_grad, bias is not None]
        with torch.no_grad():
            return torch.nn.functional.linear(input_, weight, bias)

    def backward(self, output_grad, stores, nodel=False):
        with torch.no_grad():
            input_, weight = stores[0], stores[1]
            if not nodel:
                del stores[1]
                del stores[0]
            di, dw, db = _linear_backward(self.algorithm // 10, output_grad, input_, weight,
                                          self.params)
            if self.params[3]:  # bias present: one gradient per tensor argument of the forward
                return di, dw, db
            return di, dw
