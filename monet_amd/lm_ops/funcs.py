"""Residual add and adaptive average pooling (reference:
monet/lm_ops/funcs.py:7-59).  Bandwidth-bound but stock: they call PyTorch."""
import torch

from .base import OP, implements

_ALL = ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode', 'conv_normal']


@implements(['aten::adaptive_avg_pool2d'], _ALL)
class AdaptiveAvgPool2D(OP):
    params = None

    def forward(self, x, output_size):
        with torch.no_grad():
            self.params = x.shape, x.device, x.dtype
            return torch._C._nn.adaptive_avg_pool2d(x, output_size)

    @staticmethod
    def _is_global(grad_shape):
        return len(grad_shape) == 4 and grad_shape[2] == 1 and grad_shape[3] == 1

    def backward(self, grad_output, stored, nodel=False):
        assert len(stored) == 0
        with torch.no_grad():
            shape, device, dtype = self.params
            if self._is_global(grad_output.shape) and len(shape) == 4:
                # global average: every position of a plane gets grad / (H*W); one streaming
                # write instead of the atomic scatter of the generic backward
                return (grad_output * (1.0 / (shape[2] * shape[3]))).expand(shape).contiguous()
            # the aten backward only reads the shape of its second argument
            like = torch.empty(1, dtype=dtype, device=device).expand(list(shape))
            return torch.ops.aten._adaptive_avg_pool2d_backward(grad_output.contiguous(), like)


class _AddBase(OP):
    backward_storage = None
    params = None

    def backward(self, grad_output, stored, nodel=False):
        assert len(stored) == 0
        with torch.no_grad():
            s = self.params
            return grad_output, (grad_output if s == 1 else grad_output * s)


@implements(['aten::add'], _ALL)
class Add(_AddBase):
    def forward(self, a, b, s):
        with torch.no_grad():
            self.params = s
            return torch.add(a, b, alpha=s)


@implements(['aten::add_'], _ALL)
class AddIP(_AddBase):
    inplace = False

    def forward(self, a, b, s):
        with torch.no_grad():
            self.params = s
            if self.inplace:
                return a.add_(b, alpha=s)
            return torch.add(a, b, alpha=s)
