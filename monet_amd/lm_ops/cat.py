"""Channel concatenation (reference: monet/lm_ops/cat.py:5-29)."""
import torch

from .base import OP, implements

_ALL = ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode', 'conv_normal']


@implements(['aten::cat'], _ALL)
class Cat(OP):
    params = None

    def forward(self, *input_):
        tensors, dim = input_[:-1], input_[-1]
        self.params = dim, [x.shape[dim] for x in tensors]
        with torch.no_grad():
            if len(tensors) == 1:
                return tensors[0]
            return torch.cat(tensors, dim=dim)

    def backward(self, *grad_output, nodel=False):
        dim, chunk_sizes = self.params
        with torch.no_grad():
            if len(chunk_sizes) == 1:
                return grad_output[0]
            return [part.contiguous() for part in torch.split(grad_output[0], chunk_sizes, dim=dim)]
