"""ReLU operator implementations (reference: monet/lm_ops/relu.py).

Three ways to keep what the backward needs, in the reference's registration
order for `aten::relu` / `aten::relu_`:
  InputActReLU   keeps the input            (relu.py:9-29)
  OutputActReLU  keeps the output           (relu.py:32-52)
  BinaryActReLU  keeps a 1-bit sign mask    (relu.py:94-118)
The backward of the first two is one in-place pass over the gradient; the
mask variant fuses clamp + compare + pack in the forward and unpack +
multiply in the backward into one kernel each.
"""
import torch

from .. import _lib
from .base import OP, InputStorage, IntermediateStorage, OutputStorage, implements


def _numel(shape):
    n = 1
    for d in shape:
        n *= d
    return n


def _f32_contig(t, name):
    _lib.require_gpu_tensor(t, name, torch.float32)
    return t if t.is_contiguous() else t.contiguous()


def relu_backward_from_ref(grad, ref):
    """grad <- ref > 0 ? grad : 0, in place on `grad` when it is contiguous."""
    g = _f32_contig(grad, "grad")
    r = _f32_contig(ref, "ref")
    if g.numel() != r.numel():
        raise RuntimeError("gradient and stored activation differ in size")
    _lib.call("mn_relu_bwd_ref_f32", _lib.ptr(g), _lib.ptr(r), 0.0, _lib.ptr(g), g.numel(),
              _lib.stream_ptr(g.device))
    return g.view(ref.shape)


def relu_forward_with_mask(x, inplace=False, want_output=True):
    """(relu(x) or None, packed mask of x > 0) in one pass over x."""
    xc = _f32_contig(x, "x")
    n = xc.numel()
    mask = torch.empty((n + 7) // 8, dtype=torch.uint8, device=x.device)
    if not want_output:
        y = None
    elif inplace and xc is x:
        y = x
    else:
        y = torch.empty_like(xc)
    _lib.call("mn_relu_fwd_mask_f32", _lib.ptr(xc), _lib.ptr(y), _lib.ptr(mask), n,
              _lib.stream_ptr(x.device))
    if y is not None and inplace and xc is not x:
        x.copy_(y)
        y = x
    return y, mask


def relu_backward_from_mask(grad, mask):
    """grad <- grad * bit, in place on `grad` when it is contiguous."""
    g = _f32_contig(grad, "grad")
    _lib.require_gpu_tensor(mask, "mask", torch.uint8)
    if mask.numel() * 8 < g.numel():
        raise RuntimeError("mask is too short for the gradient")
    _lib.call("mn_relu_bwd_mask_f32", _lib.ptr(g), _lib.ptr(mask), _lib.ptr(g), g.numel(),
              _lib.stream_ptr(g.device))
    return g


@implements(['aten::relu', 'aten::relu_'],
            ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode'])
class InputActReLU(OP):
    overwrites_grad = True
    backward_storage = InputStorage(0)
    params = None
    inplace = False

    def forward(self, x):
        with torch.no_grad():
            return torch.relu_(x) if self.inplace else torch.relu(x)

    def backward(self, grad, stored, nodel=False):
        with torch.no_grad():
            ip = stored[0]
            if not nodel:
                del stored[0]
            return relu_backward_from_ref(grad, ip)


@implements(['aten::relu', 'aten::relu_'],
            ['multiway', 'multiway_newnode', 'conv_multiway_newnode', 'conv_normal'])
class OutputActReLU(OP):
    overwrites_grad = True
    backward_storage = OutputStorage()
    params = None
    inplace = False

    def forward(self, x):
        with torch.no_grad():
            return torch.relu_(x) if self.inplace else torch.relu(x)

    def backward(self, grad, stored, nodel=False):
        with torch.no_grad():
            op = stored[0]
            if not nodel:
                del stored[0]
            return relu_backward_from_ref(grad, op)


@implements(['aten::relu', 'aten::relu_'], ['newnode', 'multiway_newnode', 'conv_multiway_newnode'])
class BinaryActReLU(OP):
    overwrites_grad = True
    # mask bytes for an output of `shape`
    backward_storage = IntermediateStorage(lambda shape: (_numel(shape) + 7) // 8)
    params = None
    inplace = False

    def forward(self, x):
        with torch.no_grad():
            return relu_forward_with_mask(x, inplace=self.inplace)

    def intermediate(self, x):
        with torch.no_grad():
            return relu_forward_with_mask(x, want_output=False)[1]

    def backward(self, grad, stored, nodel=False):
        with torch.no_grad():
            mask = stored[0]
            if not nodel:
                del stored[0]
            return relu_backward_from_mask(grad, mask)
