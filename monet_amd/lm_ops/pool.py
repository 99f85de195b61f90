"""Max-pool operator implementations (reference: monet/lm_ops/pool.py).

  SimpleMaxPool2D       keeps the input and re-derives the backward from a
                        stock forward (pool.py:8-36)
  IndicesActMaxPool2D   keeps 4-bit window-relative argmax indices, two per
                        byte (pool.py:38-69); forward and backward are one
                        kernel each.
"""
import torch

from .. import _lib
from .base import OP, InputStorage, IntermediateStorage, implements


def _numel(shape):
    n = 1
    for d in shape:
        n *= d
    return n


def _pair(v, name):
    v = list(v) if isinstance(v, (list, tuple)) else [v]
    if len(v) == 1:
        v = v * 2
    if len(v) != 2:
        raise RuntimeError(f"max_pool2d: {name} must be a single int or a pair")
    return int(v[0]), int(v[1])


def pool_geometry(input_shape, kernel_size, stride, padding, dilation, ceil_mode):
    """Pool2d descriptor + output shape for a 3-D / 4-D NCHW input shape."""
    kH, kW = _pair(kernel_size, "kernel_size")
    sH, sW = (kH, kW) if stride is None or (isinstance(stride, (list, tuple)) and len(stride) == 0) \
        else _pair(stride, "stride")
    pH, pW = _pair(padding, "padding")
    dH, dW = _pair(dilation, "dilation")
    if len(input_shape) not in (3, 4):
        raise RuntimeError("non-empty 3D or 4D (batch mode) tensor expected for input")
    N = input_shape[0] if len(input_shape) == 4 else 1
    C, H, W = input_shape[-3:]
    lib = _lib.load()
    PH = lib.mn_pool_out_size(H, kH, pH, sH, dH, int(bool(ceil_mode)))
    PW = lib.mn_pool_out_size(W, kW, pW, sW, dW, int(bool(ceil_mode)))
    if PH < 1 or PW < 1:
        raise RuntimeError(f"max_pool2d: output size ({PH}x{PW}) is too small")
    if pH > kH // 2 or pW > kW // 2:
        raise RuntimeError("pad should be smaller than half of kernel size")
    geo = _lib.Pool2d(N, C, H, W, kH, kW, sH, sW, pH, pW, dH, dW, PH, PW)
    out_shape = (list(input_shape[:-2]) + [PH, PW])
    return geo, out_shape


def max_pool2d_with_packed_indices(x, kernel_size, stride, padding, dilation, ceil_mode):
    """(y, packed 4-bit indices, geometry) of a max pool over NCHW fp32 `x`."""
    _lib.require_gpu_tensor(x, "input", torch.float32)
    xc = x if x.is_contiguous() else x.contiguous()
    geo, out_shape = pool_geometry(list(x.shape), kernel_size, stride, padding, dilation, ceil_mode)
    y = torch.empty(out_shape, dtype=torch.float32, device=x.device)
    idx4 = torch.empty((y.numel() + 1) // 2, dtype=torch.uint8, device=x.device)
    _lib.call("mn_maxpool_fwd_idx_f32", geo, _lib.ptr(xc), _lib.ptr(y), _lib.ptr(idx4),
              _lib.stream_ptr(x.device))
    return y, idx4, geo


def max_pool2d_backward_from_packed_indices(grad, idx4, geo, input_shape):
    _lib.require_gpu_tensor(grad, "grad_output", torch.float32)
    _lib.require_gpu_tensor(idx4, "indices", torch.uint8)
    g = grad if grad.is_contiguous() else grad.contiguous()
    out_numel = geo.N * geo.C * geo.PH * geo.PW
    if g.numel() != out_numel or idx4.numel() != (out_numel + 1) // 2:
        raise RuntimeError("grad_output / indices do not match the pooling geometry")
    dx = torch.empty(list(input_shape), dtype=torch.float32, device=grad.device)
    _lib.call("mn_maxpool_bwd_idx_f32", geo, _lib.ptr(g), _lib.ptr(idx4), _lib.ptr(dx),
              _lib.stream_ptr(grad.device))
    return dx


@implements(['aten::max_pool2d'],
            ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode',
             'conv_normal'])
class SimpleMaxPool2D(OP):
    backward_storage = InputStorage(0)
    params = None

    def forward(self, input_, kernel_size, stride, padding, dilation, ceil_mode):
        ceil_mode = bool(ceil_mode)
        self.params = kernel_size, stride, padding, dilation, ceil_mode
        with torch.no_grad():
            return torch.max_pool2d(input_, kernel_size, stride, padding, dilation, ceil_mode)

    def backward(self, grad_output, stored, nodel=False):
        ip = stored[0]
        if not nodel:
            del stored[0]
        kernel_size, stride, padding, dilation, ceil_mode = self.params
        with torch.enable_grad():
            leaf = ip.detach().requires_grad_(True)
            tmp = torch.max_pool2d(leaf, kernel_size=kernel_size, stride=stride, padding=padding,
                                   dilation=dilation, ceil_mode=ceil_mode)
            del ip
            (out,) = torch.autograd.grad(tmp, leaf, grad_output)
        del tmp, leaf
        return out


@implements(['aten::max_pool2d'], ['newnode', 'multiway_newnode', 'conv_multiway_newnode'])
class IndicesActMaxPool2D(OP):
    # bytes of packed indices for an OUTPUT of `shape`: two indices per byte
    backward_storage = IntermediateStorage(lambda shape: (_numel(shape) + 1) // 2)
    params = None

    def forward(self, input_, kernel_size, stride, padding, dilation, ceil_mode):
        with torch.no_grad():
            y, idx4, geo = max_pool2d_with_packed_indices(input_, kernel_size, stride, padding,
                                                          dilation, ceil_mode)
            self.params = (kernel_size, stride, padding, dilation, bool(ceil_mode),
                           list(input_.shape), list(input_.stride()), input_.dim(), input_.numel(),
                           y.shape, geo)
            return y, idx4

    def backward(self, grad_output, stored, nodel=False):
        with torch.no_grad():
            idx4 = stored[0]
            if not nodel:
                del stored[0]
            input_shape, geo = self.params[5], self.params[10]
            return max_pool2d_backward_from_packed_indices(grad_output, idx4, geo, input_shape)
