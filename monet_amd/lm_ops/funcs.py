"""Residual add and adaptive average pooling (reference:
monet/lm_ops/funcs.py:7-59).  Bandwidth-bound but stock: they call PyTorch."""
import torch

from .. import _lib
from .base import OP, IntermediateStorage, OutputStorage, implements
from .relu import _f32_contig, _numel, relu_backward_from_mask, relu_backward_from_ref

_ALL = ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode', 'conv_normal']


@implements(['aten::adaptive_avg_pool2d'], _ALL)
class AdaptiveAvgPool2D(OP):
    params = None

    def forward(self, x, output_size):
        with torch.no_grad():
            self.params = x.shape, x.device, x.dtype
            if self._replicates(x.shape, output_size):
                # an output that is a whole multiple of the input averages windows of one
                # element (the reference's UNet upsamples this way, unet_parts.py:45-56):
                # nearest-neighbour replication, the same values from a plain copy kernel
                return torch.ops.aten.upsample_nearest2d(x, [int(output_size[0]), int(output_size[1])])
            return torch._C._nn.adaptive_avg_pool2d(x, output_size)

    @staticmethod
    def _is_global(grad_shape):
        return len(grad_shape) == 4 and grad_shape[2] == 1 and grad_shape[3] == 1

    @staticmethod
    def _replicates(in_shape, out_size):
        if len(in_shape) != 4 or out_size is None or len(out_size) != 2:
            return False
        if out_size[0] is None or out_size[1] is None:
            return False
        h, w, oh, ow = int(in_shape[2]), int(in_shape[3]), int(out_size[0]), int(out_size[1])
        if h <= 0 or w <= 0 or oh % h or ow % w or (oh == h and ow == w):
            return False
        # powers of two only: the copy kernel finds its source as floor(i * (h / oh)) in
        # single precision, which is exact for these factors
        fh, fw = oh // h, ow // w
        return fh & (fh - 1) == 0 and fw & (fw - 1) == 0

    def backward(self, grad_output, stored, nodel=False):
        assert len(stored) == 0
        with torch.no_grad():
            shape, device, dtype = self.params
            if self._is_global(grad_output.shape) and len(shape) == 4:
                # global average: every position of a plane gets grad / (H*W); one streaming
                # write instead of the atomic scatter of the generic backward
                return (grad_output * (1.0 / (shape[2] * shape[3]))).expand(shape).contiguous()
            if len(shape) == 4 and self._replicates(shape, grad_output.shape[2:]):
                # replication forward: every input element collects its fh x fw copies, a
                # gather without the atomic scatter of the generic backward
                return torch.ops.aten.upsample_nearest2d_backward(
                    grad_output.contiguous(), [int(grad_output.shape[2]), int(grad_output.shape[3])],
                    [int(d) for d in shape])
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


FUSED_ADD_RELU = 'monet::add_relu'


def add_relu_forward(a, b, alpha, inplace=False, want_mask=False):
    """(max(a + alpha*b, 0), packed mask of a + alpha*b > 0 or None) in one pass; writes into
    `a` when `inplace`."""
    ac, bc = _f32_contig(a, "a"), _f32_contig(b, "b")
    if ac.shape != bc.shape:
        raise RuntimeError("the fused add needs operands of one shape")
    n = ac.numel()
    y = ac if (inplace and ac is a) else torch.empty_like(ac)
    mask = torch.empty((n + 7) // 8, dtype=torch.uint8, device=a.device) if want_mask else None
    _lib.call("mn_add_relu_fwd_f32", _lib.ptr(ac), _lib.ptr(bc), float(alpha), _lib.ptr(y),
              _lib.ptr(mask), n, _lib.stream_ptr(a.device))
    if inplace and ac is not a:
        a.copy_(y)
        y = a
    return y, mask


class _AddReLUBase(OP):
    """The residual add and the ReLU behind it as ONE operator (`monet::add_relu` nodes come
    from the tracer's optional fusion pass; arguments are those of aten::add_: a, b, alpha).
    Both inputs receive the ReLU-masked gradient (b's scaled by alpha)."""
    params = None
    inplace = False
    overwrites_grad = True

    def _split(self, g):
        s = self.params
        return g, (g if s == 1 else g * s)


@implements([FUSED_ADD_RELU],
            ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode',
             'conv_normal'])
class OutputActAddReLU(_AddReLUBase):
    backward_storage = OutputStorage()

    def forward(self, a, b, s):
        with torch.no_grad():
            self.params = s
            return add_relu_forward(a, b, s, inplace=self.inplace)[0]

    def backward(self, grad, stored, nodel=False):
        with torch.no_grad():
            out = stored[0]
            if not nodel:
                del stored[0]
            return self._split(relu_backward_from_ref(grad, out))


@implements([FUSED_ADD_RELU], ['newnode', 'multiway_newnode', 'conv_multiway_newnode'])
class BinaryActAddReLU(_AddReLUBase):
    backward_storage = IntermediateStorage(lambda shape: (_numel(shape) + 7) // 8)

    def forward(self, a, b, s):
        with torch.no_grad():
            self.params = s
            return add_relu_forward(a, b, s, inplace=self.inplace, want_mask=True)

    def backward(self, grad, stored, nodel=False):
        with torch.no_grad():
            mask = stored[0]
            if not nodel:
                del stored[0]
            return self._split(relu_backward_from_mask(grad, mask))
