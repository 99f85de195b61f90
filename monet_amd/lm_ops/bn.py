"""BatchNorm operator implementations (reference: monet/lm_ops/bn.py).

  InputActBatchNorm    backward from the stored INPUT   (bn.py:12-54)
  OutputActBatchNorm   backward from the stored OUTPUT  (bn.py:96-140), so an
                       in-place consumer chain can drop the input.

  InputActBatchNormReLU     relu(BN(x)) as one operator, from the stored input
  InputActBatchNormAddReLU  relu(BN(x) + alpha*r) as one operator (the end of a residual
                            block), from the stored input and output
(the last two only exist in graphs that went through the tracer's fusion passes).

The first three share the forward: the first forward of an iteration computes batch
statistics, updates the running statistics and records
`params = (training, eps, save_mean, save_invstd, reserve)`; a forward on an
instance whose `params` are already set is a RECOMPUTATION and re-applies the
saved statistics without touching the running ones.  The recomputation uses
the saved invstd as is, so it reproduces the first forward bit for bit
(the reference's F.batch_norm call at bn.py:32-34 adds eps a second time).
"""
import os

import torch

from .. import _lib
from .base import OP, InputStorage, IntermediateStorage, OutputStorage, implements
from .relu import _numel


def _as_nchw(t, name):
    _lib.require_gpu_tensor(t, name, torch.float32)
    if t.dim() < 2:
        raise RuntimeError("batch_norm expects at least a 2-D input")
    tc = t if t.is_contiguous() else t.contiguous()
    N, C = tc.shape[0], tc.shape[1]
    HW = tc.numel() // (N * C) if N * C else 0
    return tc, N, C, HW


def _workspace(N, C, HW, device):
    nbytes = _lib.load().mn_bn_ws_bytes(N, C, HW)
    return torch.empty(max(nbytes, 4), dtype=torch.uint8, device=device), nbytes


# True (or MONET_AMD_CHECK_BN_WAITS=1 in the environment): after every BatchNorm call that
# used a workspace, wait for it and raise if one of its workgroups gave up waiting for the
# others (the results are NaN then).  Costs a device synchronisation per call: for diagnosis.
check_waits = os.environ.get("MONET_AMD_CHECK_BN_WAITS", "0") not in ("", "0")


class _WaitMonitor:
    """Looks, without waiting for the device, whether a BatchNorm wait gave up (the results are
    NaN then): `poll` enqueues a 4-byte copy of the device's give-up word into pinned host
    memory and looks at the copy the previous poll enqueued once that has arrived, so a give-up
    raises one poll late.  One per device; the schedule executor polls once per step."""

    def __init__(self, device):
        self.device = device
        self.word = torch.zeros(1, dtype=torch.int32).pin_memory()
        self.event = None

    def poll(self):
        if self.event is not None:
            if not self.event.query():
                return      # the previous copy is still on its way
            self.event = None
            if int(self.word[0]) != 0:
                self.word.zero_()
                # the synchronous form clears the device's word (and reports it as MN_ELAUNCH)
                _lib.load().mn_bn_wait_status(None, _lib.stream_ptr(self.device))
                raise RuntimeError(
                    "a BatchNorm kernel gave up waiting for the other workgroups of its channel: "
                    "the results of that call are NaN (the device ran fewer workgroups at once "
                    "than the launch relies on)")
        _lib.call("mn_bn_wait_status", self.word.data_ptr(), _lib.stream_ptr(self.device))
        self.event = torch.cuda.Event()
        self.event.record(torch.cuda.current_stream(self.device))


_monitors = {}


def poll_waits(device):
    """See _WaitMonitor; `device` is a torch.device of type cuda."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _monitors:
        _monitors[index] = _WaitMonitor(torch.device("cuda", index))
    _monitors[index].poll()


def _ws_call(ws_shape, name, *args):
    _lib.call(name, *args)
    if check_waits:
        ws, nbytes, N, C, HW = ws_shape
        _lib.call("mn_bn_ws_status", _lib.ptr(ws), nbytes, N, C, HW, args[-1])


def bn_forward_train(x, weight, bias, running_mean, running_var, momentum, eps, out=None,
                     relu=False):
    """Training forward -> (y, save_mean, save_invstd); relu=True applies max(., 0) to y."""
    xc, N, C, HW = _as_nchw(x, "input")
    y = torch.empty_like(xc) if out is None else out
    save_mean = torch.empty(C, dtype=torch.float32, device=x.device)
    save_invstd = torch.empty(C, dtype=torch.float32, device=x.device)
    ws, nbytes = _workspace(N, C, HW, x.device)
    _ws_call((ws, nbytes, N, C, HW), "mn_bn_relu_fwd_train_f32" if relu else "mn_bn_fwd_train_f32", _lib.ptr(xc), _lib.ptr(weight), _lib.ptr(bias),
              _lib.ptr(running_mean), _lib.ptr(running_var), _lib.ptr(y), _lib.ptr(save_mean),
              _lib.ptr(save_invstd), N, C, HW, float(momentum), float(eps), _lib.ptr(ws), nbytes,
              _lib.stream_ptr(x.device))
    return y, save_mean, save_invstd


def bn_forward_apply(x, mean, invstd, weight, bias, relu=False):
    """y = (x - mean) * invstd * weight + bias with given per-channel vectors (then max(., 0)
    if relu)."""
    xc, N, C, HW = _as_nchw(x, "input")
    y = torch.empty_like(xc)
    _lib.call("mn_bn_relu_fwd_apply_f32" if relu else "mn_bn_fwd_apply_f32", _lib.ptr(xc), _lib.ptr(mean), _lib.ptr(invstd),
              _lib.ptr(weight), _lib.ptr(bias), _lib.ptr(y), N, C, HW, _lib.stream_ptr(x.device))
    return y


def _bn_backward(entry, grad, t, weight, shift, invstd):
    tc, N, C, HW = _as_nchw(t, "stored activation")
    g = grad if grad.is_contiguous() else grad.contiguous()
    _lib.require_gpu_tensor(g, "grad_output", torch.float32)
    if g.shape != tc.shape:
        raise RuntimeError("grad_output and the stored activation differ in shape")
    dx = torch.empty_like(tc)
    dw = torch.empty(C, dtype=torch.float32, device=t.device)
    db = torch.empty(C, dtype=torch.float32, device=t.device)
    ws, nbytes = _workspace(N, C, HW, t.device)
    _ws_call((ws, nbytes, N, C, HW), entry, _lib.ptr(g), _lib.ptr(tc), _lib.ptr(weight), _lib.ptr(shift),
              _lib.ptr(invstd), _lib.ptr(dx), _lib.ptr(dw), _lib.ptr(db), N, C, HW, _lib.ptr(ws),
              nbytes, _lib.stream_ptr(t.device))
    return dx, dw, db


def bn_relu_backward_from_input(grad, x, weight, bias, save_mean, save_invstd):
    """Backward of relu(BN(x)) from the stored input: `grad` is the gradient of the ReLU
    output; the kernel recomputes where the pre-activation was positive."""
    tc, N, C, HW = _as_nchw(x, "stored activation")
    g = grad if grad.is_contiguous() else grad.contiguous()
    _lib.require_gpu_tensor(g, "grad_output", torch.float32)
    if g.shape != tc.shape:
        raise RuntimeError("grad_output and the stored activation differ in shape")
    dx = torch.empty_like(tc)
    dw = torch.empty(C, dtype=torch.float32, device=x.device)
    db = torch.empty(C, dtype=torch.float32, device=x.device)
    ws, nbytes = _workspace(N, C, HW, x.device)
    _ws_call((ws, nbytes, N, C, HW), "mn_bn_relu_bwd_from_x_f32", _lib.ptr(g), _lib.ptr(tc), _lib.ptr(weight), _lib.ptr(bias),
              _lib.ptr(save_mean), _lib.ptr(save_invstd), _lib.ptr(dx), _lib.ptr(dw), _lib.ptr(db),
              N, C, HW, _lib.ptr(ws), nbytes, _lib.stream_ptr(x.device))
    return dx, dw, db


def bn_backward_from_input(grad, x, weight, save_mean, save_invstd):
    return _bn_backward("mn_bn_bwd_from_x_f32", grad, x, weight, save_mean, save_invstd)


def bn_backward_from_output(grad, y, weight, bias, save_invstd):
    return _bn_backward("mn_bn_bwd_from_y_f32", grad, y, weight, bias, save_invstd)


class _BatchNormForward(OP):
    params = None   # (training, eps, save_mean, save_invstd, reserve)
    running_mean = None
    running_var = None
    fused_relu = False

    def forward(self, input_, weight, bias, running_mean, running_var,
                training=False, momentum=0.1, eps=1e-5, *args, **kwargs):
        with torch.no_grad():
            if self.running_mean is None and running_mean is not None:
                self.running_mean = running_mean.requires_grad_(False)
                self.running_var = running_var.requires_grad_(False)
            if self.params is None:
                if training:
                    out, save_mean, save_invstd = bn_forward_train(
                        input_, weight, bias, self.running_mean, self.running_var, momentum, eps,
                        relu=self.fused_relu)
                else:
                    # inference statistics: normalise with the running ones
                    save_mean = self.running_mean
                    save_invstd = torch.rsqrt(self.running_var + eps)
                    out = bn_forward_apply(input_, save_mean, save_invstd, weight, bias,
                                           relu=self.fused_relu)
                self.params = bool(training), eps, save_mean, save_invstd, None
            else:
                _, _, save_mean, save_invstd, _ = self.params
                out = bn_forward_apply(input_, save_mean, save_invstd, weight, bias,
                                       relu=self.fused_relu)
            return out


@implements(['aten::batch_norm'],
            ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode',
             'conv_normal'])
class InputActBatchNorm(_BatchNormForward):
    backward_storage = InputStorage(0, 1, 2, 3, 4)

    def backward(self, grad_output, stored, nodel=False):
        with torch.no_grad():
            input_, weight, bias, running_mean, running_var = stored
            training, eps, save_mean, save_invstd, _ = self.params
            if not training:
                raise NotImplementedError
            di, dw, db = bn_backward_from_input(grad_output, input_, weight, save_mean, save_invstd)
            if not nodel:
                del stored[4], stored[3], stored[2], stored[1], stored[0]
            return di, dw, db, None, None


@implements(['aten::batch_norm'], ['multiway', 'multiway_newnode', 'conv_multiway_newnode'])
class OutputActBatchNorm(_BatchNormForward):
    backward_storage = [InputStorage(1, 2, 3, 4), OutputStorage()]

    def backward(self, grad_output, stored, nodel=False):
        with torch.no_grad():
            weight, bias, running_mean, running_var, output = stored
            training, eps, save_mean, save_invstd, _ = self.params
            if not training:
                raise NotImplementedError
            di, dw, db = bn_backward_from_output(grad_output, output, weight, bias, save_invstd)
            if not nodel:
                del stored[4], stored[3], stored[2], stored[1], stored[0]
            return di, dw, db, None, None


FUSED_BN_RELU = 'monet::batch_norm_relu'


@implements([FUSED_BN_RELU],
            ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode',
             'conv_normal'])
class InputActBatchNormReLU(_BatchNormForward):
    """BatchNorm and the ReLU behind it as ONE operator (the tracer's optional fusion pass
    produces `monet::batch_norm_relu` nodes; the reference has no such operator).  Keeps the
    BatchNorm INPUT: the backward recomputes where the pre-activation was positive, so no
    mask and no intermediate tensor exist, and each direction is one pass over the data."""
    backward_storage = InputStorage(0, 1, 2, 3, 4)
    fused_relu = True

    def backward(self, grad_output, stored, nodel=False):
        with torch.no_grad():
            input_, weight, bias, running_mean, running_var = stored
            training, eps, save_mean, save_invstd, _ = self.params
            if not training:
                raise NotImplementedError
            di, dw, db = bn_relu_backward_from_input(grad_output, input_, weight, bias, save_mean,
                                                     save_invstd)
            if not nodel:
                del stored[4], stored[3], stored[2], stored[1], stored[0]
            return di, dw, db, None, None


FUSED_BN_ADD_RELU = 'monet::batch_norm_add_relu'


def _mask_like(t):
    return torch.empty((t.numel() + 7) // 8, dtype=torch.uint8, device=t.device)


def bn_add_relu_forward_train(x, weight, bias, running_mean, running_var, added, alpha, momentum,
                              eps, want_mask=False):
    """Training forward of max(BN(x) + alpha*added, 0) -> (y, save_mean, save_invstd), with
    `want_mask` -> (y, mask of y > 0, save_mean, save_invstd)."""
    xc, N, C, HW = _as_nchw(x, "input")
    ac, _, _, _ = _as_nchw(added, "added activation")
    if ac.shape != xc.shape:
        raise RuntimeError("the added activation must have the shape of the BatchNorm input")
    y = torch.empty_like(xc)
    save_mean = torch.empty(C, dtype=torch.float32, device=x.device)
    save_invstd = torch.empty(C, dtype=torch.float32, device=x.device)
    ws, nbytes = _workspace(N, C, HW, x.device)
    if want_mask:
        mask = _mask_like(y)
        _ws_call((ws, nbytes, N, C, HW), "mn_bn_add_relu_mask_fwd_train_f32", _lib.ptr(xc), _lib.ptr(weight),
                  _lib.ptr(bias), _lib.ptr(running_mean), _lib.ptr(running_var), _lib.ptr(ac),
                  float(alpha), _lib.ptr(y), _lib.ptr(mask), _lib.ptr(save_mean),
                  _lib.ptr(save_invstd), N, C, HW, float(momentum), float(eps), _lib.ptr(ws), nbytes,
                  _lib.stream_ptr(x.device))
        return y, mask, save_mean, save_invstd
    _ws_call((ws, nbytes, N, C, HW), "mn_bn_add_relu_fwd_train_f32", _lib.ptr(xc), _lib.ptr(weight), _lib.ptr(bias),
              _lib.ptr(running_mean), _lib.ptr(running_var), _lib.ptr(ac), float(alpha), _lib.ptr(y),
              _lib.ptr(save_mean), _lib.ptr(save_invstd), N, C, HW, float(momentum), float(eps),
              _lib.ptr(ws), nbytes, _lib.stream_ptr(x.device))
    return y, save_mean, save_invstd


def bn_add_relu_forward_apply(x, mean, invstd, weight, bias, added, alpha, want_mask=False):
    """max((x - mean) * invstd * weight + bias + alpha*added, 0) with given per-channel vectors
    (`want_mask`: also the packed mask of the result > 0)."""
    xc, N, C, HW = _as_nchw(x, "input")
    ac, _, _, _ = _as_nchw(added, "added activation")
    if ac.shape != xc.shape:
        raise RuntimeError("the added activation must have the shape of the BatchNorm input")
    y = torch.empty_like(xc)
    if want_mask:
        mask = _mask_like(y)
        _lib.call("mn_bn_add_relu_mask_fwd_apply_f32", _lib.ptr(xc), _lib.ptr(mean),
                  _lib.ptr(invstd), _lib.ptr(weight), _lib.ptr(bias), _lib.ptr(ac), float(alpha),
                  _lib.ptr(y), _lib.ptr(mask), N, C, HW, _lib.stream_ptr(x.device))
        return y, mask
    _lib.call("mn_bn_add_relu_fwd_apply_f32", _lib.ptr(xc), _lib.ptr(mean), _lib.ptr(invstd),
              _lib.ptr(weight), _lib.ptr(bias), _lib.ptr(ac), float(alpha), _lib.ptr(y), N, C, HW,
              _lib.stream_ptr(x.device))
    return y


def bn_add_relu_backward(grad, x, y, weight, save_mean, save_invstd, alpha, mask=None):
    """Backward of y = relu(BN(x) + alpha*added) from x and y (or, with `mask`, from x and the
    packed mask of y > 0) in one pass -> (dx, dweight, dbias, dadded).  `grad` is overwritten:
    dadded lives in its storage."""
    tc, N, C, HW = _as_nchw(x, "stored input")
    g = grad if grad.is_contiguous() else grad.contiguous()
    _lib.require_gpu_tensor(g, "grad_output", torch.float32)
    if g.shape != tc.shape:
        raise RuntimeError("grad_output and the stored activations differ in shape")
    if mask is not None:
        _lib.require_gpu_tensor(mask, "mask", torch.uint8)
        if mask.numel() != (tc.numel() + 7) // 8:
            raise RuntimeError("the mask does not have one bit per element")
        dx = torch.empty_like(tc)
        dw = torch.empty(C, dtype=torch.float32, device=x.device)
        db = torch.empty(C, dtype=torch.float32, device=x.device)
        ws, nbytes = _workspace(N, C, HW, x.device)
        _ws_call((ws, nbytes, N, C, HW), "mn_bn_add_relu_mask_bwd_f32", _lib.ptr(g), _lib.ptr(tc), _lib.ptr(mask),
                  _lib.ptr(weight), _lib.ptr(save_mean), _lib.ptr(save_invstd), float(alpha),
                  _lib.ptr(dx), _lib.ptr(g), _lib.ptr(dw), _lib.ptr(db), N, C, HW, _lib.ptr(ws),
                  nbytes, _lib.stream_ptr(x.device))
        return dx, dw, db, g
    yc, _, _, _ = _as_nchw(y, "stored output")
    if yc.shape != tc.shape:
        raise RuntimeError("grad_output and the stored activations differ in shape")
    dx = torch.empty_like(tc)
    dw = torch.empty(C, dtype=torch.float32, device=x.device)
    db = torch.empty(C, dtype=torch.float32, device=x.device)
    ws, nbytes = _workspace(N, C, HW, x.device)
    _ws_call((ws, nbytes, N, C, HW), "mn_bn_add_relu_bwd_f32", _lib.ptr(g), _lib.ptr(tc), _lib.ptr(yc), _lib.ptr(weight),
              _lib.ptr(save_mean), _lib.ptr(save_invstd), float(alpha), _lib.ptr(dx), _lib.ptr(g),
              _lib.ptr(dw), _lib.ptr(db), N, C, HW, _lib.ptr(ws), nbytes, _lib.stream_ptr(x.device))
    return dx, dw, db, g


@implements([FUSED_BN_ADD_RELU],
            ['normal', 'multiway', 'newnode', 'multiway_newnode', 'conv_multiway_newnode',
             'conv_normal'])
class InputActBatchNormAddReLU(OP):
    """The end of a residual block, relu(BN(x) + alpha*added), as ONE operator (the tracer's
    second fusion level produces `monet::batch_norm_add_relu` nodes with the BatchNorm's
    arguments followed by the add's second operand and factor; the reference runs the three
    operators of bn.py:12-54, funcs.py:34-59 and relu.py one after the other).  The forward is
    one pass (2 reads + 1 write instead of 3 + 2).  Keeps the BatchNorm input and the output:
    the backward gates the gradient by the sign of the output (that is the gradient of `added`)
    and continues as BatchNorm backward from the input, in one pass as well (3 reads + 2 writes
    instead of 2 + 1 for the ReLU backward and 2 + 1 for the BatchNorm backward)."""
    backward_storage = [InputStorage(0, 1, 2, 3, 4), OutputStorage()]
    params = None   # (training, eps, save_mean, save_invstd, alpha)
    running_mean = None
    running_var = None
    keeps_mask = False
    overwrites_grad = True   # the gradient of `added` is written over the incoming gradient

    def forward(self, input_, weight, bias, running_mean, running_var, training, momentum, eps,
                cudnn_enabled, added, alpha=1):
        with torch.no_grad():
            if self.running_mean is None and running_mean is not None:
                self.running_mean = running_mean.requires_grad_(False)
                self.running_var = running_var.requires_grad_(False)
            m = self.keeps_mask
            if self.params is None:
                if training:
                    res = bn_add_relu_forward_train(
                        input_, weight, bias, self.running_mean, self.running_var, added, alpha,
                        momentum, eps, want_mask=m)
                    out, save_mean, save_invstd = res[:-2], res[-2], res[-1]
                else:
                    save_mean = self.running_mean
                    save_invstd = torch.rsqrt(self.running_var + eps)
                    out = bn_add_relu_forward_apply(input_, save_mean, save_invstd, weight, bias,
                                                    added, alpha, want_mask=m)
                    out = out if m else (out,)
                self.params = bool(training), eps, save_mean, save_invstd, alpha
            else:
                _, _, save_mean, save_invstd, _ = self.params
                out = bn_add_relu_forward_apply(input_, save_mean, save_invstd, weight, bias, added,
                                                alpha, want_mask=m)
                out = out if m else (out,)
            return tuple(out) if m else out[0]

    def backward(self, grad_output, stored, nodel=False):
        with torch.no_grad():
            input_, weight, bias, running_mean, running_var, output = stored
            training, eps, save_mean, save_invstd, alpha = self.params
            if not training:
                raise NotImplementedError
            di, dw, db, da = bn_add_relu_backward(grad_output, input_, output, weight, save_mean,
                                                  save_invstd, alpha)
            if not nodel:
                del stored[5], stored[4], stored[3], stored[2], stored[1], stored[0]
            return di, dw, db, None, None, da


@implements([FUSED_BN_ADD_RELU], ['newnode', 'multiway_newnode', 'conv_multiway_newnode'])
class BinaryActBatchNormAddReLU(InputActBatchNormAddReLU):
    """The same operator keeping the BatchNorm input and a 1-bit mask of the output's sign
    instead of the output: the forward writes the mask along with the output, the backward
    reads gradient, input and mask (4 + 1/32 passes instead of 5)."""
    backward_storage = [InputStorage(0, 1, 2, 3, 4),
                        IntermediateStorage(lambda shape: (_numel(shape) + 7) // 8)]
    keeps_mask = True

    def backward(self, grad_output, stored, nodel=False):
        with torch.no_grad():
            input_, weight, bias, running_mean, running_var, mask = stored
            training, eps, save_mean, save_invstd, alpha = self.params
            if not training:
                raise NotImplementedError
            di, dw, db, da = bn_add_relu_backward(grad_output, input_, None, weight, save_mean,
                                                  save_invstd, alpha, mask=mask)
            if not nodel:
                del stored[5], stored[4], stored[3], stored[2], stored[1], stored[0]
            return di, dw, db, None, None, da
