"""Convolution operator implementations (reference: monet/lm_ops/conv.py).

  GreedyAlgoConvolution    times every kernel variant on first use and keeps
                           the fastest that fits the memory budget (conv.py:105-258)
  SpecificAlgoConvolution  runs the variant the schedule solver chose
                           (conv.py:260-341)

`algorithm` follows the reference's encoding: forward uses it as the variant
index; backward uses `algorithm // 10` as what to compute (0: weight gradient
(+ bias gradient), 1: input gradient, 2: both) and `algorithm % 10` as the
variant index.  A variant that cannot run (index out of range, unsupported
shape) raises; the op then retries with variant 0, which always runs, and
rewrites `algorithm` the way the reference falls back to its default
algorithm (conv.py:279-283, 308-312, 321-325).

The variants are the kernels' own memory / speed tiers (see
include/monet_hip.h), and their workspaces are torch tensors, so the caching
allocator - and with it the solver's memory profile - sees them.
"""
import ctypes
from time import time

import torch

from .. import _lib, config
from .base import OP, InputStorage, implements

DEFAULT_VARIANT = 0


def _refused(exc):
    """True when a kernel variant was refused before anything was launched (unknown index,
    shape it does not cover): the only failures the operators answer by running variant 0.
    Launch failures, invalid arguments (MN_EINVAL: a null or misaligned pointer, a workspace
    smaller than mn_conv_ws_bytes asked for), host-side shape / dtype errors and allocator
    failures propagate."""
    return isinstance(exc, _lib.MonetHipError) and exc.status == _lib.MN_EUNSUPPORTED


def _pair(v):
    v = list(v) if isinstance(v, (list, tuple, torch.Size)) else [v]
    if len(v) == 1:
        v = v * 2
    return int(v[0]), int(v[1])


def conv_geometry(input_shape, weight_shape, stride, padding, dilation, groups):
    N, C, H, W = [int(d) for d in input_shape]
    K, Cg, R, S = [int(d) for d in weight_shape]
    sH, sW = _pair(stride)
    pH, pW = _pair(padding)
    dH, dW = _pair(dilation)
    if Cg * groups != C:
        raise RuntimeError("weight does not match the input channels")
    P = (H + 2 * pH - dH * (R - 1) - 1) // sH + 1
    Q = (W + 2 * pW - dW * (S - 1) - 1) // sW + 1
    if P <= 0 or Q <= 0:
        raise RuntimeError("convolution output would be empty")
    return _lib.Conv2d(N, C, H, W, K, R, S, sH, sW, pH, pW, dH, dW, P, Q, int(groups))


def _n_variants(direction, dtype):
    code = _lib.BF16 if dtype == torch.bfloat16 else _lib.F32
    return _lib.load().mn_conv_n_variants_for(direction, code)


def n_fwd_algos(dtype=None):
    """Kernel variants of the forward (fp32 unless `dtype` is torch.bfloat16)."""
    return _n_variants(_lib.CONV_FWD, dtype)


def n_bwd_ip_algos(dtype=None):
    return _n_variants(_lib.CONV_BWD_DATA, dtype)


def n_bwd_wt_algos(dtype=None):
    return _n_variants(_lib.CONV_BWD_WEIGHT, dtype)


def _workspace(geo, direction, variant, device, dtype=None):
    n = ctypes.c_size_t(0)
    _lib.call("mn_conv_ws_bytes", geo, direction, variant, _lib.F32 if dtype is None else dtype,
              ctypes.byref(n))
    if n.value == 0:
        return None, 0
    return torch.empty(n.value, dtype=torch.uint8, device=device), n.value


def _prep(t, name):
    """(tensor the kernels can read, library dtype code).  fp32 tensors are used as dense
    NCHW; bf16 tensors as channels-last (NHWC memory under the same logical shape)."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        _lib.require_gpu_tensor(t, name)
    t = t.detach()
    if t.dtype == torch.bfloat16:
        if t.dim() == 4:
            t = t.contiguous(memory_format=torch.channels_last)
        elif not t.is_contiguous():
            t = t.contiguous()
        return t, _lib.BF16
    _lib.require_gpu_tensor(t, name, torch.float32)
    return (t if t.is_contiguous() else t.contiguous()), _lib.F32


def _same_dtype(*codes):
    if len(set(codes)) != 1:
        raise RuntimeError("convolution operands must share one dtype (all fp32 or all bf16)")
    return codes[0]


def _empty(shape, code, device):
    shape = [int(d) for d in shape]
    if code == _lib.BF16:
        return torch.empty(shape, dtype=torch.bfloat16, device=device,
                           memory_format=torch.channels_last)
    return torch.empty(shape, dtype=torch.float32, device=device)


def conv_forward(input_, weight, bias, padding, stride, dilation, groups, variant):
    """y = conv2d(input, weight) (+ bias) with kernel variant `variant`."""
    (x, cx), (w, cw) = _prep(input_, "input"), _prep(weight, "weight")
    code = _same_dtype(cx, cw)
    b = None
    if bias is not None:
        b, cb = _prep(bias, "bias")
        _same_dtype(code, cb)
    geo = conv_geometry(x.shape, w.shape, stride, padding, dilation, groups)
    ws, nbytes = _workspace(geo, _lib.CONV_FWD, variant, x.device, code)
    y = _empty((geo.N, geo.K, geo.P, geo.Q), code, x.device)
    _lib.call("mn_conv_fwd", geo, _lib.ptr(x), _lib.ptr(w), _lib.ptr(b), _lib.ptr(y), _lib.ptr(ws),
              nbytes, variant, code, _lib.stream_ptr(x.device))
    return y


def conv_backward_input(input_shape, grad_output, weight, padding, stride, dilation, groups,
                        variant, accumulate_into=None):
    """Gradient w.r.t. the input.  `accumulate_into`: an fp32 contiguous tensor of the input's
    shape that already holds a gradient; the result is then ADDED to it by the kernel's
    epilogue and that tensor is returned (no separate addition pass)."""
    (g, cg), (w, cw) = _prep(grad_output, "grad_output"), _prep(weight, "weight")
    code = _same_dtype(cg, cw)
    geo = conv_geometry(input_shape, w.shape, stride, padding, dilation, groups)
    if tuple(g.shape) != (geo.N, geo.K, geo.P, geo.Q):
        raise RuntimeError("grad_output does not match the convolution geometry")
    ws, nbytes = _workspace(geo, _lib.CONV_BWD_DATA, variant, g.device, code)
    acc = accumulate_into
    if acc is not None and code == _lib.F32 and acc.dtype == torch.float32 and acc.is_cuda and \
            acc.is_contiguous() and list(acc.shape) == [int(d) for d in input_shape]:
        _lib.call("mn_conv_bwd_data_accumulate", geo, _lib.ptr(g), _lib.ptr(w), _lib.ptr(acc),
                  _lib.ptr(ws), nbytes, variant, code, _lib.stream_ptr(g.device))
        return acc
    dx = _empty(input_shape, code, g.device)
    _lib.call("mn_conv_bwd_data", geo, _lib.ptr(g), _lib.ptr(w), _lib.ptr(dx), _lib.ptr(ws), nbytes,
              variant, code, _lib.stream_ptr(g.device))
    return dx


def conv_backward_weight(weight_shape, grad_output, input_, padding, stride, dilation, groups,
                         variant, with_bias_grad=False):
    """Gradient w.r.t. the weights.  `with_bias_grad`: return (dw, db) with the bias gradient
    db = grad_output.sum([0, 2, 3]) (conv.py:314) reduced by the same kernel from the tiles of
    grad_output it fetches anyway (fp32); for bf16 tensors db is a separate reduction."""
    (g, cg), (x, cx) = _prep(grad_output, "grad_output"), _prep(input_, "input")
    code = _same_dtype(cg, cx)
    geo = conv_geometry(x.shape, weight_shape, stride, padding, dilation, groups)
    if tuple(g.shape) != (geo.N, geo.K, geo.P, geo.Q):
        raise RuntimeError("grad_output does not match the convolution geometry")
    ws, nbytes = _workspace(geo, _lib.CONV_BWD_WEIGHT, variant, g.device, code)
    dw = _empty(weight_shape, code, g.device)
    if with_bias_grad and code == _lib.F32:
        db = torch.empty(geo.K, dtype=torch.float32, device=g.device)
        _lib.call("mn_conv_bwd_weight_bias", geo, _lib.ptr(g), _lib.ptr(x), _lib.ptr(dw),
                  _lib.ptr(db), _lib.ptr(ws), nbytes, variant, code, _lib.stream_ptr(g.device))
        return dw, db
    _lib.call("mn_conv_bwd_weight", geo, _lib.ptr(g), _lib.ptr(x), _lib.ptr(dw), _lib.ptr(ws),
              nbytes, variant, code, _lib.stream_ptr(g.device))
    if with_bias_grad:
        return dw, grad_output.sum([0, 2, 3])
    return dw


def _depthwise_forward(input_, weight, bias, stride, padding, dilation, groups):
    return torch.ops.aten.convolution(input_, weight, bias, list(stride), list(padding),
                                      list(dilation), False, [0, 0], groups)


def _depthwise_backward(grad, input_, weight, stride, padding, dilation, groups, mask,
                        input_shape=None):
    """(di, dw) of a grouped convolution through aten.  `mask` says which of the two to
    compute.  When the executor has already dropped the input (input-gradient step of a split
    backward) di is the transposed convolution of the gradient, which reads no input at all:
    handing aten.convolution_backward a shape-only stand-in would make it materialise a
    full-size copy of it, memory the schedule counts as free."""
    if input_ is None:
        assert not mask[1] and input_shape is not None
        spatial = [int(d) for d in input_shape[2:]]
        out_pad = [spatial[i] - ((grad.shape[2 + i] - 1) * stride[i] - 2 * padding[i] +
                                 dilation[i] * (weight.shape[2 + i] - 1) + 1)
                   for i in range(len(spatial))]
        di = torch.nn.functional.conv_transpose2d(grad, weight, None, list(stride), list(padding),
                                                  out_pad, groups, list(dilation))
        return di, None
    di, dw, _ = torch.ops.aten.convolution_backward(
        grad, input_, weight, None, list(stride), list(padding), list(dilation), False, [0, 0],
        groups, [bool(mask[0]), bool(mask[1]), False])
    return di, dw


class _ConvBase(OP):
    backward_storage = InputStorage(0, 1)
    params = None
    algorithm = -1
    is_depthwise = False

    n_fwd_algos = staticmethod(n_fwd_algos)
    n_bwd_ip_algos = staticmethod(n_bwd_ip_algos)
    n_bwd_wt_algos = staticmethod(n_bwd_wt_algos)

    def _record(self, input_, weight, bias, stride, padding, dilation, groups):
        self.params = (stride, padding, dilation, groups, input_.shape, weight.shape,
                       [input_.requires_grad, weight.requires_grad,
                        bias is not None and bias.requires_grad, bias is not None])

    # hooks the two subclasses differ in
    def _fwd_variant(self, *a):
        raise NotImplementedError

    def _bwd_wt_variant(self, *a):
        raise NotImplementedError

    def _bwd_ip_variant(self, *a):
        raise NotImplementedError

    def forward(self, input_, weight, bias, stride, padding, dilation, transposed, output_padding,
                groups, *args, **kwargs):
        with torch.no_grad():
            assert not transposed
            self._record(input_, weight, bias, stride, padding, dilation, groups)
            if self.is_depthwise or groups != 1:
                return _depthwise_forward(input_, weight, bias, stride, padding, dilation, groups)
            return self._fwd_variant(input_, weight, bias, padding, stride, dilation, groups)

    # True: `backward(..., accumulate_into=t)` adds the input gradient to `t` inside the kernel
    accumulates_input_grad = False

    def backward(self, grad_output, stored, nodel=False, accumulate_into=None):
        with torch.no_grad():
            input_, weight = stored
            stride, padding, dilation, groups, input_shape, weight_shape, do_grad = self.params
            kind = self.algorithm // 10
            if not nodel:
                del stored[1]
                del stored[0]
            di = dw = db = None
            if self.is_depthwise:
                # one backward step computes everything (conv.py:301-302 in the reference)
                di, dw = _depthwise_backward(grad_output, input_, weight, stride, padding, dilation,
                                             groups, do_grad[:2])
                if do_grad[2]:
                    db = grad_output.sum([0, 2, 3])
            elif groups != 1:
                # grouped, not depthwise: split like every other convolution (kind 0: parameter
                # gradients, 1: input gradient, 2: both), the arithmetic is aten's
                want_di = kind in (1, 2) and do_grad[0] and weight is not None
                want_dw = kind in (0, 2) and do_grad[1] and input_ is not None
                if want_di or want_dw:
                    di, dw = _depthwise_backward(grad_output, input_, weight, stride, padding,
                                                 dilation, groups, [want_di, want_dw], input_shape)
                if kind in (0, 2) and do_grad[2]:
                    db = grad_output.sum([0, 2, 3])
            else:
                if kind in (0, 2) and input_ is not None:
                    if do_grad[1] and do_grad[2]:
                        dw, db = self._bwd_wt_variant(weight_shape, grad_output, input_, padding,
                                                      stride, dilation, groups, True)
                    elif do_grad[1]:
                        dw = self._bwd_wt_variant(weight_shape, grad_output, input_, padding, stride,
                                                  dilation, groups)
                    elif do_grad[2]:
                        db = grad_output.sum([0, 2, 3])
                del input_
                if kind in (1, 2) and weight is not None and do_grad[0]:
                    if accumulate_into is not None and self.accumulates_input_grad:
                        di = self._bwd_ip_variant(input_shape, grad_output, weight, padding, stride,
                                                  dilation, groups, accumulate_into)
                    else:
                        di = self._bwd_ip_variant(input_shape, grad_output, weight, padding, stride,
                                                  dilation, groups)
            if do_grad[3]:  # bias present: one gradient per tensor argument of the forward
                return di, dw, db
            return di, dw


@implements(['aten::_convolution'], ['conv_multiway_newnode', 'conv_normal'])
class SpecificAlgoConvolution(_ConvBase):
    """Runs exactly the variant in `self.algorithm`; falls back to variant 0."""
    accumulates_input_grad = True

    def _fwd_variant(self, input_, weight, bias, padding, stride, dilation, groups):
        try:
            return conv_forward(input_, weight, bias, padding, stride, dilation, groups,
                                self.algorithm)
        except _lib.MonetHipError as e:
            if not _refused(e):
                raise
            out = conv_forward(input_, weight, bias, padding, stride, dilation, groups,
                               DEFAULT_VARIANT)
            self.algorithm = DEFAULT_VARIANT
            return out

    def _bwd_wt_variant(self, weight_shape, grad, input_, padding, stride, dilation, groups,
                        with_bias_grad=False):
        kind, algo = self.algorithm // 10, self.algorithm % 10
        try:
            return conv_backward_weight(weight_shape, grad, input_, padding, stride, dilation,
                                        groups, algo, with_bias_grad)
        except _lib.MonetHipError as e:
            if not _refused(e):
                raise
            out = conv_backward_weight(weight_shape, grad, input_, padding, stride, dilation,
                                       groups, DEFAULT_VARIANT, with_bias_grad)
            self.algorithm = kind * 10 + DEFAULT_VARIANT
            return out

    def _bwd_ip_variant(self, input_shape, grad, weight, padding, stride, dilation, groups,
                        acc=None):
        kind, algo = self.algorithm // 10, self.algorithm % 10
        try:
            return conv_backward_input(input_shape, grad, weight, padding, stride, dilation, groups,
                                       algo, acc)
        except _lib.MonetHipError as e:
            if not _refused(e):
                raise
            # (a refused variant launched nothing, so nothing was added yet)
            out = conv_backward_input(input_shape, grad, weight, padding, stride, dilation, groups,
                                      DEFAULT_VARIANT, acc)
            self.algorithm = kind * 10 + DEFAULT_VARIANT
            return out


def _autotune(n_variants, run):
    """Index of the fastest variant (10 runs each) whose peak allocation stays
    under config.budget * 1.01 GB (no limit when the budget is 0)."""
    best, best_t = -1, None
    torch.cuda.empty_cache()
    for alg in range(n_variants):
        try:
            torch.cuda.reset_peak_memory_stats()
            torch.cuda.synchronize()
            t1 = time()
            for _ in range(10):
                out = run(alg)
                del out
            torch.cuda.synchronize()
            t = time() - t1
            peak_gb = torch.cuda.max_memory_allocated() / 1024 / 1024 / 1024
            fits = config.budget <= 0 or peak_gb < config.budget * 1.01
            if fits and (best_t is None or t < best_t):
                best, best_t = alg, t
        except _lib.MonetHipError as e:
            if not _refused(e):
                raise
        except torch.cuda.OutOfMemoryError:
            pass  # a variant whose workspace does not fit is not a candidate
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats()
    if best == -1:
        best = DEFAULT_VARIANT
    return best


@implements(['aten::_convolution'], ['normal', 'multiway_newnode', 'multiway', 'newnode'])
class GreedyAlgoConvolution(_ConvBase):
    """Picks each direction's variant by timing on first use, then keeps it."""
    fwd_algo = -1
    bwd_ip_algo = -1
    bwd_wt_algo = -1

    def _fwd_variant(self, input_, weight, bias, padding, stride, dilation, groups):
        if self.fwd_algo == -1:
            self.fwd_algo = _autotune(n_fwd_algos(), lambda alg: conv_forward(
                input_, weight, bias, padding, stride, dilation, groups, alg))
        try:
            return conv_forward(input_, weight, bias, padding, stride, dilation, groups,
                                self.fwd_algo)
        except _lib.MonetHipError as e:
            if not _refused(e):
                raise
            self.fwd_algo = DEFAULT_VARIANT
            return conv_forward(input_, weight, bias, padding, stride, dilation, groups,
                                DEFAULT_VARIANT)

    def _bwd_wt_variant(self, weight_shape, grad, input_, padding, stride, dilation, groups,
                        with_bias_grad=False):
        if self.bwd_wt_algo == -1:
            self.bwd_wt_algo = _autotune(n_bwd_wt_algos(), lambda alg: conv_backward_weight(
                weight_shape, grad, input_, padding, stride, dilation, groups, alg))
        try:
            return conv_backward_weight(weight_shape, grad, input_, padding, stride, dilation,
                                        groups, self.bwd_wt_algo, with_bias_grad)
        except _lib.MonetHipError as e:
            if not _refused(e):
                raise
            self.bwd_wt_algo = DEFAULT_VARIANT
            return conv_backward_weight(weight_shape, grad, input_, padding, stride, dilation,
                                        groups, DEFAULT_VARIANT, with_bias_grad)

    def _bwd_ip_variant(self, input_shape, grad, weight, padding, stride, dilation, groups):
        if self.bwd_ip_algo == -1:
            self.bwd_ip_algo = _autotune(n_bwd_ip_algos(), lambda alg: conv_backward_input(
                input_shape, grad, weight, padding, stride, dilation, groups, alg))
        try:
            return conv_backward_input(input_shape, grad, weight, padding, stride, dilation, groups,
                                       self.bwd_ip_algo)
        except _lib.MonetHipError as e:
            if not _refused(e):
                raise
            self.bwd_ip_algo = DEFAULT_VARIANT
            return conv_backward_input(input_shape, grad, weight, padding, stride, dilation, groups,
                                       DEFAULT_VARIANT)

    def backward(self, grad_output, stored, nodel=False):
        # the greedy op ignores the variant digit of `algorithm` (it uses its own choice)
        return super().backward(grad_output, stored, nodel)
