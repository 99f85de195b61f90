"""CPU oracle for the low-memory operator library.

TEST INFRASTRUCTURE ONLY.  This module restates, in numpy on the CPU, what the
reference implementation (utsaslab/MONeT, `monet/lm_ops`) computes for every
operator the GPU library implements.  Only tests, the smoke check and the
benchmark's CPU-baseline leg may import it; the product never does.

Each function cites the reference code it follows (paths relative to the
reference root).  How each one is pinned independently of this file is listed
next to it ("pinned by"); those checks live in tests/test_oracle.py.  The
reference ships no tests or golden vectors for this path, so the pins are
closed forms, library routines (numpy.packbits, torch CPU operators and
autograd) and brute force on small inputs.

Intentional differences from the reference, all in corner cases where the
reference's result is not meaningful:
  * max-pool forward: a window whose elements are all -inf reports the index
    of its first valid element (the reference stores an unrelated byte,
    maxpool.cu:55);
  * max-pool backward with dilation > 1 only credits positions that lie on the
    dilated grid (the reference's integer division also matches positions
    between grid points, maxpool.cu:111 "This works for very few cases");
  * BatchNorm recomputation re-applies the saved invstd (the reference adds
    eps twice, bn.py:32-34).
"""
import numpy as np

# --------------------------------------------------------------------- pack


def pack_bits(bools):
    """8 bools -> 1 byte, first element in bit 7; tail bits zero.

    Follows pack_cpu (monet/lm_ops/pack.cpp:6-13) / pack_kernel (pack.cu:22-31).
    Pinned by: numpy.packbits(bitorder='big'); hand-written known answers.
    """
    b = np.asarray(bools).astype(np.uint8).reshape(-1) & 1
    n = b.size
    nb = (n + 7) // 8
    padded = np.zeros(nb * 8, dtype=np.uint8)
    padded[:n] = b
    out = np.zeros(nb, dtype=np.uint8)
    for k in range(8):  # element 8j + (7-k) carries weight 2^k
        out |= padded[7 - k::8] << k
    return out


def unpack_bits(packed, n=0):
    """Inverse of pack_bits (pack.cpp:15-21, pack.cu:32-40); n defaults to 8*len."""
    p = np.asarray(packed, dtype=np.uint8).reshape(-1)
    n = n or p.size * 8
    out = np.zeros(p.size * 8, dtype=np.uint8)
    for k in range(8):
        out[7 - k::8] = (p >> k) & 1
    return out[:n].astype(bool)


def unpack_bits_mul(packed, v):
    """r[i] = bit(i) * v[i] (pack.cpp:23-30, pack.cu:41-50). Pinned by: v * unpack."""
    v = np.asarray(v)
    bits = unpack_bits(packed, v.size).astype(v.dtype)
    with np.errstate(invalid="ignore"):
        return bits * v.reshape(-1)


def pack_nibbles(u):
    """2 values < 16 -> 1 byte, even index in the high nibble (pack.cu:3-12).

    Pinned by: (a[0::2] << 4) + a[1::2] on even lengths; known answers.
    """
    a = np.asarray(u, dtype=np.uint8).reshape(-1) & 15
    n = a.size
    padded = np.zeros((n + 1) // 2 * 2, dtype=np.uint8)
    padded[:n] = a
    return ((padded[0::2] << 4) | padded[1::2]).astype(np.uint8)


def unpack_nibbles(packed, n=0):
    """Inverse of pack_nibbles (pack.cu:13-21); n defaults to 2*len."""
    p = np.asarray(packed, dtype=np.uint8).reshape(-1)
    n = n or p.size * 2
    out = np.empty(p.size * 2, dtype=np.uint8)
    out[0::2] = p >> 4
    out[1::2] = p & 15
    return out[:n]


# --------------------------------------------------------------------- relu


def relu_fwd_mask(x):
    """(clamp_min(x, 0), pack(x > 0)) - BinaryActReLU.forward (relu.py:100-104).

    NaN stays NaN in y and has a 0 bit; -0.0 has a 0 bit.
    Pinned by: torch.clamp_min / torch.relu on CPU and numpy.packbits(x > 0).
    """
    x = np.asarray(x, dtype=np.float32)
    y = np.where(x > 0, x, np.where(np.isnan(x), x, np.float32(0)))
    return y.astype(np.float32), pack_bits((x > 0).reshape(-1))


def relu_bwd_mask(grad, mask):
    """grad * unpack(mask) - BinaryActReLU.backward (relu.py:109-118).

    A multiply, so grad = inf/NaN under a 0 bit gives NaN and a negative grad
    gives -0.0.  Pinned by: grad * (x > 0) with torch on CPU.
    """
    g = np.asarray(grad, dtype=np.float32)
    return unpack_bits_mul(mask, g.reshape(-1)).reshape(g.shape)


def relu_bwd_ref(grad, ref, threshold=0.0):
    """ref > threshold ? grad : 0 - threshold_kernel (lrrelu.cu:4-9).

    Pinned by: torch.ops.aten.threshold_backward on CPU.
    """
    g = np.asarray(grad, dtype=np.float32)
    r = np.asarray(ref, dtype=np.float32)
    return np.where(r > np.float32(threshold), g, np.float32(0)).astype(np.float32)


# ------------------------------------------------------------------ maxpool


def pool_out_size(size, k, pad, stride, dil, ceil_mode):
    """Output extent - pooling_output_shape (maxpool.cpp:54-75).

    Pinned by: the output shape of torch.nn.functional.max_pool2d on CPU.
    """
    num = size + 2 * pad - dil * (k - 1) - 1 + (stride - 1 if ceil_mode else 0)
    out = num // stride + 1  # python // floors, like div_rtn
    if pad and (out - 1) * stride >= size + pad:
        out -= 1
    return out


def _pair(v):
    if isinstance(v, (list, tuple)):
        return (int(v[0]), int(v[0])) if len(v) == 1 else (int(v[0]), int(v[1]))
    return int(v), int(v)


def _axis_gather(size, pooled, k_off, stride, pad, dil):
    """Input coordinate of window element `k_off` for every pooled position."""
    pos = np.arange(pooled) * stride - pad + k_off * dil
    valid = (pos >= 0) & (pos < size)
    return np.clip(pos, 0, size - 1), valid


def maxpool_fwd_idx(x, kernel_size, stride, padding, dilation=1, ceil_mode=False):
    """(y, packed 4-bit indices, unpacked uint8 indices) of a max pool over NCHW x.

    Follows max_pool_forward_nchw (maxpool.cu:26-72) followed by pack_two
    (pool.py:43-53): the window is scanned row-major from its first in-image
    element; `val > max or isnan(val)` takes over; the index is ch*kW + cw with
    (ch, cw) counted from the unclipped window origin in dilation steps.
    Pinned by: F.max_pool2d(return_indices=True) on CPU after converting its
    flat h*W+w index to the window-relative one; a pure-Python scan on small
    inputs with planted ties, NaNs and -inf windows.
    """
    x = np.asarray(x, dtype=np.float32)
    if x.ndim == 3:
        x = x[None]
    N, C, H, W = x.shape
    kH, kW = _pair(kernel_size)
    sH, sW = _pair(stride) if stride not in (None, [], ()) else (kH, kW)
    pH, pW = _pair(padding)
    dH, dW = _pair(dilation)
    PH = pool_out_size(H, kH, pH, sH, dH, ceil_mode)
    PW = pool_out_size(W, kW, pW, sW, dW, ceil_mode)
    maxval = np.full((N, C, PH, PW), -np.inf, dtype=np.float32)
    # index of the first in-image element of each window
    ch0 = np.maximum(0, -(-(pH - np.arange(PH) * sH) // dH))
    cw0 = np.maximum(0, -(-(pW - np.arange(PW) * sW) // dW))
    maxidx = np.broadcast_to((ch0[:, None] * kW + cw0[None, :]).astype(np.uint8),
                             (N, C, PH, PW)).copy()
    for ch in range(kH):
        hh, vh = _axis_gather(H, PH, ch, sH, pH, dH)
        for cw in range(kW):
            ww, vw = _axis_gather(W, PW, cw, sW, pW, dW)
            val = x[:, :, hh][:, :, :, ww]
            valid = (vh[:, None] & vw[None, :])[None, None]
            with np.errstate(invalid="ignore"):
                take = valid & ((val > maxval) | np.isnan(val))
            maxval = np.where(take, val, maxval)
            maxidx = np.where(take, np.uint8(ch * kW + cw), maxidx)
    return maxval, pack_nibbles(maxidx.reshape(-1)), maxidx


def maxpool_bwd_idx(dy, idx4, input_shape, kernel_size, stride, padding, dilation=1):
    """dx from packed window-relative indices.

    Follows unpack_two + max_pool_backward_nchw (pool.py:55-69,
    maxpool.cu:81-131): every input pixel sums dy over the windows that cover
    it and whose index names it, window rows outer, window columns inner
    (= descending ch, then descending cw), starting from +0.
    Pinned by: autograd of F.max_pool2d on CPU (exact where a pixel has at most
    one contributing window; a few ulp otherwise) and sum(dx) == sum(dy).
    """
    dy = np.asarray(dy, dtype=np.float32)
    if dy.ndim == 3:
        dy = dy[None]
    N, C, PH, PW = dy.shape
    H, W = input_shape[-2:]
    kH, kW = _pair(kernel_size)
    sH, sW = _pair(stride) if stride not in (None, [], ()) else (kH, kW)
    pH, pW = _pair(padding)
    dH, dW = _pair(dilation)
    idx = unpack_nibbles(idx4, dy.size).reshape(dy.shape)
    dx = np.zeros((N, C, H, W), dtype=np.float32)
    for ch in range(kH - 1, -1, -1):
        hh = np.arange(PH) * sH - pH + ch * dH
        mh = (hh >= 0) & (hh < H)
        for cw in range(kW - 1, -1, -1):
            ww = np.arange(PW) * sW - pW + cw * dW
            mw = (ww >= 0) & (ww < W)
            contrib = np.where(idx == ch * kW + cw, dy, np.float32(0))
            sub = contrib[:, :, mh][:, :, :, mw]
            dx[np.ix_(np.arange(N), np.arange(C), hh[mh], ww[mw])] += sub
    return dx.reshape(list(input_shape))


# ---------------------------------------------------------------- batchnorm


def _nchw3(t, dtype):
    t = np.asarray(t, dtype=dtype)
    return t.reshape(t.shape[0], t.shape[1], -1)


def bn_fwd_train(x, gamma, beta, running_mean, running_var, momentum, eps, dtype=np.float64):
    """Training forward -> (y, save_mean, save_invstd, new_running_mean, new_running_var).

    What cudnn_batch_norm returns through do_forward (lrbn.cpp:21-41): batch
    mean and biased variance per channel, invstd = 1/sqrt(var+eps), running
    statistics blended with `momentum` using the unbiased variance.
    Pinned by: F.batch_norm(training=True) on CPU (output and running stats).
    """
    x3 = _nchw3(x, dtype)
    M = x3.shape[0] * x3.shape[2]
    mean = x3.mean(axis=(0, 2))
    var = x3.var(axis=(0, 2))
    invstd = 1.0 / np.sqrt(var + eps)
    g = np.ones_like(mean) if gamma is None else np.asarray(gamma, dtype=dtype)
    b = np.zeros_like(mean) if beta is None else np.asarray(beta, dtype=dtype)
    y = (x3 - mean[None, :, None]) * (invstd * g)[None, :, None] + b[None, :, None]
    rm = rv = None
    if running_mean is not None:
        rm = (1 - momentum) * np.asarray(running_mean, dtype=dtype) + momentum * mean
        rv = (1 - momentum) * np.asarray(running_var, dtype=dtype) + momentum * var * (
            M / max(M - 1, 1))
    return y.reshape(np.shape(x)), mean, invstd, rm, rv


def bn_fwd_apply(x, mean, invstd, gamma, beta, dtype=np.float64):
    """y = (x - mean) * invstd * gamma + beta from saved statistics."""
    x3 = _nchw3(x, dtype)
    mean = np.asarray(mean, dtype=dtype)
    invstd = np.asarray(invstd, dtype=dtype)
    g = np.ones_like(mean) if gamma is None else np.asarray(gamma, dtype=dtype)
    b = np.zeros_like(mean) if beta is None else np.asarray(beta, dtype=dtype)
    y = (x3 - mean[None, :, None]) * (invstd * g)[None, :, None] + b[None, :, None]
    return y.reshape(np.shape(x))


def add_relu_fwd(a, b, alpha=1.0):
    """(max(a + alpha*b, 0), packed 1-bit mask of a + alpha*b > 0) in the operands' dtype: the
    composition of AddIP (monet/lm_ops/funcs.py:41-59) and a ReLU with BinaryActReLU's mask
    (relu.py:94-118).  Pinned through relu_fwd_mask and plain numpy addition."""
    t = (a + np.asarray(alpha, dtype=a.dtype) * b).astype(a.dtype)
    return relu_fwd_mask(t)


def bn_relu_fwd_train(x, gamma, beta, running_mean, running_var, momentum, eps, dtype=np.float64):
    """BatchNorm (training) followed by ReLU, as one operator: the composition of bn_fwd_train
    and max(., 0).  Returns what bn_fwd_train returns with y replaced by relu(y).  (The
    reference runs the two operators separately, monet/lm_ops/bn.py:12-54 and relu.py:9-29.)
    Pinned by: torch.relu(F.batch_norm(training=True)) on CPU in float64."""
    out = list(bn_fwd_train(x, gamma, beta, running_mean, running_var, momentum, eps, dtype))
    out[0] = np.maximum(out[0], 0)
    return tuple(out)


def bn_relu_bwd_from_x(dy, x, gamma, beta, mean, invstd, positive=None, dtype=np.float64):
    """Backward of relu(BN(x)) given the gradient of the ReLU output: mask dy where the
    pre-activation is not positive, then bn_bwd_from_x.  `positive` overrides the mask (a
    caller comparing against another implementation passes that implementation's decisions,
    so that pre-activations within rounding distance of zero do not count as differences).
    Pinned by: float64 autograd through torch.relu(F.batch_norm(...)) for x, gamma and beta."""
    if positive is None:
        shape = [1, -1] + [1] * (x.ndim - 2)
        pre = (x.astype(dtype) - mean.astype(dtype).reshape(shape)) * \
            (invstd.astype(dtype) * gamma.astype(dtype)).reshape(shape) + beta.astype(dtype).reshape(shape)
        positive = pre > 0
    return bn_bwd_from_x(np.where(positive, dy, 0).astype(dy.dtype), x, gamma, mean, invstd, dtype)


def bn_add_relu_fwd_train(x, gamma, beta, added, alpha, running_mean, running_var, momentum, eps,
                          dtype=np.float64):
    """The end of a residual block as one operator: relu(BN(x) + alpha * added), the
    composition of bn_fwd_train, the residual add (monet/lm_ops/funcs.py:34-59) and max(., 0).
    Returns what bn_fwd_train returns with y replaced.
    Pinned by: torch.relu(F.batch_norm(training=True) + alpha * added) on CPU in float64."""
    out = list(bn_fwd_train(x, gamma, beta, running_mean, running_var, momentum, eps, dtype))
    out[0] = np.maximum(out[0] + dtype(alpha) * np.asarray(added, dtype=dtype), 0)
    return tuple(out)


def bn_add_relu_bwd(dy, x, y, gamma, mean, invstd, alpha=1.0, dtype=np.float64):
    """Backward of y = relu(BN(x) + alpha * added) from the stored x and y: the gradient only
    passes where y > 0; that gated gradient times alpha is the gradient of `added`, and
    bn_bwd_from_x turns it into (dx, dgamma, dbeta).  Returns (dx, dgamma, dbeta, dadded).
    Pinned by: float64 autograd through the torch composition for x, gamma, beta and added."""
    g = np.where(np.asarray(y) > 0, dy, 0).astype(np.asarray(dy).dtype)
    dx, dgamma, dbeta = bn_bwd_from_x(g, x, gamma, mean, invstd, dtype)
    return dx, dgamma, dbeta, g.astype(dtype) * dtype(alpha)


def bn_bwd_from_x(dy, x, gamma, mean, invstd, dtype=np.float64):
    """(dx, dgamma, dbeta) from the input: the standard BatchNorm backward that
    cudnn_batch_norm_backward computes for do_cudnn_backward (lrbn.cpp:43-70).

    Pinned by: autograd through F.batch_norm on CPU in float64.
    """
    g3, x3 = _nchw3(dy, dtype), _nchw3(x, dtype)
    M = x3.shape[0] * x3.shape[2]
    mean = np.asarray(mean, dtype=dtype)
    invstd = np.asarray(invstd, dtype=dtype)
    w = np.ones_like(mean) if gamma is None else np.asarray(gamma, dtype=dtype)
    xhat = (x3 - mean[None, :, None]) * invstd[None, :, None]
    dbeta = g3.sum(axis=(0, 2))
    dgamma = (g3 * xhat).sum(axis=(0, 2))
    dx = (g3 - xhat * (dgamma / M)[None, :, None] - (dbeta / M)[None, :, None]) * (
        invstd * w)[None, :, None]
    return dx.reshape(np.shape(x)), dgamma, dbeta


def bn_bwd_from_y(dy, y, gamma, beta, invstd, dtype=np.float64):
    """(dx, dgamma, dbeta) from the OUTPUT y, never touching x.

    Follows batch_norm_backward_kernel1 (lrbn.cu:138-209): gsum = sum dy,
    dot = sum dy*(y - beta); dbeta = gsum, dgamma = dot/gamma,
    dx = (dy - (y-beta)*dot/(M*gamma^2) - gsum/M) * invstd * gamma.
    Pinned by: equality with bn_bwd_from_x / float64 autograd when y is the true
    training-mode output of x.
    """
    g3, y3 = _nchw3(dy, dtype), _nchw3(y, dtype)
    M = y3.shape[0] * y3.shape[2]
    w = np.asarray(gamma, dtype=dtype)
    b = np.asarray(beta, dtype=dtype)
    invstd = np.asarray(invstd, dtype=dtype)
    yc = y3 - b[None, :, None]
    gsum = g3.sum(axis=(0, 2))
    dot = (g3 * yc).sum(axis=(0, 2))
    norm = 1.0 / M
    inv_w = 1.0 / w
    proj_scale = dot * norm * inv_w * inv_w
    dx = (g3 - yc * proj_scale[None, :, None] - (gsum * norm)[None, :, None]) * (
        invstd * w)[None, :, None]
    return dx.reshape(np.shape(y)), dot * inv_w, gsum


# ------------------------------------------------------------------ softmax


def _view3(t, dim):
    t = np.asarray(t)
    dim = dim % t.ndim
    outer = int(np.prod(t.shape[:dim], dtype=np.int64))
    inner = int(np.prod(t.shape[dim + 1:], dtype=np.int64))
    return t.reshape(outer, t.shape[dim], inner)


def softmax_fwd(x, dim, dtype=np.float64):
    """softmax over `dim` (softmax.cpp:11-15). Pinned by: torch.softmax on CPU."""
    x3 = _view3(np.asarray(x, dtype=dtype), dim)
    e = np.exp(x3 - x3.max(axis=1, keepdims=True))
    return (e / e.sum(axis=1, keepdims=True)).reshape(np.shape(x))


def softmax_bwd(dy, y, dim, dtype=np.float64):
    """t = dy*y; dx = t - y*sum_dim(t) (softmax.cpp:17-33).

    Pinned by: torch.ops.aten._softmax_backward_data on CPU.
    """
    g3 = _view3(np.asarray(dy, dtype=dtype), dim)
    y3 = _view3(np.asarray(y, dtype=dtype), dim)
    t = g3 * y3
    return (t - y3 * t.sum(axis=1, keepdims=True)).reshape(np.shape(y))


def xent_bwd(logits, labels, scale=None, dtype=np.float64):
    """(softmax(logits, 1) - onehot(labels)) * scale, scale = 1/labels.size by default.

    The loss sits outside the reference's operator library (stock
    nn.CrossEntropyLoss, examples/imagenet.py:199,327).
    Pinned by: autograd of F.cross_entropy on CPU.
    """
    p = _view3(softmax_fwd(logits, 1, dtype), 1).copy()
    lab = np.asarray(labels).reshape(p.shape[0], p.shape[2])
    scale = 1.0 / lab.size if scale is None else scale
    o, i = np.meshgrid(np.arange(p.shape[0]), np.arange(p.shape[2]), indexing="ij")
    p[o, lab, i] -= 1.0
    return (p * scale).reshape(np.shape(logits))


# -------------------------------------------------------------- convolution


def _conv_geo(x_shape, w_shape, stride, padding, dilation):
    N, C, H, W = x_shape
    K, C2, R, S = w_shape
    assert C == C2, "groups == 1 only"
    sH, sW = _pair(stride)
    pH, pW = _pair(padding)
    dH, dW = _pair(dilation)
    P = (H + 2 * pH - dH * (R - 1) - 1) // sH + 1
    Q = (W + 2 * pW - dW * (S - 1) - 1) // sW + 1
    return (N, C, H, W, K, R, S, sH, sW, pH, pW, dH, dW, P, Q)


def conv_fwd(x, w, bias=None, stride=1, padding=0, dilation=1, dtype=np.float64):
    """y[n,k,p,q] = sum_{c,r,s} w[k,c,r,s] * x[n,c,p*sH+r*dH-pH,q*sW+s*dW-pW] (+ bias[k]).

    What cudnnConvolutionForward computes for cudnn_convolution
    (monet/lm_ops/conv.cpp:299-340) with CUDNN_CROSS_CORRELATION, plus the bias
    add of conv.py:284-285.  Pinned by: F.conv2d on CPU in float64.
    """
    x = np.asarray(x, dtype=dtype)
    w = np.asarray(w, dtype=dtype)
    N, C, H, W, K, R, S, sH, sW, pH, pW, dH, dW, P, Q = _conv_geo(x.shape, w.shape, stride,
                                                                  padding, dilation)
    xp = np.zeros((N, C, H + 2 * pH, W + 2 * pW), dtype=dtype)
    xp[:, :, pH:pH + H, pW:pW + W] = x
    y = np.zeros((N, K, P, Q), dtype=dtype)
    for r in range(R):
        for s in range(S):
            patch = xp[:, :, r * dH:r * dH + (P - 1) * sH + 1:sH, s * dW:s * dW + (Q - 1) * sW + 1:sW]
            y += np.einsum("ncpq,kc->nkpq", patch, w[:, :, r, s], optimize=True)
    if bias is not None:
        y += np.asarray(bias, dtype=dtype)[None, :, None, None]
    return y


def conv_bwd_data(dy, w, x_shape, stride=1, padding=0, dilation=1, dtype=np.float64):
    """dx: every output gradient is spread back over the taps that produced it
    (cudnnConvolutionBackwardData, conv.cpp:409-449).
    Pinned by: aten.convolution_backward on CPU in float64."""
    dy = np.asarray(dy, dtype=dtype)
    w = np.asarray(w, dtype=dtype)
    N, C, H, W, K, R, S, sH, sW, pH, pW, dH, dW, P, Q = _conv_geo(x_shape, w.shape, stride,
                                                                  padding, dilation)
    dxp = np.zeros((N, C, H + 2 * pH, W + 2 * pW), dtype=dtype)
    for r in range(R):
        for s in range(S):
            dxp[:, :, r * dH:r * dH + (P - 1) * sH + 1:sH,
                s * dW:s * dW + (Q - 1) * sW + 1:sW] += np.einsum("nkpq,kc->ncpq", dy,
                                                                 w[:, :, r, s], optimize=True)
    return dxp[:, :, pH:pH + H, pW:pW + W]


def conv_bwd_weight(dy, x, w_shape, stride=1, padding=0, dilation=1, dtype=np.float64):
    """dw[k,c,r,s] = sum_{n,p,q} dy[n,k,p,q] * x[n,c,p*sH+r*dH-pH,q*sW+s*dW-pW]
    (cudnnConvolutionBackwardFilter, conv.cpp:550-591).
    Pinned by: aten.convolution_backward on CPU in float64."""
    dy = np.asarray(dy, dtype=dtype)
    x = np.asarray(x, dtype=dtype)
    N, C, H, W, K, R, S, sH, sW, pH, pW, dH, dW, P, Q = _conv_geo(x.shape, w_shape, stride,
                                                                  padding, dilation)
    xp = np.zeros((N, C, H + 2 * pH, W + 2 * pW), dtype=dtype)
    xp[:, :, pH:pH + H, pW:pW + W] = x
    dw = np.zeros((K, C, R, S), dtype=dtype)
    for r in range(R):
        for s in range(S):
            patch = xp[:, :, r * dH:r * dH + (P - 1) * sH + 1:sH, s * dW:s * dW + (Q - 1) * sW + 1:sW]
            dw[:, :, r, s] = np.einsum("nkpq,ncpq->kc", dy, patch, optimize=True)
    return dw
