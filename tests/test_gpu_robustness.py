"""What must hold when things go wrong or are done twice: a BatchNorm workgroup whose wait for
the other workgroups of its channel gives up reports it (NaN results, a raised error word)
instead of returning wrong numbers, and a forward that a schedule recomputes reproduces the
first forward bit for bit, also where the convolution splits its reduction."""
import numpy as np
import pytest
import torch

from monet_amd import _lib
from monet_amd.lm_ops import bn as bn_ops
from monet_amd.lm_ops import conv as conv_ops
from monet_amd.lm_ops import relu as relu_ops

pytestmark = pytest.mark.gpu


def _bn_case(cuda, N, C, H, W, seed=0):
    g = torch.Generator(device=cuda).manual_seed(seed)
    x = torch.randn(N, C, H, W, device=cuda, generator=g)
    gamma = torch.rand(C, device=cuda, generator=g) + 0.5
    beta = torch.randn(C, device=cuda, generator=g) * 0.1
    y, mean, invstd = bn_ops.bn_forward_train(x, gamma, beta, None, None, 0.1, 1e-5)
    dy = torch.randn(N, C, H, W, device=cuda, generator=g)
    return y, gamma, beta, invstd, dy


def _from_y_with_limits(y, gamma, beta, invstd, dy, ws, spin_limit, max_workgroups):
    N, C = y.shape[:2]
    HW = y.numel() // (N * C)
    dx = torch.empty_like(y)
    dg = torch.empty(C, device=y.device)
    db = torch.empty(C, device=y.device)
    _lib.call("mn_bn_bwd_from_y_f32_limits", _lib.ptr(dy), _lib.ptr(y), _lib.ptr(gamma),
              _lib.ptr(beta), _lib.ptr(invstd), _lib.ptr(dx), _lib.ptr(dg), _lib.ptr(db), N, C, HW,
              _lib.ptr(ws), ws.numel(), spin_limit, max_workgroups, 0, 0, _lib.stream_ptr(y.device))
    return dx, dg, db


def test_batchnorm_wait_that_gives_up_is_reported(cuda):
    """Each channel here is 13 register-resident pieces; with only two workgroups in the grid
    and a wait bound of a few polls, the first holders of every channel give up waiting for
    pieces nobody has loaded yet.  Every workgroup still runs to its end (the kernel returns);
    what was computed from the missing totals is NaN, and the workspace says so."""
    N, C, H, W = 32, 4, 56, 56
    y, gamma, beta, invstd, dy = _bn_case(cuda, N, C, H, W)
    HW = H * W
    nbytes = _lib.load().mn_bn_ws_bytes(N, C, HW)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=cuda)
    status = lambda: _lib.load().mn_bn_ws_status(_lib.ptr(ws), nbytes, N, C, HW,
                                                 _lib.stream_ptr(cuda))
    # the device's own word (for callers whose workspace is gone after the call): clear so far
    device_word = lambda: _lib.load().mn_bn_wait_status(None, _lib.stream_ptr(cuda))
    assert device_word() == _lib.MN_OK
    # default limits: everything arrives
    dx0, dg0, db0 = _from_y_with_limits(y, gamma, beta, invstd, dy, ws, 0, 0)
    assert status() == _lib.MN_OK and device_word() == _lib.MN_OK
    ref = bn_ops.bn_backward_from_output(dy, y, gamma, beta, invstd)
    assert torch.equal(dx0, ref[0]) and torch.equal(dg0, ref[1]) and torch.equal(db0, ref[2])
    # two workgroups, eight polls: the wait gives up
    dx1, dg1, db1 = _from_y_with_limits(y, gamma, beta, invstd, dy, ws, 8, 2)
    torch.cuda.synchronize()     # the launch has ended: nobody hangs
    assert status() == _lib.MN_ELAUNCH
    assert bool(torch.isnan(dg1).all()) and bool(torch.isnan(db1).all())
    assert bool(torch.isnan(dx1).any())
    with pytest.raises(_lib.MonetHipError) as info:
        _lib.call("mn_bn_ws_status", _lib.ptr(ws), nbytes, N, C, HW, _lib.stream_ptr(cuda))
    assert info.value.status == _lib.MN_ELAUNCH
    # the next launch on the same workspace starts clean
    dx2, dg2, db2 = _from_y_with_limits(y, gamma, beta, invstd, dy, ws, 0, 0)
    assert status() == _lib.MN_OK
    # ... while the device's word stays raised until it is asked for: the executor's monitor
    # (one non-blocking poll per step) raises on the poll after the one that fetched it
    bn_ops.poll_waits(cuda)
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="gave up waiting"):
        bn_ops.poll_waits(cuda)
    assert device_word() == _lib.MN_OK          # cleared by the monitor
    bn_ops.poll_waits(cuda)
    torch.cuda.synchronize()
    bn_ops.poll_waits(cuda)                     # and quiet again
    # the entry point with the library's own array answers the same question with ws == NULL
    _lib.call("mn_bn_bwd_from_y_static_f32", _lib.ptr(dy), _lib.ptr(y), _lib.ptr(gamma),
              _lib.ptr(beta), _lib.ptr(invstd), _lib.ptr(dx2), _lib.ptr(dg2), _lib.ptr(db2), N, C, HW,
              _lib.stream_ptr(cuda))
    assert _lib.load().mn_bn_ws_status(None, 0, N, C, HW, _lib.stream_ptr(cuda)) == _lib.MN_OK
    assert torch.equal(dx2, dx0) and torch.equal(dg2, dg0)
    assert torch.equal(dx2, dx0) and torch.equal(dg2, dg0) and torch.equal(db2, db0)
    # the operator classes check after every call when asked to
    bn_ops.check_waits = True
    try:
        again = bn_ops.bn_backward_from_output(dy, y, gamma, beta, invstd)
    finally:
        bn_ops.check_waits = False
    assert torch.equal(again[0], dx0)
    # formulations without a cross-workgroup wait leave the word clear as well
    for shape in ((8, 16, 14, 14), (3, 5, 7, 7)):
        ys, gs, bs, inv, dys = _bn_case(cuda, *shape, seed=1)
        n, c = shape[:2]
        hw = shape[2] * shape[3]
        nb = _lib.load().mn_bn_ws_bytes(n, c, hw)
        w2 = torch.full((nb,), 0xFF, dtype=torch.uint8, device=cuda)   # a dirty workspace
        _from_y_with_limits(ys, gs, bs, inv, dys, w2, 0, 0)
        assert _lib.load().mn_bn_ws_status(_lib.ptr(w2), nb, n, c, hw,
                                           _lib.stream_ptr(cuda)) == _lib.MN_OK


# shapes whose variant-1 forward splits its reduction (few, long workgroups): the 3x3 and the
# reducing 1x1 convolutions of ResNet-50's last two stages at batch 184, and a small one
SPLIT_SHAPES = [
    ((184, 256, 14, 14), (256, 256, 3, 3), 1, 1),
    ((184, 1024, 14, 14), (256, 1024, 1, 1), 1, 0),
    ((184, 512, 7, 7), (512, 512, 3, 3), 1, 1),
    ((184, 2048, 7, 7), (512, 2048, 1, 1), 1, 0),
    ((16, 512, 7, 7), (64, 512, 3, 3), 1, 1),
]


@pytest.mark.parametrize("xs,ws,stride,pad", SPLIT_SHAPES)
def test_recomputed_forward_reproduces_masks_bit_for_bit(cuda, xs, ws, stride, pad):
    """conv (every variant) -> BatchNorm -> ReLU with a 1-bit mask, run five times: outputs,
    statistics and masks must be identical each time, as a schedule that recomputes the chain
    in the backward pass relies on."""
    g = torch.Generator(device=cuda).manual_seed(5)
    x = torch.randn(xs, device=cuda, generator=g)
    w = torch.randn(ws, device=cuda, generator=g) * (2.0 / (ws[0] * ws[2] * ws[3])) ** 0.5
    gamma = torch.rand(ws[0], device=cuda, generator=g) + 0.5
    beta = torch.randn(ws[0], device=cuda, generator=g) * 0.1
    for v in range(conv_ops.n_fwd_algos()):
        if v in (2, 3) and ws[2] != 3:
            continue   # the Winograd variants are for 3x3 filters
        if v == 4 and not (ws[2] == 1 and stride == 1 and pad == 0 and (xs[2] * xs[3]) % 4 == 0):
            continue   # the three-slice variant is for 1x1 filters on planes of whole float4
        first = None
        for rep in range(5):
            y = conv_ops.conv_forward(x, w, None, pad, stride, 1, 1, v)
            z, mean, invstd = bn_ops.bn_forward_train(y, gamma, beta, None, None, 0.1, 1e-5)
            a, mask = relu_ops.relu_forward_with_mask(z)
            got = (y, mean, invstd, a, mask)
            if first is None:
                first = got
            else:
                for k, (p, q) in enumerate(zip(first, got)):
                    assert torch.equal(p, q), (v, rep, k)
            # the recomputation path proper: saved statistics re-applied
            z2 = bn_ops.bn_forward_apply(y, mean, invstd, gamma, beta)
            assert torch.equal(relu_ops.relu_forward_with_mask(z2)[1], first[4]), (v, rep)
