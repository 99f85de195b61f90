"""The BatchNorm backward from the output through the entry point that allocates nothing
(its workspace is a fixed array inside the library) against the entry point that takes a
caller workspace: same kernels, so the results must be identical, on two calls in a row of
which the second is smaller (the array keeps the first call's contents)."""
import pytest
import torch

from monet_amd import _lib

pytestmark = pytest.mark.gpu


def _inputs(cuda, N, C, H, W, seed):
    from monet_amd.lm_ops import bn as bn_ops
    g = torch.Generator(device=cuda).manual_seed(seed)
    x = torch.randn(N, C, H, W, device=cuda, generator=g)
    gamma = torch.rand(C, device=cuda, generator=g) + 0.5
    beta = torch.randn(C, device=cuda, generator=g) * 0.1
    y, _, invstd = bn_ops.bn_forward_train(x, gamma, beta, None, None, 0.1, 1e-5)
    dy = torch.randn(N, C, H, W, device=cuda, generator=g)
    return dy, y, gamma, beta, invstd


def _outputs(y):
    C = y.shape[1]
    return (torch.full_like(y, float("nan")), torch.full((C,), float("nan"), device=y.device),
            torch.full((C,), float("nan"), device=y.device))


def _with_workspace(dy, y, gamma, beta, invstd):
    N, C = y.shape[:2]
    HW = y.numel() // (N * C)
    nbytes = _lib.load().mn_bn_ws_bytes(N, C, HW)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=y.device)
    dx, dg, db = _outputs(y)
    _lib.call("mn_bn_bwd_from_y_f32", _lib.ptr(dy), _lib.ptr(y), _lib.ptr(gamma), _lib.ptr(beta),
              _lib.ptr(invstd), _lib.ptr(dx), _lib.ptr(dg), _lib.ptr(db), N, C, HW, _lib.ptr(ws),
              nbytes, _lib.stream_ptr(y.device))
    return dx, dg, db


def _static(dy, y, gamma, beta, invstd):
    N, C = y.shape[:2]
    HW = y.numel() // (N * C)
    dx, dg, db = _outputs(y)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    _lib.call("mn_bn_bwd_from_y_static_f32", _lib.ptr(dy), _lib.ptr(y), _lib.ptr(gamma),
              _lib.ptr(beta), _lib.ptr(invstd), _lib.ptr(dx), _lib.ptr(dg), _lib.ptr(db), N, C, HW,
              _lib.stream_ptr(y.device))
    torch.cuda.synchronize()
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == before
    return dx, dg, db


# each pair: a larger call, then a smaller one that finds the larger one's leftovers.  The
# shapes cover the one-pass kernel with 256- and 512-thread workgroups, whole channels in one
# workgroup, the scalar path (HW not a multiple of 4) and the two-launch formulation.
PAIRS = [
    ((64, 64, 56, 56), (16, 32, 56, 56)),
    ((184, 8, 112, 112), (48, 8, 112, 112)),
    ((184, 64, 14, 14), (32, 16, 7, 7)),
    ((16, 24, 31, 29), (16, 8, 15, 15)),
    ((4, 2, 1024, 1280), (1, 2, 1024, 1280)),
]


@pytest.mark.parametrize("big,small", PAIRS)
def test_static_workspace_entry_point_matches_the_workspace_one(cuda, big, small):
    for k, shape in enumerate((big, small)):
        args = _inputs(cuda, *shape, seed=7 + k)
        want = _with_workspace(*args)
        got = _static(*args)
        for name, a, b in zip(("dx", "dgamma", "dbeta"), got, want):
            assert bool(torch.isfinite(b).all()), (shape, name)
            assert torch.equal(a, b), (shape, name)


def test_static_workspace_entry_point_refuses_what_does_not_fit(cuda):
    # 10000 channels need more room for partial sums than the fixed array holds
    N, C, HW = 64, 10000, 56 * 56
    assert _lib.load().mn_bn_ws_bytes(N, C, HW) > 4 << 20
    one = torch.ones(1, device=cuda)
    with pytest.raises(_lib.MonetHipError) as info:
        _lib.call("mn_bn_bwd_from_y_static_f32", _lib.ptr(one), _lib.ptr(one), _lib.ptr(one),
                  _lib.ptr(one), _lib.ptr(one), _lib.ptr(one), _lib.ptr(one), _lib.ptr(one), N, C,
                  HW, _lib.stream_ptr(cuda))
    assert info.value.status == _lib.MN_ELIMIT
    # empty tensors are fine and touch nothing
    assert _lib.load().mn_bn_bwd_from_y_static_f32(None, None, None, None, None, None, None, None,
                                                   0, 8, 49, _lib.stream_ptr(cuda)) == _lib.MN_OK
