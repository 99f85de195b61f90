"""GPU parity of the convolution kernels (all directions, all variants) against
the float64 CPU oracle, through the operator classes and the C ABI."""
import numpy as np
import pytest
import torch

import monet_amd.lm_ops as lm_ops
from monet_amd.lm_ops import conv as conv_ops
from oracle import lm_oracle as O

pytestmark = pytest.mark.gpu

# fp32 matrix-core accumulation against a float64 oracle: error relative to the largest
# magnitude of the expected tensor
TOL = 1e-5

CASES = [
    # (x shape, w shape, stride, padding, dilation)
    ((2, 3, 9, 9), (4, 3, 3, 3), 1, 1, 1),
    ((1, 5, 12, 10), (7, 5, 3, 3), 2, 1, 1),
    ((2, 4, 8, 8), (6, 4, 1, 1), 1, 0, 1),
    ((2, 4, 9, 9), (6, 4, 1, 1), 2, 0, 1),
    ((1, 3, 15, 15), (8, 3, 7, 7), 2, 3, 1),
    ((1, 2, 11, 11), (3, 2, 3, 3), 1, 2, 2),
    ((2, 3, 7, 9), (2, 3, 2, 3), (2, 1), (1, 0), 1),
    ((3, 130, 14, 14), (140, 130, 3, 3), 1, 1, 1),     # tiles with ragged edges in every dimension
    ((4, 256, 14, 14), (256, 256, 3, 3), 1, 1, 1),     # ResNet-50 layer3 shape at a small batch
    ((2, 64, 56, 56), (256, 64, 1, 1), 1, 0, 1),       # 1x1 expansion
    ((2, 128, 28, 28), (128, 128, 3, 3), 2, 1, 1),     # strided 3x3
    ((2, 256, 28, 28), (512, 256, 1, 1), 2, 0, 1),     # strided 1x1 (downsample)
    ((2, 3, 64, 64), (64, 3, 7, 7), 2, 3, 1),          # stem (forward variant 1: the kernel of its own)
    ((1, 16, 33, 47), (24, 16, 3, 3), 1, 1, 1),        # odd spatial sizes
    ((5, 128, 7, 7), (128, 128, 3, 3), 1, 1, 1),       # 49-pixel images: no 16-byte alignment along the depth
    ((5, 128, 7, 7), (256, 128, 1, 1), 1, 0, 1),       # the same, 1x1
    ((3, 64, 9, 11), (64, 64, 3, 3), 1, 1, 1),         # 99 pixels, 64-channel tiles
    ((2, 32, 13, 17), (48, 32, 3, 3), 2, (2, 1), 2),   # tap-major path with stride, dilation, uneven padding
    ((2, 64, 12, 12), (64, 64, 5, 5), 1, 2, 1),        # 25 taps, windows hanging over every border
    ((1, 128, 6, 10), (128, 128, 3, 3), (1, 2), (1, 0), (1, 1)),  # stride on one axis only
    ((2, 32, 10, 9), (40, 32, 3, 3), 1, 0, 1),         # 3x3 without padding (Winograd: backward pads by 2)
    ((2, 16, 6, 7), (16, 16, 3, 3), 1, 2, 1),          # 3x3 padded by 2: output larger than the input
    ((2, 20, 11, 13), (48, 20, 3, 3), 1, 1, 1),        # Winograd backward-data only (K % 16 == 0, C is not)
    ((3, 48, 5, 5), (32, 48, 3, 3), 1, 1, 1),          # odd planes: ragged 2x2 output tiles
    ((3, 96, 10, 10), (48, 96, 1, 1), 1, 0, 1),        # 1x1: 48 output channels in a 64-wide tile, pixel tiles across images
    ((5, 256, 14, 14), (320, 256, 1, 1), 1, 0, 1),     # 1x1: 256-channel tiles with a ragged second one
    ((2, 144, 12, 12), (128, 144, 1, 1), 1, 0, 1),     # 1x1: nine 16-deep stages (an odd number)
    # the stem again at odd sizes: forward variant 1 (the kernel of its own) stages scalars and
    # has ragged row blocks
    ((3, 3, 75, 97), (64, 3, 7, 7), 2, 3, 1),
    # backward-weight variant 3 (Winograd in one kernel): 64-channel blocks, W % 4 == 0; one and
    # several chunks per tile row, ranges of one tile row (padded to four chunks), uneven ranges
    ((2, 64, 16, 16), (64, 64, 3, 3), 1, 1, 1),
    ((3, 128, 24, 32), (64, 128, 3, 3), 1, 1, 1),
    ((1, 64, 6, 8), (128, 64, 3, 3), 1, 1, 1),
    ((37, 64, 18, 24), (64, 64, 3, 3), 1, 1, 1),       # 333 tile rows over 256 ranges
    # the stem's backward-weight kernel (variant 1): 112 output columns (the group count the kernel
    # is specialised for) with a ragged last row block; more items than workgroups
    ((2, 3, 42, 224), (64, 3, 7, 7), 2, 3, 1),
    ((150, 3, 32, 32), (64, 3, 7, 7), 2, 3, 1),
    # backward-weight variant 3 with a ragged last chunk (14 and 22 tiles per row) and rows that
    # need one group and two
    ((3, 64, 10, 28), (64, 64, 3, 3), 1, 1, 1),
    ((2, 64, 6, 44), (128, 64, 3, 3), 1, 1, 1),
]


def winograd_applies(ws, st, pad, dil, reduced_channels):
    """Variants 2 and 3 (Winograd F(2x2, 3x3), through transformed tensors in the workspace /
    in one kernel) cover 3x3 filters, stride 1, dilation 1, equal
    padding <= 2 on both axes and a reduction over a multiple of 16 channels; anything else
    must be refused with MN_EUNSUPPORTED."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    return (ws[2] == 3 and ws[3] == 3 and pair(st) == (1, 1) and pair(dil) == (1, 1) and
            pair(pad)[0] == pair(pad)[1] and pair(pad)[0] <= 2 and reduced_channels % 16 == 0)


def winograd_wgrad_applies(xs, ws, st, pad, dil):
    """Variant 2 of backward-weight: 3x3, stride 1, dilation 1, equal padding <= 2, C % 4 == 0."""
    return winograd_applies(ws, st, pad, dil, 16) and xs[1] % 4 == 0


def fused_winograd_wgrad_applies(xs, ws, st, pad, dil):
    """Variant 3 of backward-weight (Winograd in one kernel): 3x3, stride 1, dilation 1, padding 1,
    even height, W % 4 == 0, K and C multiples of 64."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    return (winograd_applies(ws, st, pad, dil, 16) and pair(pad) == (1, 1) and xs[2] % 2 == 0 and
            xs[3] % 4 == 0 and xs[1] % 64 == 0 and ws[0] % 64 == 0)


def split_applies(xs, ws, st, pad, dil, reduced_channels):
    """Variant 4 of forward and backward-data (fp32 through three bf16 slices per operand on the
    bf16 matrix cores): 1x1 filters, stride 1, no padding, planes of a multiple of 4 pixels and
    a reduction over a multiple of 16 channels; anything else is refused."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    return (ws[2] == 1 and ws[3] == 1 and pair(st) == (1, 1) and pair(pad) == (0, 0) and
            (xs[2] * xs[3]) % 4 == 0 and reduced_channels % 16 == 0)


def refused(call):
    from monet_amd import _lib
    with pytest.raises(_lib.MonetHipError) as e:
        call()
    assert e.value.status == _lib.MN_EUNSUPPORTED
    return True


def dev(a, cuda):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(cuda)


def host(t):
    return t.detach().cpu().numpy()


def assert_rel(got, exp, tol, what):
    exp = np.asarray(exp, np.float64)
    err = np.abs(np.asarray(got, np.float64) - exp).max()
    scale = max(np.abs(exp).max(), 1e-30)
    # what was achieved, for whoever reads the log (pytest -s): tolerances are set from these
    print(f"achieved {what}: {err / scale:.2e} of scale (tolerance {tol:.0e})")
    assert err <= tol * scale, f"{what}: max err {err:.3e} vs scale {scale:.3e} ({err / scale:.2e})"


def problem(xs, ws, seed=0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(xs).astype(np.float32)
    fan_out = ws[0] * ws[2] * ws[3]
    w = (rng.standard_normal(ws) * np.sqrt(2.0 / fan_out)).astype(np.float32)
    b = rng.standard_normal(ws[0]).astype(np.float32)
    return x, w, b


@pytest.mark.parametrize("xs,ws,st,pad,dil", CASES)
def test_conv_forward(cuda, xs, ws, st, pad, dil):
    x, w, b = problem(xs, ws)
    exp = O.conv_fwd(x, w, b, st, pad, dil)
    exp_nobias = O.conv_fwd(x, w, None, st, pad, dil)
    assert conv_ops.n_fwd_algos() == 5
    for v in range(conv_ops.n_fwd_algos()):
        if (v in (2, 3) and not winograd_applies(ws, st, pad, dil, xs[1])) or \
                (v == 4 and not split_applies(xs, ws, st, pad, dil, xs[1])):
            assert refused(lambda: conv_ops.conv_forward(dev(x, cuda), dev(w, cuda), None, pad, st,
                                                         dil, 1, v))
            continue
        y = conv_ops.conv_forward(dev(x, cuda), dev(w, cuda), dev(b, cuda), pad, st, dil, 1, v)
        assert list(y.shape) == list(exp.shape)
        assert_rel(host(y), exp, TOL, f"forward variant {v}")
        y = conv_ops.conv_forward(dev(x, cuda), dev(w, cuda), None, pad, st, dil, 1, v)
        assert_rel(host(y), exp_nobias, TOL, f"forward variant {v} (no bias)")


@pytest.mark.parametrize("xs,ws,st,pad,dil", CASES)
def test_conv_backward_data(cuda, xs, ws, st, pad, dil):
    x, w, _ = problem(xs, ws, 1)
    yshape = O.conv_fwd(x, w, None, st, pad, dil).shape
    dy = np.random.default_rng(2).standard_normal(yshape).astype(np.float32)
    exp = O.conv_bwd_data(dy, w, xs, st, pad, dil)
    assert conv_ops.n_bwd_ip_algos() == 5
    for v in range(conv_ops.n_bwd_ip_algos()):
        if (v in (2, 3) and not winograd_applies(ws, st, pad, dil, ws[0])) or \
                (v == 4 and not split_applies(xs, ws, st, pad, dil, ws[0])):
            assert refused(lambda: conv_ops.conv_backward_input(xs, dev(dy, cuda), dev(w, cuda),
                                                                pad, st, dil, 1, v))
            continue
        dx = conv_ops.conv_backward_input(xs, dev(dy, cuda), dev(w, cuda), pad, st, dil, 1, v)
        assert_rel(host(dx), exp, TOL, f"backward-data variant {v}")


@pytest.mark.parametrize("xs,ws,st,pad,dil", CASES)
def test_conv_backward_weight(cuda, xs, ws, st, pad, dil):
    x, w, _ = problem(xs, ws, 3)
    yshape = O.conv_fwd(x, w, None, st, pad, dil).shape
    dy = np.random.default_rng(4).standard_normal(yshape).astype(np.float32)
    exp = O.conv_bwd_weight(dy, x, ws, st, pad, dil)
    outs = []
    assert conv_ops.n_bwd_wt_algos() == 4
    for v in range(conv_ops.n_bwd_wt_algos()):
        if (v == 2 and not winograd_wgrad_applies(xs, ws, st, pad, dil)) or \
                (v == 3 and not fused_winograd_wgrad_applies(xs, ws, st, pad, dil)):
            assert refused(lambda: conv_ops.conv_backward_weight(ws, dev(dy, cuda), dev(x, cuda),
                                                                 pad, st, dil, 1, v))
            continue
        dw = conv_ops.conv_backward_weight(ws, dev(dy, cuda), dev(x, cuda), pad, st, dil, 1, v)
        assert_rel(host(dw), exp, TOL, f"backward-weight variant {v}")
        outs.append(dw)
        if v >= 2:   # partial results added in a fixed order: bit-identical run to run
            assert torch.equal(dw, conv_ops.conv_backward_weight(ws, dev(dy, cuda), dev(x, cuda), pad,
                                                                 st, dil, 1, v))
    # the workspace variant sums its partials in a fixed order: bit-identical run to run
    again = conv_ops.conv_backward_weight(ws, dev(dy, cuda), dev(x, cuda), pad, st, dil, 1, 1)
    assert torch.equal(again, outs[1])


def test_conv_op_classes_follow_the_algorithm_encoding(cuda):
    xs, ws = (2, 8, 10, 10), (12, 8, 3, 3)
    x, w, b = problem(xs, ws, 5)
    tx = dev(x, cuda).requires_grad_(True)
    tw = dev(w, cuda).requires_grad_(True)
    tb = dev(b, cuda).requires_grad_(True)
    args = (tx, tw, tb, [1, 1], [1, 1], [1, 1], False, [0, 0], 1, False, False, True, True)
    exp_y = O.conv_fwd(x, w, b, 1, 1, 1)
    dy = np.random.default_rng(6).standard_normal(exp_y.shape).astype(np.float32)
    exp_dx = O.conv_bwd_data(dy, w, xs, 1, 1, 1)
    exp_dw = O.conv_bwd_weight(dy, x, ws, 1, 1, 1)
    for cls in (lm_ops.conv.SpecificAlgoConvolution, lm_ops.conv.GreedyAlgoConvolution):
        op = cls()
        op.algorithm = 0
        y = op.forward(*args)
        assert_rel(host(y), exp_y, TOL, "op forward")
        # timestep t-1: parameter gradients (kind 0); both stored tensors present
        op.algorithm = 0 * 10 + 1
        stored = [tx.detach(), tw.detach()]
        di, dw, db = op.backward(dev(dy, cuda), stored)
        assert stored == [] and di is None
        assert_rel(host(dw), exp_dw, TOL, "op dw")
        assert_rel(host(db), dy.sum(axis=(0, 2, 3)), TOL, "op db")
        # timestep t: input gradient (kind 1); only the weight is guaranteed
        op.algorithm = 1 * 10 + 1
        di, dw, db = op.backward(dev(dy, cuda), [None, tw.detach()], nodel=True)
        assert dw is None
        assert_rel(host(di), exp_dx, TOL, "op dx")
        # kind 2: everything at once, no bias -> 2-tuple
        op2 = cls()
        op2.algorithm = 0
        op2.forward(tx, tw, None, [1, 1], [1, 1], [1, 1], False, [0, 0], 1)
        op2.algorithm = 20
        out = op2.backward(dev(dy, cuda), [tx.detach(), tw.detach()])
        assert len(out) == 2
        assert_rel(host(out[0]), exp_dx, TOL, "op2 dx")
        assert_rel(host(out[1]), exp_dw, TOL, "op2 dw")


def test_conv_unsupported_variant_falls_back(cuda):
    xs, ws = (1, 4, 6, 6), (4, 4, 3, 3)
    x, w, _ = problem(xs, ws, 7)
    with pytest.raises(RuntimeError, match="unsupported"):
        conv_ops.conv_forward(dev(x, cuda), dev(w, cuda), None, 1, 1, 1, 1, 7)
    op = lm_ops.conv.SpecificAlgoConvolution()
    op.algorithm = 7
    y = op.forward(dev(x, cuda).requires_grad_(True), dev(w, cuda), None, [1, 1], [1, 1], [1, 1],
                   False, [0, 0], 1)
    assert op.algorithm == 0
    assert_rel(host(y), O.conv_fwd(x, w, None, 1, 1, 1), TOL, "fallback forward")
    op.algorithm = 19
    di, dw = op.backward(torch.ones_like(y), [None, dev(w, cuda)], nodel=True)
    assert op.algorithm == 10 and di is not None


def test_depthwise_passthrough(cuda):
    x = torch.randn(2, 6, 9, 9, device=cuda, requires_grad=True)
    w = torch.randn(6, 1, 3, 3, device=cuda, requires_grad=True)
    op = lm_ops.conv.SpecificAlgoConvolution()
    op.is_depthwise = True
    y = op.forward(x, w, None, [1, 1], [1, 1], [1, 1], False, [0, 0], 6)
    ref = torch.nn.functional.conv2d(x, w, None, 1, 1, 1, 6)
    torch.testing.assert_close(y, ref)
    g = torch.randn_like(y)
    ref.backward(g)
    op.algorithm = 20
    di, dw = op.backward(g, [x.detach(), w.detach()])
    torch.testing.assert_close(di, x.grad)
    torch.testing.assert_close(dw, w.grad)


# ------------------------------------------------------------------ bf16 path
# bf16 channels-last tensors, bf16 matrix cores, fp32 accumulation: inputs are rounded to
# bf16 first and the float64 oracle runs on the ROUNDED values, so what is left is the
# accumulation order and the single rounding of the output: 2^-9 of the value at worst,
# checked at 1e-2 of the tensor's scale as the configuration states (a wrong operand layout
# or tap table gives errors of order 1).
BF16_TOL = 1e-2
BF16_CASES = [
    ((4, 64, 14, 14), (128, 64, 3, 3), 1, 1, 1),
    ((3, 128, 9, 11), (64, 128, 3, 3), 2, 1, 1),        # strided, odd sizes, ragged row tiles
    ((2, 64, 8, 8), (64, 64, 1, 1), 1, 0, 1),
    ((2, 64, 9, 9), (192, 64, 1, 1), 2, 0, 1),          # parity classes no tap reaches; K % 128 != 0
    ((1, 64, 11, 11), (64, 64, 3, 3), 1, 2, 2),         # dilation
    ((2, 128, 7, 9), (128, 128, 2, 3), (2, 1), (1, 0), 1),
    ((8, 256, 14, 14), (256, 256, 3, 3), 1, 1, 1),      # ResNet-50 layer3 shape at a small batch
    ((2, 64, 56, 56), (256, 64, 1, 1), 1, 0, 1),
    # more than 4096 positions and at least 128 output channels: the large-tile kernel (feeding
    # and multiplying wavefronts), 256- and 128-channel tiles, ragged in both directions
    ((24, 256, 14, 14), (256, 256, 3, 3), 1, 1, 1),
    ((80, 64, 15, 15), (192, 64, 3, 3), 2, 1, 1),
    ((23, 128, 14, 14), (128, 128, 5, 5), 1, 2, 1),
    ((34, 128, 12, 12), (320, 128, 1, 1), 1, 0, 1),
    # backward-weight variant 1 with feeding and multiplying wavefronts (both channel counts
    # multiples of 128, more than 4096 positions): 128 x 256 tiles, and strided with odd planes
    ((12, 256, 20, 20), (128, 256, 3, 3), 1, 1, 1),
    ((40, 128, 23, 21), (384, 128, 3, 3), 2, 1, 1),
]


def bf16_round(a):
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(torch.bfloat16).float().numpy()


def dev16(a, cuda):
    t = torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(cuda).to(torch.bfloat16)
    return t.contiguous(memory_format=torch.channels_last) if t.dim() == 4 else t


@pytest.mark.parametrize("xs,ws,st,pad,dil", BF16_CASES)
def test_conv_bf16_all_directions(cuda, xs, ws, st, pad, dil):
    x, w, b = problem(xs, ws, seed=3)
    x, w, b = bf16_round(x), bf16_round(w), bf16_round(b)
    exp = O.conv_fwd(x, w, b, st, pad, dil)
    rng = np.random.default_rng(5)
    dy = bf16_round(rng.standard_normal(exp.shape))
    assert conv_ops.n_fwd_algos(torch.bfloat16) == 2
    for v in (0, 1):    # weights read in place / packed in fragment order in the workspace
        y = conv_ops.conv_forward(dev16(x, cuda), dev16(w, cuda), dev16(b, cuda), pad, st, dil, 1, v)
        assert y.dtype == torch.bfloat16 and y.is_contiguous(memory_format=torch.channels_last)
        assert_rel(host(y.float()), exp, BF16_TOL, f"bf16 forward variant {v}")
    y = conv_ops.conv_forward(dev16(x, cuda), dev16(w, cuda), None, pad, st, dil, 1, 0)
    assert_rel(host(y.float()), O.conv_fwd(x, w, None, st, pad, dil), BF16_TOL, "bf16 forward, no bias")
    exp_dx = O.conv_bwd_data(dy, w, xs, st, pad, dil)
    for v in (0, 1):
        dx = conv_ops.conv_backward_input(xs, dev16(dy, cuda), dev16(w, cuda), pad, st, dil, 1, v)
        assert dx.dtype == torch.bfloat16 and list(dx.shape) == list(xs)
        assert_rel(host(dx.float()), exp_dx, BF16_TOL, f"bf16 backward-data variant {v}")
    exp_dw = O.conv_bwd_weight(dy, x, ws, st, pad, dil)
    for v in (0, 1):
        dw = conv_ops.conv_backward_weight(ws, dev16(dy, cuda), dev16(x, cuda), pad, st, dil, 1, v)
        assert dw.dtype == torch.bfloat16 and list(dw.shape) == list(ws)
        assert_rel(host(dw.float()), exp_dw, BF16_TOL, f"bf16 backward-weight variant {v}")
        # reproducible: fixed-order reduction of the split partials
        dw2 = conv_ops.conv_backward_weight(ws, dev16(dy, cuda), dev16(x, cuda), pad, st, dil, 1, v)
        assert torch.equal(dw, dw2)
    # there is no bf16 Winograd tier
    assert refused(lambda: conv_ops.conv_forward(dev16(x, cuda), dev16(w, cuda), None, pad, st, dil, 1, 2))


def test_conv_bf16_rejects_channel_counts_the_tiles_cannot_hold(cuda):
    from monet_amd import _lib
    x = torch.randn(1, 3, 8, 8, device=cuda).to(torch.bfloat16)
    w = torch.randn(64, 3, 3, 3, device=cuda).to(torch.bfloat16)
    with pytest.raises(_lib.MonetHipError) as e:
        conv_ops.conv_forward(x, w, None, 1, 1, 1, 1, 0)
    assert e.value.status == _lib.MN_EUNSUPPORTED
    with pytest.raises(RuntimeError):
        conv_ops.conv_forward(x, w.float(), None, 1, 1, 1, 1, 0)   # mixed dtypes


def test_conv_bf16_channel_counts_that_only_fit_the_shallow_tiles(cuda):
    """C = 96 and K = 32 are multiples of 32 but not 64: forward and backward-data stage
    32-deep tiles there; backward-weight needs multiples of 64 and must say so."""
    from monet_amd import _lib
    xs, ws, st, pad, dil = (2, 96, 10, 10), (32, 96, 3, 3), 1, 1, 1
    x, w, b = problem(xs, ws, seed=7)
    x, w = bf16_round(x), bf16_round(w)
    exp = O.conv_fwd(x, w, None, st, pad, dil)
    y = conv_ops.conv_forward(dev16(x, cuda), dev16(w, cuda), None, pad, st, dil, 1, 0)
    assert_rel(host(y.float()), exp, BF16_TOL, "bf16 forward, 32-deep tiles")
    dy = bf16_round(np.random.default_rng(8).standard_normal(exp.shape))
    dx = conv_ops.conv_backward_input(xs, dev16(dy, cuda), dev16(w, cuda), pad, st, dil, 1, 0)
    assert_rel(host(dx.float()), O.conv_bwd_data(dy, w, xs, st, pad, dil), BF16_TOL,
               "bf16 backward-data, 32-deep tiles")
    with pytest.raises(_lib.MonetHipError) as e:
        conv_ops.conv_backward_weight(ws, dev16(dy, cuda), dev16(x, cuda), pad, st, dil, 1, 0)
    assert e.value.status == _lib.MN_EUNSUPPORTED


@pytest.mark.parametrize("xs,ws,st,pad,dil", [CASES[8], CASES[10], CASES[11], CASES[1], CASES[9], CASES[25]])
def test_conv_backward_data_accumulates_into_an_existing_gradient(cuda, xs, ws, st, pad, dil):
    """dx += conv_backward_data(dy): every variant, dense and strided (parity-class) outputs,
    positions no tap reaches keep their value, split reductions add onto what is there."""
    x, w, _ = problem(xs, ws, seed=11)
    rng = np.random.default_rng(12)
    dy = rng.standard_normal(O.conv_fwd(x, w, None, st, pad, dil).shape).astype(np.float32)
    prior = rng.standard_normal(xs).astype(np.float32)
    exp = prior.astype(np.float64) + O.conv_bwd_data(dy, w, xs, st, pad, dil)
    for v in range(conv_ops.n_bwd_ip_algos()):
        if v in (2, 3) and not winograd_applies(ws, st, pad, dil, ws[0]):
            continue
        if v == 4 and not split_applies(xs, ws, st, pad, dil, ws[0]):
            continue
        acc = dev(prior, cuda)
        out = conv_ops.conv_backward_input(xs, dev(dy, cuda), dev(w, cuda), pad, st, dil, 1, v,
                                           accumulate_into=acc)
        assert out is acc
        assert_rel(host(acc), exp, TOL, f"accumulating backward-data variant {v}")


BIAS_GRAD_CASES = CASES + [
    ((1, 4, 5, 5), (6, 4, 3, 3), 1, 1, 1),             # one depth tile: a single plain store
    ((1, 64, 4, 4), (64, 64, 3, 3), 1, 1, 1),          # the same through the tap-major kernel
    ((1, 1024, 4, 4), (1024, 1024, 3, 3), 1, 1, 1),    # more output tiles than resident slots: no split
    ((2, 64, 40, 40), (64, 64, 3, 3), 1, 1, 1),        # UNet-like: bias, 64 channels, long reduction
]


@pytest.mark.parametrize("xs,ws,st,pad,dil", BIAS_GRAD_CASES)
def test_conv_backward_weight_with_bias_gradient(cuda, xs, ws, st, pad, dil):
    """db = sum of dy over (n, p, q), from the weight-gradient kernel itself: against the
    float64 sum, every variant; dw unchanged by the extra epilogue; variant 1 reproducible."""
    x, w, _ = problem(xs, ws, 21)
    yshape = O.conv_fwd(x, w, None, st, pad, dil).shape
    dy = np.random.default_rng(22).standard_normal(yshape).astype(np.float32)
    exp_dw = O.conv_bwd_weight(dy, x, ws, st, pad, dil)
    exp_db = dy.astype(np.float64).sum(axis=(0, 2, 3))
    # a sum of M unit-variance terms: tolerance relative to its typical size sqrt(M), not to
    # the largest of K sums
    scale_db = np.sqrt(dy.size / ws[0])
    for v in range(conv_ops.n_bwd_wt_algos()):
        if (v == 2 and not winograd_wgrad_applies(xs, ws, st, pad, dil)) or \
                (v == 3 and not fused_winograd_wgrad_applies(xs, ws, st, pad, dil)):
            continue
        alone = conv_ops.conv_backward_weight(ws, dev(dy, cuda), dev(x, cuda), pad, st, dil, 1, v)
        dw, db = conv_ops.conv_backward_weight(ws, dev(dy, cuda), dev(x, cuda), pad, st, dil, 1, v,
                                               with_bias_grad=True)
        assert_rel(host(dw), exp_dw, TOL, f"dw with bias gradient, variant {v}")
        assert list(db.shape) == [ws[0]]
        err = np.abs(host(db).astype(np.float64) - exp_db).max()
        assert err <= TOL * scale_db, f"db variant {v}: {err:.3e} vs {scale_db:.3e}"
        if v >= 1:
            assert torch.equal(dw, alone)
            dw2, db2 = conv_ops.conv_backward_weight(ws, dev(dy, cuda), dev(x, cuda), pad, st, dil,
                                                     1, v, with_bias_grad=True)
            assert torch.equal(db, db2) and torch.equal(dw, dw2)


def test_conv_bias_gradient_entry_point_rejects_bf16_and_null(cuda):
    from monet_amd import _lib
    geo = conv_ops.conv_geometry((2, 64, 8, 8), (64, 64, 3, 3), 1, 1, 1, 1)
    buf = torch.zeros(64 * 64 * 9, device=cuda)
    with pytest.raises(_lib.MonetHipError) as e:
        _lib.call("mn_conv_bwd_weight_bias", geo, _lib.ptr(buf), _lib.ptr(buf), _lib.ptr(buf),
                  _lib.ptr(buf), None, 0, 0, _lib.BF16, _lib.stream_ptr(buf.device))
    assert e.value.status == _lib.MN_EUNSUPPORTED
    with pytest.raises(_lib.MonetHipError) as e:
        _lib.call("mn_conv_bwd_weight_bias", geo, _lib.ptr(buf), _lib.ptr(buf), _lib.ptr(buf),
                  None, None, 0, 0, _lib.F32, _lib.stream_ptr(buf.device))
    assert e.value.status == _lib.MN_EINVAL


def test_winograd_runs_slice_after_slice_when_its_buffers_would_pass_512_MB(cuda):
    """Variant 2 keeps its transformed tensors under 512 MB: a larger problem is cut into
    ranges of tiles that run one after the other through the same buffers (forward and
    backward-data), or into passes whose results are added in order (backward-weight).
    [4, 256, 161, 159] -> 256 channels is 25 920 tiles of 32 KB = two slices, the second one
    shorter, with ragged tiles at the right and bottom edges.  Checked against float64 on
    sampled output elements and against variant 1 everywhere."""
    xs, ws, pad = (4, 256, 161, 159), (256, 256, 3, 3), 1
    rng = np.random.default_rng(5)
    x, w, b = problem(xs, ws, 7)
    dy = rng.standard_normal((xs[0], ws[0], xs[2], xs[3])).astype(np.float32)
    xd, wd, bd, dyd = dev(x, cuda), dev(w, cuda), dev(b, cuda), dev(dy, cuda)
    xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (1, 1), (1, 1)))
    dyp = np.pad(dy.astype(np.float64), ((0, 0), (0, 0), (1, 1), (1, 1)))
    w64 = w.astype(np.float64)

    y1 = conv_ops.conv_forward(xd, wd, bd, pad, 1, 1, 1, 1)
    idx = [(rng.integers(xs[0]), rng.integers(ws[0]), rng.integers(xs[2]), rng.integers(xs[3]))
           for _ in range(256)] + [(3, 255, 160, 158), (0, 0, 0, 0), (2, 17, 160, 0)]
    exp = np.array([(xp[n, :, h:h + 3, q:q + 3] * w64[k]).sum() + b[k] for n, k, h, q in idx])
    for v in (2, 3):   # in slices through the workspace; in one kernel (405 blocks of 64 tiles)
        y = conv_ops.conv_forward(xd, wd, bd, pad, 1, 1, 1, v)
        assert_rel(host(y), host(y1), 2e-5, f"Winograd forward variant {v} vs variant 1")
        assert_rel(host(y)[tuple(np.array(idx).T)], exp, TOL,
                   f"Winograd forward variant {v} vs float64 samples")
        del y

    dx1 = conv_ops.conv_backward_input(xs, dyd, wd, pad, 1, 1, 1, 1)
    idx = [(rng.integers(xs[0]), rng.integers(xs[1]), rng.integers(xs[2]), rng.integers(xs[3]))
           for _ in range(256)] + [(3, 255, 160, 158), (0, 0, 0, 0)]
    # dx[n, c, h, q] = sum over k, r, s of dy[n, k, h + 1 - r, q + 1 - s] w[k, c, r, s]
    exp = np.array([(dyp[n, :, h:h + 3, q:q + 3][:, ::-1, ::-1] * w64[:, c]).sum()
                    for n, c, h, q in idx])
    for v in (2, 3):
        dx = conv_ops.conv_backward_input(xs, dyd, wd, pad, 1, 1, 1, v)
        assert_rel(host(dx), host(dx1), 2e-5, f"Winograd backward-data variant {v} vs variant 1")
        assert_rel(host(dx)[tuple(np.array(idx).T)], exp, TOL,
                   f"Winograd backward-data variant {v} vs float64 samples")
        del dx

    dw1 = conv_ops.conv_backward_weight(ws, dyd, xd, pad, 1, 1, 1, 1)
    dw2 = conv_ops.conv_backward_weight(ws, dyd, xd, pad, 1, 1, 1, 2)
    assert_rel(host(dw2), host(dw1), 2e-5, "Winograd backward-weight in passes vs variant 1")
    idx = [(rng.integers(ws[0]), rng.integers(ws[1]), rng.integers(3), rng.integers(3))
           for _ in range(48)]
    dy64 = dy.astype(np.float64)
    exp = np.array([(dy64[:, k] * xp[:, c, r:r + xs[2], s:s + xs[3]]).sum() for k, c, r, s in idx])
    got = host(dw2)[tuple(np.array(idx).T)]
    assert_rel(got, exp, TOL, "Winograd backward-weight in passes vs float64 samples")
    # the same call again gives the same bits (fixed order of slices and passes)
    assert torch.equal(dw2, conv_ops.conv_backward_weight(ws, dyd, xd, pad, 1, 1, 1, 2))


def _random_winograd_shapes(count, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        n = int(rng.integers(1, 4))
        c = int(rng.choice([16, 32, 48, 64, 80]))
        k = int(rng.choice([4, 16, 24, 64, 72, 130]))
        h, w = int(rng.integers(4, 41)), int(rng.integers(4, 41))
        pad = int(rng.integers(0, 3))
        out.append(((n, c, h, w), (k, c, 3, 3), pad))
    return out


@pytest.mark.parametrize("xs,ws,pad", _random_winograd_shapes(16, 2024))
def test_winograd_variants_on_random_shapes(cuda, xs, ws, pad):
    """Both Winograd forms (through the workspace, in one kernel) in every direction they serve,
    on shapes drawn at random: planes from 4 x 4 to 40 x 40 (ragged tiles, rows shorter than a
    wavefront, tile blocks that span several images), outputs that do not fill a block of 64,
    every padding; against the float64 oracle.  Backward-data also in its accumulating form."""
    x, w, b = problem(xs, ws, 11)
    exp = O.conv_fwd(x, w, b, 1, pad, 1)
    dy = np.random.default_rng(12).standard_normal(exp.shape).astype(np.float32)
    exp_dx = O.conv_bwd_data(dy, w, xs, 1, pad, 1)
    exp_dw = O.conv_bwd_weight(dy, x, ws, 1, pad, 1)
    xd, wd, bd, dyd = dev(x, cuda), dev(w, cuda), dev(b, cuda), dev(dy, cuda)
    for v in (2, 3):
        y = conv_ops.conv_forward(xd, wd, bd, pad, 1, 1, 1, v)
        assert_rel(host(y), exp, TOL, f"forward variant {v} {xs} {ws} pad {pad}")
        if ws[0] % 16 == 0:   # backward-data reduces over K
            dx = conv_ops.conv_backward_input(xs, dyd, wd, pad, 1, 1, 1, v)
            assert_rel(host(dx), exp_dx, TOL, f"backward-data variant {v} {xs} {ws} pad {pad}")
        else:
            assert refused(lambda: conv_ops.conv_backward_input(xs, dyd, wd, pad, 1, 1, 1, v))
    dw = conv_ops.conv_backward_weight(ws, dyd, xd, pad, 1, 1, 1, 2)
    assert_rel(host(dw), exp_dw, TOL, f"backward-weight variant 2 {xs} {ws} pad {pad}")
