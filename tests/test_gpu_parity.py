"""GPU parity: every kernel, called through the operator classes (and so
through the C ABI of libmonet_hip.so), against the CPU oracle on the same
seeded inputs.  Integer / bit results must be identical; float results are
compared with the tolerance written next to each check."""
import numpy as np
import pytest
import torch

import monet_amd.lm_ops as lm_ops
from monet_amd.lm_ops import bn as bn_ops
from monet_amd.lm_ops import pack as pk
from monet_amd.lm_ops import pool as pool_ops
from monet_amd.lm_ops import relu as relu_ops
from monet_amd.lm_ops import softmax as sm_ops
from oracle import lm_oracle as O

pytestmark = pytest.mark.gpu

SIZES = [1, 7, 8, 9, 31, 32, 33, 255, 1023, 1024, 1025, 4096 * 3 + 5, 1 << 20, (1 << 20) + 13]


def dev(a, cuda):
    return torch.from_numpy(np.ascontiguousarray(a)).to(cuda)


def host(t):
    return t.detach().cpu().numpy()


def special_floats(n, seed):
    x = np.random.default_rng(seed).standard_normal(n).astype(np.float32)
    sp = np.array([0.0, -0.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45, 3.0], np.float32)
    x[:min(n, 8)] = sp[:min(n, 8)]
    return x


# ------------------------------------------------------------------- packing
@pytest.mark.parametrize("n", SIZES)
def test_pack_unpack_bits(cuda, n):
    bits = np.random.default_rng(n).random(n) > 0.5
    p = pk.pack(dev(bits, cuda))
    assert np.array_equal(host(p), O.pack_bits(bits))
    assert np.array_equal(host(pk.unpack(p, n)), bits)
    full = host(pk.unpack(p))
    assert full.size == p.numel() * 8 and not full[n:].any()
    q = torch.zeros_like(p)
    pk.pack_(dev(bits, cuda), q)
    assert torch.equal(p, q)


@pytest.mark.parametrize("n", SIZES)
def test_pack_unpack_nibbles(cuda, n):
    v = np.random.default_rng(n).integers(0, 16, n).astype(np.uint8)
    p = pk.pack_two(dev(v, cuda))
    assert np.array_equal(host(p), O.pack_nibbles(v))
    assert np.array_equal(host(pk.unpack_two(p, n)), v)


def test_pack_unaligned_views(cuda):
    for off in (1, 3, 5):
        bits = np.random.default_rng(off).random(1000 + off) > 0.5
        t = dev(bits, cuda)[off:]
        assert np.array_equal(host(pk.pack(t)), O.pack_bits(bits[off:]))
        v = np.random.default_rng(off).integers(0, 16, 1000 + off).astype(np.uint8)
        assert np.array_equal(host(pk.pack_two(dev(v, cuda)[off:])), O.pack_nibbles(v[off:]))


@pytest.mark.parametrize("n", [5, 64, 1027, 1 << 18])
def test_unpack_multiply(cuda, n):
    v = special_floats(n, 7)
    bits = np.random.default_rng(8).random(n) > 0.5
    r = pk.unpack_multiply(dev(O.pack_bits(bits), cuda), dev(v, cuda))
    assert np.array_equal(host(r), O.unpack_bits_mul(O.pack_bits(bits), v), equal_nan=True)


def test_empty_inputs(cuda):
    e = torch.empty(0, dtype=torch.bool, device=cuda)
    assert pk.pack(e).numel() == 0
    assert pk.pack_two(torch.empty(0, dtype=torch.uint8, device=cuda)).numel() == 0
    y, m = relu_ops.relu_forward_with_mask(torch.empty(0, device=cuda))
    assert y.numel() == 0 and m.numel() == 0


# ---------------------------------------------------------------------- relu
@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("inplace", [False, True])
def test_binary_relu_forward(cuda, n, inplace):
    x = special_floats(n, n)
    oy, omask = O.relu_fwd_mask(x)
    op = lm_ops.relu.BinaryActReLU()
    op.inplace = inplace
    tx = dev(x, cuda)
    y, mask = op.forward(tx)
    assert np.array_equal(host(mask), omask)          # bit-exact
    assert np.array_equal(host(y), oy, equal_nan=True)  # exact
    assert (y.data_ptr() == tx.data_ptr()) == inplace
    if not inplace:
        assert np.array_equal(host(tx), x, equal_nan=True)
        assert np.array_equal(host(op.intermediate(tx)), omask)


@pytest.mark.parametrize("n", SIZES)
def test_binary_relu_backward(cuda, n):
    x = special_floats(n, n + 1)
    g = special_floats(n, n + 2)[::-1].copy()
    _, omask = O.relu_fwd_mask(x)
    tg = dev(g, cuda)
    stored = [dev(omask, cuda)]
    out = lm_ops.relu.BinaryActReLU().backward(tg, stored)
    assert stored == []                               # consumed
    assert out.data_ptr() == tg.data_ptr()            # in place on the gradient
    exp = O.relu_bwd_mask(g, omask)
    got = host(out)
    assert np.array_equal(got, exp, equal_nan=True)
    assert np.array_equal(np.signbit(got), np.signbit(exp))  # the multiply keeps -0.0


@pytest.mark.parametrize("cls", ["InputActReLU", "OutputActReLU"])
@pytest.mark.parametrize("n", [1, 5, 1024, 4099, 1 << 20])
def test_relu_backward_from_stored_activation(cuda, cls, n):
    x = special_floats(n, 3)
    g = np.random.default_rng(4).standard_normal(n).astype(np.float32)
    op = getattr(lm_ops.relu, cls)()
    ref = x if cls == "InputActReLU" else O.relu_fwd_mask(x)[0]
    y = op.forward(dev(x, cuda))
    assert np.array_equal(host(y), O.relu_fwd_mask(x)[0], equal_nan=True)
    stored = [dev(ref, cuda)]
    out = op.backward(dev(g, cuda), stored, nodel=True)
    assert len(stored) == 1
    assert np.array_equal(host(out), O.relu_bwd_ref(g, ref))


def test_relu_4d_and_unaligned(cuda):
    x = special_floats(2 * 3 * 5 * 7 + 3, 5)
    tx = dev(x, cuda)[3:].view(2, 3, 5, 7)           # 12-byte offset: scalar path
    y, mask = lm_ops.relu.BinaryActReLU().forward(tx)
    oy, omask = O.relu_fwd_mask(x[3:].reshape(2, 3, 5, 7))
    assert y.shape == tx.shape
    assert np.array_equal(host(mask), omask) and np.array_equal(host(y), oy, equal_nan=True)
    g = dev(special_floats(x.size, 6), cuda)[3:].view(2, 3, 5, 7)
    exp = O.relu_bwd_mask(host(g), omask)
    out = lm_ops.relu.BinaryActReLU().backward(g, [mask])
    assert np.array_equal(host(out), exp, equal_nan=True)


# ------------------------------------------------------------------- maxpool
POOL_CASES = [
    ((2, 3, 12, 12), 3, 2, 1, 1, False),
    ((1, 2, 13, 11), 3, 2, 1, 1, True),
    ((2, 2, 8, 10), 2, 2, 0, 1, False),
    ((1, 1, 9, 9), (2, 3), (1, 2), (1, 1), 1, False),
    ((1, 2, 11, 11), 3, 1, 1, 2, False),
    ((1, 1, 7, 7), 4, 3, 2, 1, True),
    ((3, 1, 5, 5), 3, 2, 1, 1, False),
    ((4, 16, 112, 112), 3, 2, 1, 1, False),
    ((2, 8, 52, 76), 2, 2, 0, 1, False),
    ((3, 5, 7, 7), 3, 2, 1, 1, False),              # odd plane: index pairs straddle planes
    ((2, 3, 12, 12), 3, 2, 1, 1, True),             # ceil_mode adds a pooled row and column: 7 x 7
    ((2, 2, 16, 24), 3, 2, 1, 1, True),
]


@pytest.mark.parametrize("shape,k,s,p,d,ceil", POOL_CASES)
@pytest.mark.parametrize("kind", ["ties", "normal", "special"])
def test_maxpool_indices_forward_backward(cuda, shape, k, s, p, d, ceil, kind):
    rng = np.random.default_rng(13)
    if kind == "ties":
        x = rng.integers(-3, 4, shape).astype(np.float32)
    else:
        x = rng.standard_normal(shape).astype(np.float32)
    if kind == "special":
        flat = x.reshape(-1)
        flat[rng.integers(0, flat.size, max(flat.size // 10, 1))] = np.nan
        flat[rng.integers(0, flat.size, max(flat.size // 3, 1))] = -np.inf
    oy, opacked, _ = O.maxpool_fwd_idx(x, k, s, p, d, ceil)
    op = lm_ops.pool.IndicesActMaxPool2D()
    y, packed = op.forward(dev(x, cuda), k, s, p, d, ceil)
    assert list(y.shape) == list(oy.shape)
    assert np.array_equal(host(packed), opacked)                 # bit-exact
    assert np.array_equal(host(y), oy, equal_nan=True)           # exact
    dy = rng.standard_normal(oy.shape).astype(np.float32)
    stored = [packed]
    dx = op.backward(dev(dy, cuda), stored)
    assert stored == []
    odx = O.maxpool_bwd_idx(dy, opacked, shape, k, s, p, d)
    assert np.array_equal(host(dx), odx)                         # same summation order: exact


def test_maxpool_simple_matches_indices(cuda):
    x = torch.randn(3, 4, 20, 20, device=cuda)
    dy = torch.randn(3, 4, 10, 10, device=cuda)
    a, b = lm_ops.pool.SimpleMaxPool2D(), lm_ops.pool.IndicesActMaxPool2D()
    ya = a.forward(x, 3, 2, 1, 1, False)
    yb, idx = b.forward(x, 3, 2, 1, 1, False)
    assert torch.equal(ya, yb)
    da = a.backward(dy, [x])
    db = b.backward(dy, [idx])
    torch.testing.assert_close(da, db, rtol=1e-6, atol=1e-6)


def test_maxpool_rejects_what_a_nibble_cannot_hold(cuda):
    with pytest.raises(RuntimeError, match="unsupported"):
        lm_ops.pool.IndicesActMaxPool2D().forward(torch.randn(1, 1, 16, 16, device=cuda), 5, 2, 2,
                                                  1, False)


# ----------------------------------------------------------------- batchnorm
BN_SHAPES = [(4, 3, 5, 5), (2, 8, 7, 3), (16, 4, 6, 6), (8, 64, 56, 56), (32, 16, 7, 7),
             (3, 5, 1, 1), (2, 2, 130, 70), (184, 8, 28, 28),
             (184, 6, 14, 14), (184, 5, 7, 7),   # whole channel in one workgroup
             (184, 2, 112, 112)]   # channels long enough for the 512-thread one-pass kernel


def bn_problem(shape, seed):
    rng = np.random.default_rng(seed)
    C = shape[1]
    x = (rng.standard_normal(shape) * 1.7 + 0.4).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, C).astype(np.float32)
    beta = (rng.standard_normal(C) * 0.1).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    return x, gamma, beta, dy


def assert_rel(got, exp, tol, what):
    """max |got - exp| <= tol * max |exp| (error relative to the tensor's scale)."""
    exp = np.asarray(exp, np.float64)
    err = np.abs(np.asarray(got, np.float64) - exp).max()
    scale = max(np.abs(exp).max(), 1e-30)
    # what was achieved, for whoever reads the log (pytest -s): tolerances are set from these
    print(f"achieved {what}: {err / scale:.2e} of scale (tolerance {tol:.0e})")
    assert err <= tol * scale, f"{what}: max err {err:.3e} vs scale {scale:.3e}"


@pytest.mark.parametrize("shape", BN_SHAPES)
def test_bn_forward_train_and_recompute(cuda, shape):
    x, gamma, beta, _ = bn_problem(shape, 0)
    C = shape[1]
    rm0 = np.linspace(-1, 1, C).astype(np.float32)
    rv0 = np.linspace(0.5, 2, C).astype(np.float32)
    oy, omean, oinv, orm, orv = O.bn_fwd_train(x, gamma, beta, rm0, rv0, 0.1, 1e-5)
    op = lm_ops.bn.InputActBatchNorm()
    trm, trv = dev(rm0, cuda), dev(rv0, cuda)
    tx, tw, tb = dev(x, cuda), dev(gamma, cuda), dev(beta, cuda)
    y = op.forward(tx, tw, tb, trm, trv, True, 0.1, 1e-5)
    training, eps, save_mean, save_invstd, _ = op.params
    assert training is True and eps == 1e-5
    # fp32 kernel vs float64 oracle: 1e-5 relative to each tensor's scale
    assert_rel(host(y), oy, 1e-5, "y")
    assert_rel(host(save_mean), omean, 1e-5, "save_mean")
    assert_rel(host(save_invstd), oinv, 1e-5, "save_invstd")
    assert_rel(host(trm), orm, 1e-5, "running_mean")
    assert_rel(host(trv), orv, 1e-5, "running_var")
    # recomputation: same instance, params set -> identical bits, running stats untouched
    rm_before, rv_before = trm.clone(), trv.clone()
    y2 = op.forward(tx, tw, tb, trm, trv, True, 0.1, 1e-5)
    assert torch.equal(trm, rm_before) and torch.equal(trv, rv_before)
    assert np.array_equal(host(y2), host(y)), "recomputed y"   # the saved statistics re-applied: bit for bit


@pytest.mark.parametrize("n", [1, 7, 8, 31, 32, 33, 1000, 4099, 1 << 18])
@pytest.mark.parametrize("cls", ["OutputActAddReLU", "BinaryActAddReLU"])
def test_add_relu_fused(cuda, cls, n):
    """relu(a + b) as one operator: output, mask and both gradients exact (alpha = 1 is a plain
    fp32 addition), out of place and in place; unaligned views take the scalar kernel."""
    rng = np.random.default_rng(n)
    a = rng.standard_normal(n + 3).astype(np.float32)
    b = rng.standard_normal(n + 3).astype(np.float32)
    b[::5] = -a[::5]                       # exact zeros in the sum
    dy = rng.standard_normal(n).astype(np.float32)
    for off in (0, 3):                     # 3: breaks the 16-byte alignment
        av, bv = a[off:off + n], b[off:off + n]
        oy, omask = O.add_relu_fwd(av, bv)
        for inplace in (False, True):
            op = getattr(lm_ops.funcs, cls)()
            op.inplace = inplace
            ta, tb = dev(a, cuda)[off:off + n], dev(b, cuda)[off:off + n]
            res = op.forward(ta, tb, 1)
            y, mask = res if isinstance(res, tuple) else (res, None)
            assert np.array_equal(host(y), oy)
            if inplace:
                assert y.data_ptr() == ta.data_ptr()
            if mask is not None:
                assert np.array_equal(host(mask), omask)
            stored = [mask if mask is not None else y]
            ga, gb = op.backward(dev(dy, cuda), stored)
            assert stored == []
            exp = np.where(oy > 0, dy, 0).astype(np.float32)
            assert np.array_equal(host(ga), exp) and np.array_equal(host(gb), exp)
    # alpha != 1: the kernel may contract a + alpha*b into one fused multiply-add
    op = getattr(lm_ops.funcs, cls)()
    res = op.forward(dev(a[:n], cuda), dev(b[:n], cuda), 0.5)
    y = res[0] if isinstance(res, tuple) else res
    np.testing.assert_allclose(host(y), np.maximum(a[:n] + 0.5 * b[:n], 0), rtol=0, atol=1e-6)


@pytest.mark.parametrize("shape", BN_SHAPES)
def test_bn_relu_fused_forward_backward_and_recompute(cuda, shape):
    """relu(BN(x)) as one operator: forward against the oracle; backward against the oracle
    fed the GPU's own sign decisions (a pre-activation within rounding distance of zero may
    legitimately fall on either side); recomputation from the saved statistics."""
    x, gamma, beta, dy = bn_problem(shape, 4)
    oy, omean, oinv, _, _ = O.bn_relu_fwd_train(x, gamma, beta, None, None, 0.1, 1e-5)
    op = lm_ops.bn.InputActBatchNormReLU()
    tx, tw, tb, tg = dev(x, cuda), dev(gamma, cuda), dev(beta, cuda), dev(dy, cuda)
    C = shape[1]
    rm, rv = torch.zeros(C, device=cuda), torch.ones(C, device=cuda)
    y = op.forward(tx, tw, tb, rm, rv, True, 0.1, 1e-5)
    assert_rel(host(y), oy, 1e-5, "relu(bn(x))")
    assert float(y.min()) >= 0.0
    # where the oracle is clearly positive / negative the GPU agrees
    clear = np.abs(O.bn_fwd_train(x, gamma, beta, None, None, 0.1, 1e-5)[0]) > 1e-4
    assert np.array_equal((host(y) > 0)[clear], (oy > 0)[clear])
    y2 = op.forward(tx, tw, tb, rm, rv, True, 0.1, 1e-5)          # recomputation
    assert np.array_equal(host(y2), host(y)), "recomputed relu(bn(x))"   # the saved statistics re-applied: bit for bit
    assert np.array_equal(host(y2) > 0, host(y) > 0)
    odx, odg, odb = O.bn_relu_bwd_from_x(dy, x, gamma, beta, omean, oinv, positive=host(y) > 0)
    stored = [tx, tw, tb, rm, rv]
    dx, dg, db, n1, n2 = op.backward(tg.clone(), stored)
    assert stored == [] and n1 is None and n2 is None
    assert_rel(host(dx), odx, 1e-5, "dx")
    assert_rel(host(dg), odg, 1e-5, "dgamma")
    assert_rel(host(db), odb, 1e-5, "dbeta")


@pytest.mark.parametrize("alpha", [1, 0.5])
@pytest.mark.parametrize("shape", BN_SHAPES)
def test_bn_add_relu_fused_forward_backward_and_recompute(cuda, shape, alpha):
    """relu(BN(x) + alpha*r) as one operator: forward against the oracle, recomputation from
    the saved statistics, backward against the oracle fed the GPU's own output (an output
    within rounding distance of zero may legitimately fall on either side)."""
    x, gamma, beta, dy = bn_problem(shape, 8)
    r = np.random.default_rng(9).standard_normal(shape).astype(np.float32)
    oy, omean, oinv, _, _ = O.bn_add_relu_fwd_train(x, gamma, beta, r, alpha, None, None, 0.1, 1e-5)
    op = lm_ops.bn.InputActBatchNormAddReLU()
    tx, tw, tb, tg, tr = (dev(x, cuda), dev(gamma, cuda), dev(beta, cuda), dev(dy, cuda),
                          dev(r, cuda))
    C = shape[1]
    rm, rv = torch.zeros(C, device=cuda), torch.ones(C, device=cuda)
    y = op.forward(tx, tw, tb, rm, rv, True, 0.1, 1e-5, True, tr, alpha)
    assert_rel(host(y), oy, 1e-5, "relu(bn(x) + r)")
    assert float(y.min()) >= 0.0
    assert np.array_equal(host(tx), x) and np.array_equal(host(tr), r)   # operands untouched
    # the statistics are those of the plain forward
    plain = lm_ops.bn.InputActBatchNorm()
    rm2, rv2 = torch.zeros(C, device=cuda), torch.ones(C, device=cuda)
    plain.forward(tx, tw, tb, rm2, rv2, True, 0.1, 1e-5)
    # (another piece length, hence another summation order: equal to rounding, not bit for bit)
    assert_rel(host(op.params[2]), host(plain.params[2]), 1e-6, "save_mean")
    assert_rel(host(op.params[3]), host(plain.params[3]), 1e-6, "save_invstd")
    assert_rel(host(rm), host(rm2), 1e-6, "running_mean")
    assert_rel(host(rv), host(rv2), 1e-6, "running_var")
    rm_after_first = rm.clone()
    pre = O.bn_fwd_train(x, gamma, beta, None, None, 0.1, 1e-5)[0] + alpha * r.astype(np.float64)
    clear = np.abs(pre) > 1e-4
    assert np.array_equal((host(y) > 0)[clear], (oy > 0)[clear])
    y2 = op.forward(tx, tw, tb, rm, rv, True, 0.1, 1e-5, True, tr, alpha)   # recomputation
    assert np.array_equal(host(y2), host(y)), "recomputed relu(bn(x) + r)"   # the saved statistics re-applied: bit for bit
    assert torch.equal(rm, rm_after_first)                                 # no second update
    odx, odg, odb, odr = O.bn_add_relu_bwd(dy, x, host(y), gamma, omean, oinv, alpha)
    stored = [tx, tw, tb, rm, rv, y]
    dx, dg, db, n1, n2, dr = op.backward(tg.clone(), stored)
    assert stored == [] and n1 is None and n2 is None
    assert_rel(host(dx), odx, 1e-5, "dx")
    assert_rel(host(dg), odg, 1e-5, "dgamma")
    assert_rel(host(db), odb, 1e-5, "dbeta")
    assert np.array_equal(host(dr), odr.astype(np.float32))               # a gated copy: exact


@pytest.mark.parametrize("shape", BN_SHAPES)
def test_bn_backward_from_input_and_from_output(cuda, shape):
    x, gamma, beta, dy = bn_problem(shape, 1)
    oy, omean, oinv, _, _ = O.bn_fwd_train(x, gamma, beta, None, None, 0.1, 1e-5)
    odx, odg, odb = O.bn_bwd_from_x(dy, x, gamma, omean, oinv)   # float64 truth
    tx, tw, tb, tg = dev(x, cuda), dev(gamma, cuda), dev(beta, cuda), dev(dy, cuda)
    C = shape[1]
    rm, rv = torch.zeros(C, device=cuda), torch.ones(C, device=cuda)

    a = lm_ops.bn.InputActBatchNorm()
    y = a.forward(tx, tw, tb, rm, rv, True, 0.1, 1e-5)
    stored = [tx, tw, tb, rm, rv]
    dx, dg, db, n1, n2 = a.backward(tg, stored)
    assert stored == [] and n1 is None and n2 is None
    # sums over up to 577k fp32 terms: 1e-5 of the tensor's scale (achieved: below 1e-6)
    assert_rel(host(dx), odx, 1e-5, "dx from x")
    assert_rel(host(dg), odg, 1e-5, "dgamma from x")
    assert_rel(host(db), odb, 1e-5, "dbeta from x")

    b = lm_ops.bn.OutputActBatchNorm()
    b.params = a.params                      # the executor ferries params between instances
    stored = [tw, tb, rm, rv, y]
    dx2, dg2, db2, _, _ = b.backward(tg, stored, nodel=True)
    assert len(stored) == 5
    assert_rel(host(dx2), odx, 1e-5, "dx from y")
    assert_rel(host(dg2), odg, 1e-5, "dgamma from y")
    assert_rel(host(db2), odb, 1e-5, "dbeta from y")
    # and against the float64 oracle of the from-output formula fed the GPU's own y
    edx, edg, edb = O.bn_bwd_from_y(dy, host(y), gamma, beta, host(a.params[3]))
    assert_rel(host(dx2), edx, 1e-5, "dx from y (same y)")


def test_bn_from_output_with_large_mean_and_small_gamma(cuda):
    shape = (16, 6, 9, 9)
    x, gamma, beta, dy = bn_problem(shape, 2)
    x += 50.0                                   # mean >> std: variance must not cancel
    gamma[:3] = [0.01, -0.7, 1e-3]
    oy, omean, oinv, _, _ = O.bn_fwd_train(x, gamma, beta, None, None, 0.1, 1e-5)
    odx, odg, odb = O.bn_bwd_from_x(dy, x, gamma, omean, oinv)
    y, mean, invstd = bn_ops.bn_forward_train(dev(x, cuda), dev(gamma, cuda), dev(beta, cuda), None,
                                              None, 0.1, 1e-5)
    assert_rel(host(invstd), oinv, 1e-5, "invstd with large mean")
    assert_rel(host(y), oy, 1e-5, "y with large mean")
    dx, dg, db = bn_ops.bn_backward_from_input(dev(dy, cuda), dev(x, cuda), dev(gamma, cuda), mean,
                                               invstd)
    assert_rel(host(dx), odx, 1e-5, "dx")
    assert_rel(host(dg), odg, 1e-5, "dgamma")


def test_bn_channel_too_large_to_keep_on_chip(cuda):
    # 4.3M elements per channel: more than 256 register-resident pieces, so the
    # two-launch (reduce, apply) formulation runs
    shape = (1, 2, 2100, 2048)
    x, gamma, beta, dy = bn_problem(shape, 5)
    oy, omean, oinv, _, _ = O.bn_fwd_train(x, gamma, beta, None, None, 0.1, 1e-5)
    odx, odg, odb = O.bn_bwd_from_x(dy, x, gamma, omean, oinv)
    tw, tb = dev(gamma, cuda), dev(beta, cuda)
    y, mean, invstd = bn_ops.bn_forward_train(dev(x, cuda), tw, tb, None, None, 0.1, 1e-5)
    assert_rel(host(y), oy, 1e-5, "y")
    dx, dg, db = bn_ops.bn_backward_from_output(dev(dy, cuda), y, tw, tb, invstd)
    assert_rel(host(dx), odx, 1e-5, "dx from y")
    assert_rel(host(dg), odg, 1e-5, "dgamma")
    assert_rel(host(db), odb, 1e-5, "dbeta")


@pytest.mark.parametrize("alpha", [1, 0.5])
@pytest.mark.parametrize("shape", BN_SHAPES + [(8, 6, 8, 8), (1, 2, 2100, 2048)])
def test_bn_add_relu_with_mask_forward_backward_and_recompute(cuda, shape, alpha):
    """The mask-keeping variant: same output as the output-keeping one bit for bit, mask =
    packed sign of the GPU's own output, recomputation reproduces both, backward against the
    oracle fed that output.  Shapes with planes of a multiple of 8 elements write the mask in
    the BatchNorm kernel, the others in a second launch; the last shape runs the two-launch
    formulation."""
    x, gamma, beta, dy = bn_problem(shape, 12)
    r = np.random.default_rng(13).standard_normal(shape).astype(np.float32)
    tx, tw, tb, tg, tr = (dev(x, cuda), dev(gamma, cuda), dev(beta, cuda), dev(dy, cuda),
                          dev(r, cuda))
    C = shape[1]
    rm, rv = torch.zeros(C, device=cuda), torch.ones(C, device=cuda)
    rm0, rv0 = rm.clone(), rv.clone()
    plain = lm_ops.bn.InputActBatchNormAddReLU()
    y0 = plain.forward(tx, tw, tb, rm0, rv0, True, 0.1, 1e-5, True, tr, alpha)
    op = lm_ops.bn.BinaryActBatchNormAddReLU()
    y, mask = op.forward(tx, tw, tb, rm, rv, True, 0.1, 1e-5, True, tr, alpha)
    assert torch.equal(y, y0) and torch.equal(rm, rm0) and torch.equal(rv, rv0)
    assert mask.dtype == torch.uint8 and mask.numel() == (y.numel() + 7) // 8
    assert np.array_equal(host(mask), O.pack_bits(host(y).ravel() > 0))
    y2, mask2 = op.forward(tx, tw, tb, rm, rv, True, 0.1, 1e-5, True, tr, alpha)   # recomputation
    assert np.array_equal(host(y2), host(y)), "recomputed output"   # the saved statistics re-applied: bit for bit
    assert np.array_equal(host(mask2), O.pack_bits(host(y2).ravel() > 0))
    assert torch.equal(rm, rm0)
    _, omean, oinv, _, _ = O.bn_fwd_train(x, gamma, beta, None, None, 0.1, 1e-5)
    odx, odg, odb, odr = O.bn_add_relu_bwd(dy, x, host(y), gamma, omean, oinv, alpha)
    stored = [tx, tw, tb, rm, rv, mask]
    dx, dg, db, n1, n2, dr = op.backward(tg.clone(), stored)
    assert stored == [] and n1 is None and n2 is None
    big = shape[2] * shape[3] > 1000000
    assert_rel(host(dx), odx, 1e-5, "dx")
    assert_rel(host(dg), odg, 1e-5, "dgamma")
    assert_rel(host(db), odb, 1e-5, "dbeta")
    assert np.array_equal(host(dr), odr.astype(np.float32))


def test_bn_add_relu_channel_too_large_to_keep_on_chip(cuda):
    # the fused end of a residual block on the two-launch (reduce, apply) formulation
    shape = (1, 2, 2100, 2048)
    x, gamma, beta, dy = bn_problem(shape, 6)
    r = np.random.default_rng(10).standard_normal(shape).astype(np.float32)
    oy, omean, oinv, _, _ = O.bn_add_relu_fwd_train(x, gamma, beta, r, 1.0, None, None, 0.1, 1e-5)
    tx, tw, tb, tr = dev(x, cuda), dev(gamma, cuda), dev(beta, cuda), dev(r, cuda)
    y, mean, invstd = bn_ops.bn_add_relu_forward_train(tx, tw, tb, None, None, tr, 1, 0.1, 1e-5)
    assert_rel(host(y), oy, 1e-5, "y")
    y2 = bn_ops.bn_add_relu_forward_apply(tx, mean, invstd, tw, tb, tr, 1)
    assert np.array_equal(host(y2), host(y)), "recomputed y"   # the saved statistics re-applied: bit for bit
    odx, odg, odb, odr = O.bn_add_relu_bwd(dy, x, host(y), gamma, omean, oinv, 1.0)
    dx, dg, db, dr = bn_ops.bn_add_relu_backward(dev(dy, cuda), tx, y, tw, mean, invstd, 1)
    assert_rel(host(dx), odx, 1e-5, "dx")
    assert_rel(host(dg), odg, 1e-5, "dgamma")
    assert_rel(host(db), odb, 1e-5, "dbeta")
    assert np.array_equal(host(dr), odr.astype(np.float32))


def test_bn_add_relu_eval_mode_uses_running_statistics(cuda):
    op = lm_ops.bn.InputActBatchNormAddReLU()
    x = torch.randn(2, 3, 4, 4, device=cuda)
    r = torch.randn(2, 3, 4, 4, device=cuda)
    w, b = torch.rand(3, device=cuda) + 0.5, torch.randn(3, device=cuda)
    rm, rv = torch.randn(3, device=cuda), torch.rand(3, device=cuda) + 0.5
    y = op.forward(x, w, b, rm, rv, False, 0.1, 1e-5, True, r, 1)
    ref = torch.relu(torch.nn.functional.batch_norm(x, rm, rv, w, b, False, 0.1, 1e-5) + r)
    torch.testing.assert_close(y, ref, rtol=1e-5, atol=1e-6)
    with pytest.raises(NotImplementedError):
        op.backward(torch.ones_like(y), [x, w, b, rm, rv, y])


def test_bn_non_affine_and_inplace_output(cuda):
    shape = (4, 3, 8, 8)
    x, _, _, dy = bn_problem(shape, 3)
    oy, omean, oinv, _, _ = O.bn_fwd_train(x, None, None, None, None, 0.1, 1e-5)
    tx = dev(x, cuda)
    y, mean, invstd = bn_ops.bn_forward_train(tx, None, None, None, None, 0.1, 1e-5, out=tx)
    assert y.data_ptr() == tx.data_ptr()
    assert_rel(host(y), oy, 1e-5, "in-place y")
    odx, _, _ = O.bn_bwd_from_x(dy, x, None, omean, oinv)
    dx, dg, db = bn_ops.bn_backward_from_input(dev(dy, cuda), dev(x, cuda), None, mean, invstd)
    assert_rel(host(dx), odx, 1e-5, "dx non-affine")


def test_bn_eval_backward_is_not_implemented(cuda):
    op = lm_ops.bn.InputActBatchNorm()
    x = torch.randn(2, 3, 4, 4, device=cuda)
    w, b = torch.ones(3, device=cuda), torch.zeros(3, device=cuda)
    rm, rv = torch.zeros(3, device=cuda), torch.ones(3, device=cuda)
    y = op.forward(x, w, b, rm, rv, False, 0.1, 1e-5)
    torch.testing.assert_close(y, torch.nn.functional.batch_norm(x, rm, rv, w, b, False, 0.1, 1e-5),
                               rtol=1e-5, atol=1e-6)
    with pytest.raises(NotImplementedError):
        op.backward(torch.randn_like(x), [x, w, b, rm, rv])


# ------------------------------------------------------------------- softmax
@pytest.mark.parametrize("shape,dim", [((184, 1000), 1), ((7, 10), 1), ((3, 2, 50, 40), 1),
                                       ((4, 6, 3), 2), ((5, 3000), -1), ((2, 21, 33, 17), 1)])
def test_softmax_forward_backward(cuda, shape, dim):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    op = lm_ops.softmax.Softmax()
    y = op.forward(dev(x, cuda), dim, None)
    oy = O.softmax_fwd(x, dim)
    np.testing.assert_allclose(host(y), oy, rtol=1e-5, atol=1e-7)   # fp32 exp vs float64
    stored = [y]
    dx = op.backward(dev(dy, cuda), stored)
    assert stored == []
    odx = O.softmax_bwd(dy, host(y), dim)
    assert_rel(host(dx), odx, 1e-5, "softmax dx")


@pytest.mark.parametrize("shape", [(184, 1000), (9, 13), (2, 2, 40, 60), (3, 5, 7)])
def test_cross_entropy_backward(cuda, shape):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(shape) * 2).astype(np.float32)
    labels = rng.integers(0, shape[1], (shape[0],) + tuple(shape[2:]))
    got = sm_ops.cross_entropy_backward(dev(x, cuda), dev(labels, cuda))
    assert_rel(host(got), O.xent_bwd(x, labels), 1e-5, "xent grad")


# ---------------------------------------------------------------- glue on GPU
def test_glue_ops_backward_matches_autograd(cuda):
    x = torch.randn(4, 6, 7, 7, device=cuda)
    op = lm_ops.funcs.AdaptiveAvgPool2D()
    y = op.forward(x, [1, 1])
    g = torch.randn_like(y)
    xr = x.clone().requires_grad_(True)
    torch.nn.functional.adaptive_avg_pool2d(xr, [1, 1]).backward(g)
    torch.testing.assert_close(op.backward(g, []), xr.grad)

    # an output that is a whole (power of two) multiple of the input: replication, taken by a
    # copy kernel / gather instead of the generic pooling kernels; also a size that is not
    for in_hw, out_hw in (((5, 7), (10, 14)), ((3, 4), (12, 4)), ((5, 7), (15, 21)), ((6, 6), (4, 9))):
        xu = torch.randn(2, 3, *in_hw, device=cuda)
        up = lm_ops.funcs.AdaptiveAvgPool2D()
        yu = up.forward(xu, list(out_hw))
        xur = xu.clone().requires_grad_(True)
        ref = torch.nn.functional.adaptive_avg_pool2d(xur, list(out_hw))
        assert torch.equal(yu, ref.detach())
        gu = torch.randn_like(yu)
        ref.backward(gu)
        torch.testing.assert_close(up.backward(gu, []), xur.grad)

    lin = lm_ops.linear.LowMemLinear()
    inp = torch.randn(5, 8, device=cuda, requires_grad=True)
    w = torch.randn(3, 8, device=cuda, requires_grad=True)
    b = torch.randn(3, device=cuda, requires_grad=True)
    out = lin.forward(inp, w, b)
    go = torch.randn_like(out)
    torch.nn.functional.linear(inp, w, b).backward(go)
    lin.algorithm = 0
    di, dw, db = lin.backward(go, [inp.detach(), w.detach()], nodel=True)
    assert di is None
    torch.testing.assert_close(dw, w.grad)
    torch.testing.assert_close(db, b.grad)
    lin.algorithm = 10
    di, dw, db = lin.backward(go, [None, w.detach()], nodel=True)
    torch.testing.assert_close(di, inp.grad)

    fl = lm_ops.elementary.Flatten()
    z = fl.forward(x, 1, -1)
    assert z.shape == (4, 6 * 49)
    assert fl.backward(torch.ones_like(z), []).shape == x.shape
