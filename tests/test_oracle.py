"""Pins the CPU oracle (oracle/lm_oracle.py) against things that do not depend
on it: hand-derived known answers, numpy / torch CPU library routines, float64
autograd and pure-Python brute force.  Runs without a GPU."""
import json
from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import lm_oracle as O

GOLD = json.loads((Path(__file__).parent / "golden" / "packing.json").read_text())


# ------------------------------------------------------------------- packing
def test_pack_bits_known_answers():
    for case in GOLD["pack_bits"]:
        got = O.pack_bits(np.array(case["bits"], dtype=bool))
        assert got.tolist() == case["bytes"]
        assert O.unpack_bits(got, len(case["bits"])).astype(int).tolist() == case["bits"]


@pytest.mark.parametrize("n", [1, 7, 8, 9, 63, 64, 65, 1000, 4099])
def test_pack_bits_matches_numpy_packbits(n):
    bits = np.random.default_rng(n).random(n) > 0.5
    assert np.array_equal(O.pack_bits(bits), np.packbits(bits, bitorder="big"))
    assert np.array_equal(O.unpack_bits(O.pack_bits(bits), n), bits)


def test_pack_nibbles_known_answers():
    for case in GOLD["pack_nibbles"]:
        got = O.pack_nibbles(np.array(case["values"], dtype=np.uint8))
        assert got.tolist() == case["bytes"]
        assert O.unpack_nibbles(got, len(case["values"])).tolist() == case["values"]


@pytest.mark.parametrize("n", [2, 10, 256, 1002])
def test_pack_nibbles_closed_form(n):
    a = np.random.default_rng(n).integers(0, 16, n).astype(np.uint8)
    assert np.array_equal(O.pack_nibbles(a), (a[0::2] << 4) + a[1::2])


def test_unpack_mul_is_a_multiply():
    rng = np.random.default_rng(0)
    v = rng.standard_normal(37).astype(np.float32)
    v[3], v[4], v[5] = np.inf, np.nan, -2.0
    bits = rng.random(37) > 0.5
    bits[3] = bits[4] = bits[5] = False
    r = O.unpack_bits_mul(O.pack_bits(bits), v)
    ref = (torch.from_numpy(v) * torch.from_numpy(bits)).numpy()
    assert np.array_equal(r, ref, equal_nan=True)
    assert np.isnan(r[3]) and np.isnan(r[4]) and np.signbit(r[5]) and r[5] == 0


# ---------------------------------------------------------------------- relu
def _special_floats(n, seed):
    x = np.random.default_rng(seed).standard_normal(n).astype(np.float32)
    x[:8] = [0.0, -0.0, np.nan, np.inf, -np.inf, 1e-45, -1e-45, 3.0]
    return x


def test_relu_fwd_mask_matches_torch():
    x = _special_floats(1003, 1)
    y, mask = O.relu_fwd_mask(x)
    t = torch.from_numpy(x)
    assert np.array_equal(y, torch.clamp_min(t, 0).numpy(), equal_nan=True)
    assert np.array_equal(y, torch.relu(t).numpy(), equal_nan=True)
    assert np.array_equal(mask, np.packbits(x > 0, bitorder="big"))
    assert mask[0] == 0b00010101  # 0,-0,nan,inf,-inf,denorm,-denorm,3 -> bits 3,5,7


def test_relu_bwd_matches_torch():
    x = _special_floats(515, 2)
    g = np.random.default_rng(3).standard_normal(515).astype(np.float32)
    _, mask = O.relu_fwd_mask(x)
    ref = torch.ops.aten.threshold_backward(torch.from_numpy(g), torch.from_numpy(x), 0).numpy()
    # ATen passes the gradient where the stored value is NaN (`x <= 0 ? 0 : g`); the reference's
    # kernel tests `x > 0` (lrrelu.cu:7) and therefore gives 0 there.
    assert np.isnan(x[2]) and ref[2] == g[2]
    ref[2] = 0
    assert np.array_equal(O.relu_bwd_ref(g, x), ref)
    got = O.relu_bwd_mask(g, mask)
    assert np.array_equal(got, (torch.from_numpy(g) * torch.from_numpy(x > 0)).numpy())
    assert np.array_equal(got, ref)  # equal as values (-0.0 == 0.0)


# ------------------------------------------------------------------- maxpool
POOL_CASES = [
    # (shape, k, s, p, d, ceil)
    ((2, 3, 12, 12), 3, 2, 1, 1, False),
    ((1, 2, 13, 11), 3, 2, 1, 1, True),
    ((2, 2, 8, 10), 2, 2, 0, 1, False),
    ((1, 1, 9, 9), (2, 3), (1, 2), (1, 1), 1, False),
    ((1, 2, 11, 11), 3, 1, 1, 2, False),
    ((1, 1, 7, 7), 4, 3, 2, 1, True),
    ((3, 1, 5, 5), 3, 2, 1, 1, False),
]


def _rel_from_flat(flat, W, k, s, p, d, PH, PW):
    """Window-relative index from torch's flat h*W+w argmax."""
    kH, kW = O._pair(k)
    sH, sW = O._pair(s)
    pH, pW = O._pair(p)
    dH, dW = O._pair(d)
    h, w = flat // W, flat % W
    ph = np.arange(PH)[None, None, :, None]
    pw = np.arange(PW)[None, None, None, :]
    return ((h - (ph * sH - pH)) // dH) * kW + (w - (pw * sW - pW)) // dW


@pytest.mark.parametrize("shape,k,s,p,d,ceil", POOL_CASES)
def test_maxpool_fwd_matches_torch(shape, k, s, p, d, ceil):
    rng = np.random.default_rng(5)
    # few distinct values -> many ties, so "first maximum wins" is exercised
    x = rng.integers(-3, 4, shape).astype(np.float32)
    y, packed, idx = O.maxpool_fwd_idx(x, k, s, p, d, ceil)
    ty, tidx = F.max_pool2d(torch.from_numpy(x), k, s, p, d, ceil_mode=ceil, return_indices=True)
    assert list(y.shape) == list(ty.shape)
    assert np.array_equal(y, ty.numpy())
    rel = _rel_from_flat(tidx.numpy(), shape[3], k, s, p, d, y.shape[2], y.shape[3])
    assert np.array_equal(idx, rel)
    assert idx.max() < 16
    assert np.array_equal(O.unpack_nibbles(packed, idx.size), idx.reshape(-1))


def _brute_pool(x, k, s, p, d, ceil):
    kH, kW = O._pair(k)
    sH, sW = O._pair(s)
    pH, pW = O._pair(p)
    dH, dW = O._pair(d)
    N, C, H, W = x.shape
    PH = O.pool_out_size(H, kH, pH, sH, dH, ceil)
    PW = O.pool_out_size(W, kW, pW, sW, dW, ceil)
    y = np.zeros((N, C, PH, PW), np.float32)
    idx = np.zeros((N, C, PH, PW), np.uint8)
    for n in range(N):
        for c in range(C):
            for ph in range(PH):
                for pw in range(PW):
                    best, bi, first = -np.inf, None, None
                    for ch in range(kH):
                        for cw in range(kW):
                            h, w = ph * sH - pH + ch * dH, pw * sW - pW + cw * dW
                            if not (0 <= h < H and 0 <= w < W):
                                continue
                            if first is None:
                                first = ch * kW + cw
                            v = x[n, c, h, w]
                            if v > best or np.isnan(v):
                                best, bi = v, ch * kW + cw
                    y[n, c, ph, pw] = best
                    idx[n, c, ph, pw] = first if bi is None else bi
    return y, idx


@pytest.mark.parametrize("shape,k,s,p,d,ceil", POOL_CASES)
def test_maxpool_fwd_brute_force_with_nan_and_inf(shape, k, s, p, d, ceil):
    rng = np.random.default_rng(9)
    x = rng.integers(-2, 3, shape).astype(np.float32)
    flat = x.reshape(-1)
    flat[rng.integers(0, flat.size, max(flat.size // 10, 1))] = np.nan
    flat[rng.integers(0, flat.size, max(flat.size // 3, 1))] = -np.inf
    y, _, idx = O.maxpool_fwd_idx(x, k, s, p, d, ceil)
    by, bidx = _brute_pool(x, k, s, p, d, ceil)
    assert np.array_equal(y, by, equal_nan=True)
    assert np.array_equal(idx, bidx)


def test_maxpool_known_answer():
    g = GOLD["maxpool_3x3_s2_p1"]
    x = np.array(g["x"], np.float32)[None, None]
    y, packed, idx = O.maxpool_fwd_idx(x, 3, 2, 1)
    assert y[0, 0].tolist() == g["y"] and idx[0, 0].tolist() == g["idx"]
    assert packed.tolist() == g["packed"]
    dx = O.maxpool_bwd_idx(np.array(g["dy"], np.float32)[None, None], packed, x.shape, 3, 2, 1)
    assert dx[0, 0].tolist() == g["dx"]


@pytest.mark.parametrize("shape,k,s,p,d,ceil", POOL_CASES)
def test_maxpool_bwd_matches_autograd(shape, k, s, p, d, ceil):
    rng = np.random.default_rng(11)
    x = rng.standard_normal(shape).astype(np.float32)  # distinct values: unique argmax
    tx = torch.from_numpy(x).requires_grad_(True)
    ty = F.max_pool2d(tx, k, s, p, d, ceil_mode=ceil)
    dy = rng.standard_normal(tuple(ty.shape)).astype(np.float32)
    ty.backward(torch.from_numpy(dy))
    _, packed, _ = O.maxpool_fwd_idx(x, k, s, p, d, ceil)
    dx = O.maxpool_bwd_idx(dy, packed, shape, k, s, p, d)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(dx.sum(), dy.sum(), rtol=1e-4)


@pytest.mark.parametrize("size,k,p,s,d,ceil", [(112, 3, 1, 2, 1, False), (13, 3, 1, 2, 1, True),
                                                (7, 4, 2, 3, 1, True), (416, 2, 0, 2, 1, False),
                                                (5, 3, 1, 1, 2, False), (6, 2, 1, 2, 1, True)])
def test_pool_out_size_matches_torch(size, k, p, s, d, ceil):
    t = F.max_pool2d(torch.zeros(1, 1, size, size), k, s, p, d, ceil_mode=ceil)
    assert O.pool_out_size(size, k, p, s, d, ceil) == t.shape[-1]


# ----------------------------------------------------------------- batchnorm
def _bn_problem(shape, seed):
    rng = np.random.default_rng(seed)
    C = shape[1]
    x = (rng.standard_normal(shape) * 1.7 + 0.4).astype(np.float64)
    gamma = rng.uniform(0.5, 1.5, C)
    beta = rng.standard_normal(C) * 0.1
    dy = rng.standard_normal(shape)
    return x, gamma, beta, dy


@pytest.mark.parametrize("shape", [(4, 3, 5, 5), (2, 8, 7, 3), (6, 2, 1, 1)])
def test_bn_forward_matches_torch(shape):
    x, gamma, beta, _ = _bn_problem(shape, 0)
    rm0, rv0 = np.linspace(-1, 1, shape[1]), np.linspace(0.5, 2, shape[1])
    y, mean, invstd, rm, rv = O.bn_fwd_train(x, gamma, beta, rm0, rv0, 0.1, 1e-5)
    trm, trv = torch.from_numpy(rm0.copy()), torch.from_numpy(rv0.copy())
    ty = F.batch_norm(torch.from_numpy(x), trm, trv, torch.from_numpy(gamma),
                      torch.from_numpy(beta), True, 0.1, 1e-5)
    np.testing.assert_allclose(y, ty.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(rm, trm.numpy(), rtol=1e-12)
    np.testing.assert_allclose(rv, trv.numpy(), rtol=1e-12)
    np.testing.assert_allclose(O.bn_fwd_apply(x, mean, invstd, gamma, beta), y, rtol=1e-12)


@pytest.mark.parametrize("shape", [(4, 3, 5, 5), (2, 8, 7, 3), (16, 4, 6, 6)])
def test_bn_backward_both_forms_match_autograd(shape):
    x, gamma, beta, dy = _bn_problem(shape, 1)
    tx = torch.from_numpy(x).requires_grad_(True)
    tw = torch.from_numpy(gamma).requires_grad_(True)
    tb = torch.from_numpy(beta).requires_grad_(True)
    ty = F.batch_norm(tx, None, None, tw, tb, True, 0.1, 1e-5)
    ty.backward(torch.from_numpy(dy))
    y, mean, invstd, _, _ = O.bn_fwd_train(x, gamma, beta, None, None, 0.1, 1e-5)
    for dx, dg, db in (O.bn_bwd_from_x(dy, x, gamma, mean, invstd),
                       O.bn_bwd_from_y(dy, y, gamma, beta, invstd)):
        np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-9, atol=1e-10)
        np.testing.assert_allclose(dg, tw.grad.numpy(), rtol=1e-9, atol=1e-10)
        np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-9, atol=1e-10)
        # invariants of the BN input gradient
        np.testing.assert_allclose(dx.sum(axis=(0, 2, 3)), 0, atol=1e-9)


def test_add_relu_is_the_composition():
    rng = np.random.default_rng(6)
    a = rng.standard_normal(1001).astype(np.float32)
    b = rng.standard_normal(1001).astype(np.float32)
    y, mask = O.add_relu_fwd(a, b)
    t = torch.relu(torch.from_numpy(a) + torch.from_numpy(b)).numpy()
    assert np.array_equal(y, t)
    assert np.array_equal(O.unpack_bits(mask, 1001), (a + b) > 0)


@pytest.mark.parametrize("shape", [(4, 3, 5, 5), (2, 8, 7, 3), (16, 4, 6, 6)])
def test_bn_relu_fused_matches_autograd_of_the_composition(shape):
    x, gamma, beta, dy = _bn_problem(shape, 5)
    tx = torch.from_numpy(x).requires_grad_(True)
    tw = torch.from_numpy(gamma).requires_grad_(True)
    tb = torch.from_numpy(beta).requires_grad_(True)
    ty = torch.relu(F.batch_norm(tx, None, None, tw, tb, True, 0.1, 1e-5))
    ty.backward(torch.from_numpy(dy))
    y, mean, invstd, _, _ = O.bn_relu_fwd_train(x, gamma, beta, None, None, 0.1, 1e-5)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-12, atol=1e-14)
    assert (y >= 0).all() and (y == 0).any()
    dx, dg, db = O.bn_relu_bwd_from_x(dy, x, gamma, beta, mean, invstd)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(dg, tw.grad.numpy(), rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-9, atol=1e-10)
    # an explicit mask replaces the recomputed one
    dx2, _, _ = O.bn_relu_bwd_from_x(dy, x, gamma, beta, mean, invstd, positive=y > 0)
    np.testing.assert_allclose(dx2, dx, rtol=1e-12)


@pytest.mark.parametrize("shape,alpha", [((4, 3, 5, 5), 1.0), ((2, 8, 7, 3), 0.5), ((16, 4, 6, 6), 1.0)])
def test_bn_add_relu_fused_matches_autograd_of_the_composition(shape, alpha):
    x, gamma, beta, dy = _bn_problem(shape, 6)
    r = np.random.default_rng(7).standard_normal(shape)
    tx = torch.from_numpy(x).requires_grad_(True)
    tw = torch.from_numpy(gamma).requires_grad_(True)
    tb = torch.from_numpy(beta).requires_grad_(True)
    tr = torch.from_numpy(r).requires_grad_(True)
    ty = torch.relu(F.batch_norm(tx, None, None, tw, tb, True, 0.1, 1e-5) + alpha * tr)
    ty.backward(torch.from_numpy(dy))
    y, mean, invstd, _, _ = O.bn_add_relu_fwd_train(x, gamma, beta, r, alpha, None, None, 0.1, 1e-5)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-12, atol=1e-14)
    assert (y >= 0).all() and (y == 0).any() and (y > 0).any()
    dx, dg, db, dr = O.bn_add_relu_bwd(dy, x, y, gamma, mean, invstd, alpha)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(dg, tw.grad.numpy(), rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(dr, tr.grad.numpy(), rtol=1e-12, atol=1e-14)


# ------------------------------------------------------------------- softmax
@pytest.mark.parametrize("shape,dim", [((7, 10), 1), ((3, 2, 5, 4), 1), ((4, 6, 3), 2), ((5,), 0)])
def test_softmax_matches_torch(shape, dim):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(shape) * 3
    dy = rng.standard_normal(shape)
    y = O.softmax_fwd(x, dim)
    ty = torch.softmax(torch.from_numpy(x), dim)
    np.testing.assert_allclose(y, ty.numpy(), rtol=1e-12)
    ref = torch.ops.aten._softmax_backward_data(torch.from_numpy(dy), ty, dim, torch.float64)
    np.testing.assert_allclose(O.softmax_bwd(dy, y, dim), ref.numpy(), rtol=1e-10, atol=1e-13)


@pytest.mark.parametrize("shape", [(9, 13), (2, 3, 4, 5)])
def test_xent_bwd_matches_autograd(shape):
    rng = np.random.default_rng(4)
    x = rng.standard_normal(shape) * 2
    lab_shape = (shape[0],) + tuple(shape[2:])
    labels = rng.integers(0, shape[1], lab_shape)
    tx = torch.from_numpy(x).requires_grad_(True)
    F.cross_entropy(tx, torch.from_numpy(labels)).backward()
    np.testing.assert_allclose(O.xent_bwd(x, labels), tx.grad.numpy(), rtol=1e-10, atol=1e-13)


# --------------------------------------------------------------- convolution
CONV_CASES = [
    # (x shape, w shape, stride, padding, dilation)
    ((2, 3, 9, 9), (4, 3, 3, 3), 1, 1, 1),
    ((1, 5, 12, 10), (7, 5, 3, 3), 2, 1, 1),
    ((2, 4, 8, 8), (6, 4, 1, 1), 1, 0, 1),
    ((2, 4, 9, 9), (6, 4, 1, 1), 2, 0, 1),
    ((1, 3, 15, 15), (8, 3, 7, 7), 2, 3, 1),
    ((1, 2, 11, 11), (3, 2, 3, 3), 1, 2, 2),
    ((2, 3, 7, 9), (2, 3, 2, 3), (2, 1), (1, 0), 1),
]


@pytest.mark.parametrize("xs,ws,st,pad,dil", CONV_CASES)
def test_conv_oracle_matches_torch(xs, ws, st, pad, dil):
    rng = np.random.default_rng(7)
    x, w = rng.standard_normal(xs), rng.standard_normal(ws)
    b = rng.standard_normal(ws[0])
    tx = torch.from_numpy(x).requires_grad_(True)
    tw = torch.from_numpy(w).requires_grad_(True)
    ty = F.conv2d(tx, tw, torch.from_numpy(b), st, pad, dil)
    y = O.conv_fwd(x, w, b, st, pad, dil)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-11, atol=1e-11)
    dy = rng.standard_normal(y.shape)
    ty.backward(torch.from_numpy(dy))
    np.testing.assert_allclose(O.conv_bwd_data(dy, w, xs, st, pad, dil), tx.grad.numpy(),
                               rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(O.conv_bwd_weight(dy, x, ws, st, pad, dil), tw.grad.numpy(),
                               rtol=1e-11, atol=1e-11)


def test_conv_oracle_brute_force():
    rng = np.random.default_rng(8)
    x, w = rng.standard_normal((1, 2, 5, 6)), rng.standard_normal((3, 2, 3, 2))
    st, pad, dil = (2, 1), (1, 1), (1, 2)
    y = O.conv_fwd(x, w, None, st, pad, dil)
    N, C, H, W = x.shape
    K, _, R, S = w.shape
    for k in range(K):
        for p in range(y.shape[2]):
            for q in range(y.shape[3]):
                acc = 0.0
                for c in range(C):
                    for r in range(R):
                        for s in range(S):
                            h, ww = p * st[0] + r * dil[0] - pad[0], q * st[1] + s * dil[1] - pad[1]
                            if 0 <= h < H and 0 <= ww < W:
                                acc += w[k, c, r, s] * x[0, c, h, ww]
                assert abs(acc - y[0, k, p, q]) < 1e-12
