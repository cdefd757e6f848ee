"""Pins the CPU oracle where the reference's own vectors leave room: brute force on tiny inputs,
adjoint identities, float64 closed forms and textbook library routines (torch CPU autograd).
Each check is chosen so that a dropped term, a wrong sign/index or a transposed operand fails."""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import cpu_oracle as O
from util import nl2, randn, rng

CONV_CASES = [
    # N, C, H, W, K, R, S, stride, pad
    (2, 3, 7, 6, 4, 3, 3, (1, 1), (1, 1)),
    (2, 3, 9, 8, 5, 3, 3, (2, 2), (1, 1)),
    (1, 2, 8, 8, 3, 1, 1, (2, 2), (0, 0)),
    (2, 3, 11, 10, 4, 5, 5, (1, 1), (2, 2)),
    (1, 3, 15, 14, 2, 7, 7, (2, 2), (3, 3)),
    (2, 2, 6, 7, 3, 3, 2, (2, 1), (0, 1)),   # non-square everything
    (1, 1, 5, 5, 1, 3, 3, (1, 1), (2, 2)),   # padding larger than needed
    (2, 2, 8, 8, 2, 3, 3, (3, 3), (1, 1)),   # stride that does not tile the image exactly
]


def direct_conv(x, w, stride, pad):
    """7-loop direct convolution in float64."""
    N, C, H, W = x.shape
    K, _, R, S = w.shape
    P = (H + 2 * pad[0] - R) // stride[0] + 1
    Q = (W + 2 * pad[1] - S) // stride[1] + 1
    y = np.zeros((N, K, P, Q))
    for n, k, p, q, c, r, s in itertools.product(range(N), range(K), range(P), range(Q), range(C), range(R), range(S)):
        h, ww = p * stride[0] - pad[0] + r, q * stride[1] - pad[1] + s
        if 0 <= h < H and 0 <= ww < W:
            y[n, k, p, q] += float(x[n, c, h, ww]) * float(w[k, c, r, s])
    return y


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_against_brute_force_and_adjoints(case):
    N, C, H, W, K, R, S, stride, pad = case
    r = rng(hash(case) % 2**31)
    x, w = randn(r, N, C, H, W), randn(r, K, C, R, S)
    b = randn(r, K)
    y = O.conv_fwd(x, w, b, stride, pad)
    yd = direct_conv(x, w, stride, pad) + b.reshape(1, K, 1, 1)
    assert nl2(y, yd) < 1e-6
    dy = randn(r, *y.shape)
    dx, dw = O.conv_bwd(dy, x, w, stride, pad)
    # adjoint identities: <conv(x, w), dy> = <x, dgrad> = <w, wgrad>
    y0 = direct_conv(x, w, stride, pad)
    lhs = float((y0 * dy).sum())
    assert abs(lhs - float((x.astype(np.float64) * dx).sum())) < 1e-4 * max(1, abs(lhs))
    assert abs(lhs - float((w.astype(np.float64) * dw).sum())) < 1e-4 * max(1, abs(lhs))
    # and elementwise against the textbook library routine
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    F.conv2d(xt, wt, None, stride, pad).backward(torch.tensor(dy, dtype=torch.float64))
    assert nl2(dx, xt.grad.numpy()) < 1e-6
    assert nl2(dw, wt.grad.numpy()) < 1e-6
    np.testing.assert_allclose(O.conv_bgrad(dy), dy.astype(np.float64).sum(axis=(0, 2, 3)), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("case", [(2, 4, 6, 5, 6, 3, 3, (1, 1), (1, 1), 2), (3, 6, 7, 7, 6, 3, 3, (2, 2), (1, 1), 6),
                                  (2, 8, 5, 6, 4, 1, 1, (1, 1), (0, 0), 4), (1, 6, 9, 8, 9, 5, 3, (2, 1), (2, 1), 3)])
def test_grouped_conv_against_torch(case):
    """The grouped convolution of the oracle (per-group calls of the dense functions) against an independent
    implementation: torch's conv2d with `groups` in float64 and its autograd."""
    import torch
    N, C, H, W, K, R, S, stride, pad, G = case
    r = np.random.default_rng(sum(case[:7]) + G)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = r.standard_normal((K, C // G, R, S)).astype(np.float32)
    b = r.standard_normal(K).astype(np.float32)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tw = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    ty = torch.nn.functional.conv2d(tx, tw, torch.tensor(b, dtype=torch.float64), stride, pad, 1, G)
    y = O.conv_fwd_grouped(x, w, b, stride, pad, G)
    assert y.shape == tuple(ty.shape) and nl2(y, ty.detach().numpy()) < 1e-6
    dy = r.standard_normal(y.shape).astype(np.float32)
    ty.backward(torch.tensor(dy, dtype=torch.float64))
    dx, dw = O.conv_bwd_grouped(dy, x, w, stride, pad, G)
    assert nl2(dx, tx.grad.numpy()) < 1e-6 and nl2(dw, tw.grad.numpy()) < 1e-6


def test_im2col_matches_definition():
    r = rng(3)
    im = randn(r, 2, 5, 4)
    col = O.im2col(im, 3, 2, (1, 0), (2, 1))
    P, Q = (5 + 2 - 3) // 2 + 1, (4 - 2) // 1 + 1
    assert col.shape == (2 * 3 * 2, P * Q)
    for c, rr, s, p, q in itertools.product(range(2), range(3), range(2), range(P), range(Q)):
        h, w = p * 2 - 1 + rr, q + s
        exp = im[c, h, w] if 0 <= h < 5 and 0 <= w < 4 else 0.0
        assert col[(c * 3 + rr) * 2 + s, p * Q + q] == exp


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_sgemm(ta, tb):
    r = rng(10 + 2 * ta + tb)
    M, N, K = 37, 29, 53
    A = randn(r, *((K, M) if ta else (M, K)))
    B = randn(r, *((N, K) if tb else (K, N)))
    C0 = randn(r, M, N)
    out = O.sgemm(A, B, bool(ta), bool(tb), alpha=0.5, beta=2.0, Cm=C0.copy())
    A64, B64 = A.astype(np.float64), B.astype(np.float64)
    exp = 0.5 * (A64.T if ta else A64) @ (B64.T if tb else B64) + 2.0 * C0
    assert nl2(out, exp) < 1e-6


POOL_CASES = [
    # N, C, H, W, kernel, stride, pad
    (2, 3, 8, 8, (2, 2), (2, 2), (0, 0)),
    (2, 2, 9, 9, (3, 3), (2, 2), (1, 1)),     # ResNet stem shape class: overlapping + padded
    (1, 2, 7, 5, (3, 2), (1, 2), (1, 0)),
    (1, 1, 7, 7, (7, 7), (1, 1), (0, 0)),
    (2, 2, 6, 6, (2, 2), (3, 3), (0, 0)),     # stride > kernel: some inputs in no window
]


def naive_max_pool_bwd(x, dy, kernel, stride, pad):
    N, C, H, W = x.shape
    P, Q = dy.shape[2:]
    dx = np.zeros_like(x)
    for n, c, p, q in itertools.product(range(N), range(C), range(P), range(Q)):
        best, bi = -np.inf, None
        for h in range(max(p * stride[0] - pad[0], 0), min(p * stride[0] - pad[0] + kernel[0], H)):
            for w in range(max(q * stride[1] - pad[1], 0), min(q * stride[1] - pad[1] + kernel[1], W)):
                if x[n, c, h, w] > best:
                    best, bi = x[n, c, h, w], (h, w)
        dx[n, c, bi[0], bi[1]] = np.float32(dx[n, c, bi[0], bi[1]] + dy[n, c, p, q])
    return dx


@pytest.mark.parametrize("case", POOL_CASES)
@pytest.mark.parametrize("ties", [False, True])
def test_max_pool(case, ties):
    N, C, H, W, kernel, stride, pad = case
    r = rng(7)
    x = randn(r, N, C, H, W)
    if ties:  # few distinct values -> many ties: first maximum in row-major order must win
        x = np.round(x).astype(np.float32)
    y, mask = O.pool_max_fwd(x, kernel, stride, pad)
    dy = randn(r, *y.shape)
    dx = O.pool_max_bwd(dy, mask, x.shape)
    assert np.array_equal(dx, naive_max_pool_bwd(x, dy, kernel, stride, pad))
    yt = F.max_pool2d(torch.tensor(x), kernel, stride, pad)
    assert np.array_equal(y, yt.numpy())
    assert abs(float(dx.sum()) - float(dy.sum())) < 1e-3  # every dy lands somewhere exactly once


@pytest.mark.parametrize("case", POOL_CASES)
def test_avg_pool_exclude_pad(case):
    N, C, H, W, kernel, stride, pad = case
    r = rng(8)
    x = randn(r, N, C, H, W)
    y = O.pool_avg_fwd(x, kernel, stride, pad, include_pad=False)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    yt = F.avg_pool2d(xt, kernel, stride, pad, count_include_pad=False)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-5, atol=1e-6)
    dy = randn(r, *y.shape)
    yt.backward(torch.tensor(dy, dtype=torch.float64))
    dx = O.pool_avg_bwd(dy, x.shape, kernel, stride, pad, include_pad=False)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-5, atol=1e-6)


def test_avg_pool_include_pad_divisor():
    x = np.ones((1, 1, 4, 4), np.float32)
    y = O.pool_avg_fwd(x, (3, 3), (1, 1), (1, 1), include_pad=True)
    assert y[0, 0, 0, 0] == np.float32(4 / 9) and y[0, 0, 1, 1] == 1
    y = O.pool_avg_fwd(x, (3, 3), (1, 1), (1, 1), include_pad=False)
    assert np.all(y == 1)


@pytest.mark.parametrize("shape", [(4, 3, 5, 6), (2, 5, 7, 7), (8, 4, 1, 1), (16, 6)])
def test_batchnorm_closed_form(shape):
    r = rng(11)
    x = (randn(r, *shape) * 3 + 1.5).astype(np.float32)
    C = shape[1]
    gamma, beta = randn(r, C) + 1, randn(r, C)
    rm, rv = randn(r, C), np.abs(randn(r, C))
    rm0, rv0 = rm.copy(), rv.copy()
    y, mean, invstd = O.bn_fwd_train(x, gamma, beta, rm, rv, factor=0.1)
    axes = (0,) if len(shape) == 2 else (0, 2, 3)
    xs = x.astype(np.float64)
    m, v = xs.mean(axis=axes), xs.var(axis=axes)
    M = x.size // C
    bshape = (1, C) + (1,) * (len(shape) - 2)
    np.testing.assert_allclose(mean, m, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(invstd, 1 / np.sqrt(v + 1e-5), rtol=1e-5)
    np.testing.assert_allclose(rm, 0.9 * rm0 + 0.1 * m, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(rv, 0.9 * rv0 + 0.1 * v * M / (M - 1), rtol=1e-5, atol=1e-6)
    xhat = (xs - m.reshape(bshape)) / np.sqrt(v.reshape(bshape) + 1e-5)
    assert nl2(y, xhat * gamma.reshape(bshape) + beta.reshape(bshape)) < 1e-6
    # backward against autograd of the textbook definition
    dy = randn(r, *shape)
    xt = torch.tensor(xs, requires_grad=True)
    gt = torch.tensor(gamma, dtype=torch.float64, requires_grad=True)
    bt = torch.tensor(beta, dtype=torch.float64, requires_grad=True)
    F.batch_norm(xt, None, None, gt, bt, True, 0.1, 1e-5).backward(torch.tensor(dy, dtype=torch.float64))
    dx, dg, db = O.bn_bwd(dy, x, gamma, mean, invstd)
    assert nl2(dx, xt.grad.numpy()) < 1e-5
    assert nl2(dg, gt.grad.numpy()) < 1e-5
    assert nl2(db, bt.grad.numpy()) < 1e-5


def test_softmax_ce_closed_form():
    r = rng(12)
    x = randn(r, 9, 17) * 4
    p = O.softmax(x)
    xs = x.astype(np.float64)
    e = np.exp(xs - xs.max(axis=1, keepdims=True))
    np.testing.assert_allclose(p, e / e.sum(axis=1, keepdims=True), rtol=2e-6)
    t = r.integers(0, 17, size=9).astype(np.int32)
    onehot = np.eye(17, dtype=np.int32)[t]
    np.testing.assert_allclose(O.cross_entropy_fwd(p, t), -np.log(p[np.arange(9), t].astype(np.float64)), rtol=1e-6)
    g1, g2 = O.softmax_ce_bwd(p, t), O.softmax_ce_bwd(p, onehot)
    assert np.array_equal(g1, g2) and np.array_equal(g1, (p - onehot).astype(np.float32))
    # multi-hot target: normalised by its row sum
    multi = onehot.copy()
    multi[:, 0] += 1
    np.testing.assert_allclose(O.softmax_ce_bwd(p, multi), p - multi / multi.sum(axis=1, keepdims=True), rtol=1e-6,
                               atol=1e-7)
    # the /N that autograd applies is a multiply by the fp32 reciprocal
    g3 = O.softmax_ce_bwd(p, t, div_by=9)
    assert np.array_equal(g3, g1 * np.float32(np.float32(1) / np.float32(9)))


def test_sgd_momentum_float64_trajectory():
    r = rng(13)
    p, g0 = randn(r, 1000), randn(r, 1000)
    for nesterov, damp, wd in [(False, 0.0, 0.0), (False, 0.1, 0.01), (True, 0.0, 0.001)]:
        pp, v = p.copy(), np.zeros(1000, np.float32)
        p64, v64 = p.astype(np.float64), np.zeros(1000)
        for step in range(3):
            g = (g0 * (step + 1)).astype(np.float32)
            O.sgd_momentum(pp, g.copy(), v, 0.05, mu=0.9, damp=damp, wd=wd, nesterov=nesterov)
            g64 = g.astype(np.float64) + wd * p64
            v64 = 0.9 * v64 + (1 - damp) * g64
            p64 = p64 - 0.05 * ((g64 + 0.9 * v64) if nesterov else v64)
        np.testing.assert_allclose(pp, p64, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(v, v64, rtol=1e-5, atol=1e-6)


def test_elementwise_definitions():
    r = rng(14)
    a, b = randn(r, 1001), randn(r, 1001)
    assert np.array_equal(O.add(a, b), a + b)
    assert np.array_equal(O.eltwise_mult(a, b), a * b)
    assert np.array_equal(O.eltwise_mult(a, np.array([0.9], np.float32)), a * np.float32(0.9))
    y = b.copy()
    O.axpy(0.3, a, y)
    assert np.array_equal(y, b + np.float32(0.3) * a)
    assert np.array_equal(O.sum_rows(a[:1000].reshape(10, 100)),
                          np.add.reduce(a[:1000].reshape(10, 100), axis=0, dtype=np.float32))


# ---- the remaining tensor functions and the seeded generator

def test_transform_walks_a_view_like_numpy():
    r = np.random.default_rng(3)
    a = r.standard_normal(4 * 5 * 6).astype(np.float32)
    cube = a.reshape(4, 5, 6)
    # transposed, sliced with a step, broadcast (stride 0), and all at once
    for view in (cube.transpose(2, 0, 1), cube[:, ::2, 1:5], np.broadcast_to(cube[:, :1, :], (4, 7, 6)),
                 np.broadcast_to(cube.transpose(1, 2, 0)[None, :, ::3, :], (3, 5, 2, 4)), cube[1:2, 2, 3:4]):
        strides = [s // 4 for s in view.strides]
        base = (view.__array_interface__["data"][0] - a.__array_interface__["data"][0]) // 4
        got = O.transform(a[base:], view.shape, strides)
        assert np.array_equal(got, np.ascontiguousarray(view))


def test_row_max_starts_from_zero():
    m = np.array([[-3.0, -1.0, -2.0], [0.5, 4.0, -7.0], [0.0, 0.0, 0.0]], np.float32)
    assert np.array_equal(O.row_max(m), np.array([0.0, 4.0, 0.0], np.float32))   # not -1: the maximum starts at 0
    r = np.random.default_rng(5).standard_normal((37, 101)).astype(np.float32)
    assert np.array_equal(O.row_max(r), np.maximum(0, r.max(axis=1)))


def test_dot_and_sum_against_float64():
    r = np.random.default_rng(6)
    for n in (1, 17, 4096, 100003):
        a, b = r.standard_normal(n).astype(np.float32), r.standard_normal(n).astype(np.float32)
        assert abs(O.dot(a, b) - float(a.astype(np.float64) @ b.astype(np.float64))) <= 1e-6 * float(np.abs(a * b).sum()) + 1e-12
        assert abs(O.sum_all(a) - float(a.astype(np.float64).sum())) <= 1e-6 * float(np.abs(a).sum()) + 1e-12
    assert O.dot(np.zeros(0, np.float32), np.zeros(0, np.float32)) == 0.0


def test_seeded_generator_twins_and_known_answers():
    """splitmix64's published first outputs for seed 0 and for seed 1234567 (the reference C
    program by its author prints them), the C and NumPy twins agreeing bit for bit, and the
    moments of the derived distributions."""
    from singa_amd import rng
    assert [O.rng_raw(0, k) for k in range(3)] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    assert [O.rng_raw(1234567, k) for k in range(3)] == [6457827717110365317, 3203168211198807973, 9817491932198370423]
    ks = np.arange(1000, dtype=np.uint64)
    assert [int(v) for v in rng.raw(99, ks)] == [O.rng_raw(99, int(k)) for k in ks]
    assert int(rng.raw(0xFFFFFFFFFFFFFFFF, 5)) == O.rng_raw(0xFFFFFFFFFFFFFFFF, 5)      # wrap-around of the state
    n = 200000
    z_c, z_py = O.rng_normal(0x5167A400, n), rng.normal(0x5167A400, (n,))
    assert (z_c.view(np.uint32) != z_py.view(np.uint32)).sum() <= 2      # libm vs NumPy: a last-place flip at most, rarely
    assert abs(z_py.mean()) < 0.01 and abs(z_py.std() - 1) < 0.01 and abs((z_py ** 4).mean() - 3) < 0.1
    assert np.array_equal(z_py[:1000], rng.normal(0x5167A400, (1000,)))  # a smaller tensor is a prefix
    assert np.array_equal(rng.normal(7, (10,), offset=2 * 5)[:5], rng.normal(7, (15,))[5:10])   # offsets continue a stream
    u = rng.uniform(5, (n,), -1.0, 3.0)
    assert np.array_equal(u, O.rng_uniform(5, n, -1.0, 3.0)) and u.min() >= -1 and u.max() < 3 and abs(u.mean() - 1) < 0.02
    k = rng.integers(11, (n,), 1000)
    assert np.array_equal(k, O.rng_integers(11, n, 1000)) and k.min() == 0 and k.max() == 999
    assert abs(np.bincount(k, minlength=1000).std() - np.sqrt(n / 1000)) < 3
