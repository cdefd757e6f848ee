"""NumPy-facing loader of the CPU oracle (``oracle/singa_cpu_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the CPU-baseline leg
of ``bench.py``; never by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SO = os.path.join(HERE, "libsinga_cpu_oracle.so")
SRC = os.path.join(HERE, "singa_cpu_oracle.c")


def build():
    subprocess.check_call(["make", "-B", "-C", HERE, "libsinga_cpu_oracle.so"])
    return SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(SO):
            build()
        _lib = C.CDLL(SO)
        _lib.oracle_get_threads.restype = C.c_int
    return _lib


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(C.c_void_p)


def _i(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(C.c_void_p)


def _out(shape):
    a = np.empty(shape, dtype=np.float32)
    return a, a.ctypes.data_as(C.c_void_p)


def set_threads(n):
    lib().oracle_set_threads(C.c_int(n))


def get_threads():
    return lib().oracle_get_threads()


def sgemm(A, B, transA=False, transB=False, alpha=1.0, beta=0.0, Cm=None):
    A, pa = _f(A)
    B, pb = _f(B)
    M = A.shape[1] if transA else A.shape[0]
    K = A.shape[0] if transA else A.shape[1]
    N = B.shape[0] if transB else B.shape[1]
    if Cm is None:
        Cm = np.zeros((M, N), dtype=np.float32)
    Cm, pc = _f(Cm)
    lib().oracle_sgemm(C.c_int(transA), C.c_int(transB), C.c_int(M), C.c_int(N), C.c_int(K),
                       C.c_float(alpha), pa, C.c_int(A.shape[1]), pb, C.c_int(B.shape[1]),
                       C.c_float(beta), pc, C.c_int(N))
    return Cm


def relu_fwd(x):
    x, px = _f(x)
    y, py = _out(x.shape)
    lib().oracle_relu_fwd(px, py, C.c_size_t(x.size))
    return y


def relu_bwd(dy, x):
    dy, pd = _f(dy)
    x, px = _f(x)
    dx, po = _out(x.shape)
    lib().oracle_relu_bwd(pd, px, po, C.c_size_t(x.size))
    return dx


def axpy(alpha, x, y):
    """in place on y (must be a contiguous float32 array)"""
    x, px = _f(x)
    assert y.dtype == np.float32 and y.flags.c_contiguous
    lib().oracle_axpy(C.c_float(alpha), px, y.ctypes.data_as(C.c_void_p), C.c_size_t(x.size))
    return y


def eltwise_mult(a, b):
    a, pa = _f(a)
    b, pb = _f(b)
    scalar = b.size == 1 and a.size != 1
    out, po = _out(a.shape)
    lib().oracle_eltwise_mult(pa, pb, C.c_int(scalar), po, C.c_size_t(a.size))
    return out


def add(a, b):
    a, pa = _f(a)
    b, pb = _f(b)
    out, po = _out(a.shape)
    lib().oracle_add(pa, pb, po, C.c_size_t(a.size))
    return out


def sgd_momentum(p, g, v, lr, mu=0.0, damp=0.0, wd=0.0, nesterov=False):
    """in place on p, g, v (float32 contiguous arrays; v may be None when mu == 0)"""
    for a in (p, g) + ((v,) if v is not None else ()):
        assert a.dtype == np.float32 and a.flags.c_contiguous
    pv = v.ctypes.data_as(C.c_void_p) if v is not None else None
    lib().oracle_sgd_momentum(p.ctypes.data_as(C.c_void_p), g.ctypes.data_as(C.c_void_p), pv,
                              C.c_size_t(p.size), C.c_float(lr), C.c_float(mu), C.c_float(damp),
                              C.c_float(wd), C.c_int(bool(nesterov)))


def softmax(x):
    x, px = _f(x)
    batch = x.shape[0] if x.ndim == 2 else 1
    p, pp = _out(x.shape)
    lib().oracle_softmax(px, pp, C.c_size_t(batch), C.c_size_t(x.size // batch))
    return p


def cross_entropy_fwd(p, t):
    p, pp = _f(p)
    t, pt = _i(t)
    batch = p.shape[0] if p.ndim == 2 else 1
    loss, pl = _out((batch,))
    rc = lib().oracle_cross_entropy_fwd(pp, pt, C.c_int(t.size == batch), C.c_size_t(batch),
                                        C.c_size_t(p.size // batch), pl)
    if rc != 0:
        raise ValueError("label out of range (rc=%d)" % rc)
    return loss


def softmax_ce_bwd(p, t, div_by=None):
    """SoftmaxCrossEntropyBwd on a copy of p; div_by applies the reference's ``dx /= N``."""
    g = np.array(p, dtype=np.float32, copy=True, order="C")
    t, pt = _i(t)
    batch = g.shape[0] if g.ndim == 2 else 1
    rc = lib().oracle_softmax_ce_bwd(g.ctypes.data_as(C.c_void_p), pt, C.c_int(t.size == batch),
                                     C.c_size_t(batch), C.c_size_t(g.size // batch))
    if rc != 0:
        raise ValueError("label out of range (rc=%d)" % rc)
    if div_by is not None:
        lib().oracle_div_scalar(g.ctypes.data_as(C.c_void_p), C.c_float(div_by), C.c_size_t(g.size))
    return g


def _conv_out(H, W, R, S, sh, sw, ph, pw):
    return (H + 2 * ph - R) // sh + 1, (W + 2 * pw - S) // sw + 1


def conv_fwd(x, Wt, b, stride, pad):
    x, px = _f(x)
    Wt, pw_ = _f(Wt)
    N, Cc, H, W = x.shape
    K, _, R, S = Wt.shape
    P, Q = _conv_out(H, W, R, S, stride[0], stride[1], pad[0], pad[1])
    y, py = _out((N, K, P, Q))
    pb = None
    if b is not None:
        b, pb = _f(b)
    lib().oracle_conv_fwd(px, pw_, pb, py, *[C.c_int(v) for v in
                                              (N, Cc, H, W, K, R, S, stride[0], stride[1], pad[0], pad[1])])
    return y


def conv_bwd(dy, x, Wt, stride, pad, want_dx=True, want_dw=True):
    dy, pdy = _f(dy)
    x, px = _f(x)
    Wt, pw_ = _f(Wt)
    N, Cc, H, W = x.shape
    K, _, R, S = Wt.shape
    dx = pdx = dw = pdw = None
    if want_dx:
        dx, pdx = _out(x.shape)
    if want_dw:
        dw, pdw = _out(Wt.shape)
    lib().oracle_conv_bwd(pdy, px, pw_, pdx, pdw, *[C.c_int(v) for v in
                                                    (N, Cc, H, W, K, R, S, stride[0], stride[1], pad[0], pad[1])])
    return dx, dw


def conv_fwd_grouped(x, Wt, b, stride, pad, groups):
    """Grouped convolution as its definition: group i convolves input channels [i C/G, (i+1) C/G) with filters
    [i K/G, (i+1) K/G) of the [K, C/G, R, S] weight tensor (the reference runs it through
    cudnnSetConvolutionGroupCount, src/model/operation/convolution.cc:486-490, and has no CPU path for it:
    python/singa/layer.py:668-669).  Each group is one call of the dense convolution above."""
    x = np.asarray(x, np.float32)
    Wt = np.asarray(Wt, np.float32)
    Cg, Kg = x.shape[1] // groups, Wt.shape[0] // groups
    assert Cg * groups == x.shape[1] and Kg * groups == Wt.shape[0] and Wt.shape[1] == Cg
    return np.concatenate([conv_fwd(x[:, i * Cg:(i + 1) * Cg], Wt[i * Kg:(i + 1) * Kg],
                                    None if b is None else b[i * Kg:(i + 1) * Kg], stride, pad)
                           for i in range(groups)], axis=1)


def conv_bwd_grouped(dy, x, Wt, stride, pad, groups):
    """(dx, dW) of the grouped convolution: the dense gradients of each group on its channel slices."""
    dy = np.asarray(dy, np.float32)
    x = np.asarray(x, np.float32)
    Wt = np.asarray(Wt, np.float32)
    Cg, Kg = x.shape[1] // groups, Wt.shape[0] // groups
    parts = [conv_bwd(dy[:, i * Kg:(i + 1) * Kg], x[:, i * Cg:(i + 1) * Cg], Wt[i * Kg:(i + 1) * Kg], stride, pad)
             for i in range(groups)]
    return np.concatenate([p[0] for p in parts], axis=1), np.concatenate([p[1] for p in parts], axis=0)


def conv_bgrad(dy):
    dy, pdy = _f(dy)
    N, K = dy.shape[:2]
    db, pdb = _out((K,))
    lib().oracle_conv_bgrad(pdy, pdb, C.c_int(N), C.c_int(K), C.c_int(dy.size // (N * K)))
    return db


def im2col(im, R, S, pad, stride):
    im, pi = _f(im)
    Cc, H, W = im.shape
    P, Q = _conv_out(H, W, R, S, stride[0], stride[1], pad[0], pad[1])
    col, pc = _out((Cc * R * S, P * Q))
    lib().oracle_im2col(pi, *[C.c_int(v) for v in (Cc, H, W, R, S, pad[0], pad[1], stride[0], stride[1])], pc)
    return col


def pool_max_fwd(x, kernel, stride, pad):
    x, px = _f(x)
    N, Cc, H, W = x.shape
    P, Q = _conv_out(H, W, kernel[0], kernel[1], stride[0], stride[1], pad[0], pad[1])
    y, py = _out((N, Cc, P, Q))
    mask = np.empty((N, Cc, P, Q), dtype=np.int32)
    lib().oracle_pool_max_fwd(px, py, mask.ctypes.data_as(C.c_void_p),
                              *[C.c_int(v) for v in (N, Cc, H, W, kernel[0], kernel[1], stride[0], stride[1],
                                                     pad[0], pad[1])])
    return y, mask


def pool_max_bwd(dy, mask, x_shape):
    dy, pdy = _f(dy)
    mask, pm = _i(mask)
    N, Cc, H, W = x_shape
    dx, pdx = _out(x_shape)
    lib().oracle_pool_max_bwd(pdy, pm, pdx, *[C.c_int(v) for v in (N, Cc, H, W, dy.shape[2], dy.shape[3])])
    return dx


def pool_avg_fwd(x, kernel, stride, pad, include_pad=False):
    x, px = _f(x)
    N, Cc, H, W = x.shape
    P, Q = _conv_out(H, W, kernel[0], kernel[1], stride[0], stride[1], pad[0], pad[1])
    y, py = _out((N, Cc, P, Q))
    lib().oracle_pool_avg_fwd(px, py, *[C.c_int(v) for v in (N, Cc, H, W, kernel[0], kernel[1], stride[0],
                                                             stride[1], pad[0], pad[1], int(include_pad))])
    return y


def pool_avg_bwd(dy, x_shape, kernel, stride, pad, include_pad=False):
    dy, pdy = _f(dy)
    N, Cc, H, W = x_shape
    dx, pdx = _out(x_shape)
    lib().oracle_pool_avg_bwd(pdy, pdx, *[C.c_int(v) for v in (N, Cc, H, W, kernel[0], kernel[1], stride[0],
                                                               stride[1], pad[0], pad[1], int(include_pad))])
    return dx


def bn_fwd_train(x, gamma, beta, running_mean=None, running_var=None, factor=0.9, eps=1e-5):
    """returns y, save_mean, save_invstd; running_* (float32 arrays) are updated in place"""
    x, px = _f(x)
    gamma, pg = _f(gamma)
    beta, pb = _f(beta)
    if x.ndim == 2:
        N, Cc, HW = x.shape[0], x.shape[1], 1
    else:
        N, Cc, HW = x.shape[0], x.shape[1], x.shape[2] * x.shape[3]
    y, py = _out(x.shape)
    sm, psm = _out((Cc,))
    si, psi = _out((Cc,))
    prm = running_mean.ctypes.data_as(C.c_void_p) if running_mean is not None else None
    prv = running_var.ctypes.data_as(C.c_void_p) if running_var is not None else None
    lib().oracle_bn_fwd_train(px, pg, pb, prm, prv, C.c_float(factor), C.c_float(eps), py, psm, psi,
                              C.c_int(N), C.c_int(Cc), C.c_int(HW))
    return y, sm, si


def bn_bwd(dy, x, gamma, save_mean, save_invstd):
    dy, pdy = _f(dy)
    x, px = _f(x)
    gamma, pg = _f(gamma)
    save_mean, psm = _f(save_mean)
    save_invstd, psi = _f(save_invstd)
    if x.ndim == 2:
        N, Cc, HW = x.shape[0], x.shape[1], 1
    else:
        N, Cc, HW = x.shape[0], x.shape[1], x.shape[2] * x.shape[3]
    dx, pdx = _out(x.shape)
    dg, pdg = _out((Cc,))
    db, pdb = _out((Cc,))
    lib().oracle_bn_bwd(pdy, px, pg, psm, psi, pdx, pdg, pdb, C.c_int(N), C.c_int(Cc), C.c_int(HW))
    return dx, dg, db


def sum_rows(m):
    m, pm = _f(m)
    out, po = _out((m.shape[1],))
    lib().oracle_sum_rows(pm, po, C.c_int(m.shape[0]), C.c_int(m.shape[1]))
    return out


# ---- the remaining tensor functions (Transform, RowMax, Dot, Sum) and the seeded input generator

def transform(a, shape, strides):
    """Dense row-major copy of the view (shape, strides in elements) of the flat array `a`."""
    a, pa = _f(a)
    shape = [int(s) for s in shape]
    out, po = _out(shape)
    sh = (C.c_size_t * len(shape))(*shape)
    st = (C.c_long * len(shape))(*[int(s) for s in strides])
    lib().oracle_transform(pa, po, C.c_int(len(shape)), sh, st)
    return out


def row_max(m):
    m, pm = _f(m)
    out, po = _out((m.shape[0],))
    lib().oracle_row_max(pm, po, C.c_size_t(m.shape[0]), C.c_size_t(m.shape[1]))
    return out


def dot(a, b):
    a, pa = _f(a)
    b, pb = _f(b)
    fn = lib().oracle_dot
    fn.restype = C.c_float
    return float(fn(pa, pb, C.c_size_t(a.size)))


def sum_all(a):
    a, pa = _f(a)
    fn = lib().oracle_sum_all
    fn.restype = C.c_float
    return float(fn(pa, C.c_size_t(a.size)))


def rng_raw(seed, k):
    fn = lib().oracle_rng_raw
    fn.restype = C.c_uint64
    return int(fn(C.c_uint64(seed), C.c_uint64(k)))


def rng_uniform(seed, n, low=0.0, high=1.0, offset=0):
    out, po = _out((n,))
    lib().oracle_rng_uniform(C.c_uint64(seed), C.c_uint64(offset), C.c_double(low), C.c_double(high), po, C.c_size_t(n))
    return out


def rng_normal(seed, n, mean=0.0, std=1.0, offset=0):
    out, po = _out((n,))
    lib().oracle_rng_normal(C.c_uint64(seed), C.c_uint64(offset), C.c_double(mean), C.c_double(std), po, C.c_size_t(n))
    return out


def rng_integers(seed, n, hi, offset=0):
    out = np.empty(n, dtype=np.int32)
    lib().oracle_rng_integers(C.c_uint64(seed), C.c_uint64(offset), C.c_uint64(hi), out.ctypes.data_as(C.c_void_p),
                              C.c_size_t(n))
    return out
