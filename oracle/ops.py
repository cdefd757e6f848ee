"""The whole-step drivers' "ops" interface implemented on NumPy arrays by the CPU oracle.

TEST INFRASTRUCTURE ONLY (tests/, the smoke check, the CPU-baseline leg of bench.py)."""
import numpy as np

from . import cpu_oracle as O


class _ConvH(object):
    def __init__(self, kernel, stride, pad):
        self.kernel, self.stride, self.pad = tuple(kernel), tuple(stride), tuple(pad)


class _PoolH(object):
    def __init__(self, kernel, stride, pad, is_max):
        self.kernel, self.stride, self.pad, self.is_max = tuple(kernel), tuple(stride), tuple(pad), is_max
        self.mask = None


class _SGD(object):
    """python/singa/opt.py:269-310 through oracle_sgd_momentum."""

    def __init__(self, lr, momentum):
        self.lr, self.momentum, self.moments = lr, momentum, {}

    def apply(self, name, p, g):
        v = None
        if self.momentum != 0:
            if name not in self.moments:
                self.moments[name] = np.zeros_like(p)
            v = self.moments[name]
        O.sgd_momentum(p.reshape(-1), np.array(g, np.float32).reshape(-1), None if v is None else v.reshape(-1),
                       self.lr, mu=self.momentum)

    def apply_all(self, items):
        for n, p, g in items:
            self.apply(n, p, g)

    def step(self):
        pass


class OracleOps(object):
    name = "cpu-oracle"

    def from_numpy(self, a):
        a = np.asarray(a)
        return np.array(a, dtype=np.int32 if a.dtype.kind == "i" else np.float32, order="C", copy=True)

    def to_numpy(self, t):
        return t

    def reshape(self, t, shape):
        return t.reshape(shape)

    def shape(self, t):
        return tuple(t.shape)

    def sync(self):
        pass

    def conv_handle(self, x, kernel, stride, pad, cin, cout, bias):
        return _ConvH(kernel, stride, pad)

    def bn_handle(self, momentum, x):
        return momentum

    def pool_handle(self, x, kernel, stride, pad, is_max):
        return _PoolH(kernel, stride, pad, is_max)

    def conv_fwd(self, x, W, b, h):
        return O.conv_fwd(x, W, b, h.stride, h.pad)

    def bn_fwd_train(self, h, x, g, b, rm, rv):
        return list(O.bn_fwd_train(x, g, b, rm, rv, factor=h))

    def pool_fwd(self, h, x):
        if h.is_max:
            y, h.mask = O.pool_max_fwd(x, h.kernel, h.stride, h.pad)
            return y
        return O.pool_avg_fwd(x, h.kernel, h.stride, h.pad, include_pad=False)

    def relu(self, x):
        return O.relu_fwd(x)

    def matmul(self, x, W):
        return O.sgemm(x, W)

    def add_bias(self, x, b):
        x += b.reshape(1, -1)
        return x

    def add(self, a, b):
        return O.add(a, b)

    def softmax(self, x):
        return O.softmax(x)

    def ce_fwd(self, p, t):
        return O.cross_entropy_fwd(p, t)

    def softmax_ce_bwd(self, p, t, batch):
        return O.softmax_ce_bwd(p, t, div_by=batch)

    def matmul_bwd(self, dy, x, W):
        return O.sgemm(dy, W, transB=True), O.sgemm(x, dy, transA=True)

    def sum0(self, dy):
        return O.sum_rows(dy)

    def relu_bwd(self, dy, x):
        return O.relu_bwd(dy, x)

    def pool_bwd(self, h, dy, x, y):
        if h.is_max:
            return O.pool_max_bwd(dy, h.mask, x.shape)
        return O.pool_avg_bwd(dy, x.shape, h.kernel, h.stride, h.pad, include_pad=False)

    def bn_bwd(self, h, dy, x, g, mean, var):
        return list(O.bn_bwd(dy, x, g, mean, var))

    def conv_bwd_x(self, dy, W, x, h):
        return O.conv_bwd(dy, x, W, h.stride, h.pad, want_dw=False)[0]

    def conv_bwd_w(self, dy, x, W, h):
        return O.conv_bwd(dy, x, W, h.stride, h.pad, want_dx=False)[1]

    def conv_bwd_b(self, dy, b, h):
        return O.conv_bgrad(dy)

    def accumulate(self, a, b):
        a[...] = O.add(a, b)
        return a

    def make_sgd(self, lr, momentum):
        return _SGD(lr, momentum)
