"""16-bit storage variants (binary16 and bfloat16) of the elementwise backward ops and the casts,
checked bit for bit against numpy: numpy's float32 -> float16 conversion rounds to nearest even, as
the kernels do, and the bfloat16 reference rounding is written out in singa_wrap.float_to_bf16_bits.
(The reference has no CPU half arithmetic to restate: its half_float type is "for labeling only",
src/core/tensor/tensor_math_cuda.h:195; the CUDA kernels compute in fp32 and round once.)"""
import numpy as np
import pytest

from util import rng

pytestmark = pytest.mark.gpu

@pytest.fixture(scope="module")
def singa():
    from singa_amd import singa_wrap
    return singa_wrap


SIZES = [0, 1, 7, 8, 9, 1000, 4096 + 3, 64 * 1024 + 5, 3 * 1000 * 1000 + 1]


def _special(r, n):
    """N(0,1) values salted with zeros, signed zeros, subnormals, huge values, infinities and NaN."""
    a = r.standard_normal(n).astype(np.float32)
    if n >= 64:
        a[1:64:7] = [0.0, -0.0, 1e-7, -1e-7, 6.0e-5, 65504.0, 65520.0, 1e38, np.inf][: len(a[1:64:7])]
        a[5] = np.nan
    return a


def _to(singa, dev, a32, kind):
    if kind == "f16":
        with np.errstate(over="ignore"):
            h = a32.astype(np.float16)
        return singa.from_numpy(h, dev), h.astype(np.float32)
    bits = singa.float_to_bf16_bits(a32)
    t = singa.Tensor(a32.shape, dev, singa.kBFloat16)
    t.CopyHalfDataFromHostPtr(bits)
    return t, singa.bf16_bits_to_float(bits)


def _round(singa, a32, kind):
    """fp32 result -> the values the 16-bit store keeps (as float32)."""
    if kind == "f16":
        with np.errstate(over="ignore"):
            return a32.astype(np.float16).astype(np.float32)
    return singa.bf16_bits_to_float(singa.float_to_bf16_bits(a32))


def _same_bits(got, want, what):
    g, w = np.asarray(got, np.float32).ravel(), np.asarray(want, np.float32).ravel()
    both_nan = np.isnan(g) & np.isnan(w)
    bad = (g.view(np.uint32) != w.view(np.uint32)) & ~both_nan
    assert not bad.any(), "%s: %d of %d differ, first at %d: %r vs %r" % (
        what, bad.sum(), g.size, np.argmax(bad), g[np.argmax(bad)], w[np.argmax(bad)])


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("n", SIZES)
def test_casts(singa, dev, kind, n):
    r = rng(n)
    a = _special(r, n)
    dtype = singa.kFloat16 if kind == "f16" else singa.kBFloat16
    t = singa.from_numpy(a, dev).AsType(dtype)
    assert t.data_type() == dtype and t.MemSize() == 2 * n
    _same_bits(t.to_numpy(), _round(singa, a, kind), "fp32 -> " + kind)
    back = t.AsType(singa.kFloat32)
    _same_bits(back.to_numpy(), _round(singa, a, kind), kind + " -> fp32")


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("n", SIZES)
def test_relu_backward_add_mult_axpy(singa, dev, kind, n):
    r = rng(1000 + n)
    dyt, dy = _to(singa, dev, _special(r, n), kind)
    xt, x = _to(singa, dev, _special(r, n), kind)
    # ReLU backward: a select, so exact; gradient 0 at x == 0 (and at -0.0, NaN)
    _same_bits(singa.ReLUBackward(dyt, xt).to_numpy(), np.where(x > 0, dy, np.float32(0)), "relu_bwd " + kind)
    # ReLU backward of a gradient in two summands: the fp32 sum rounded once, then the select
    d1t, d1 = _to(singa, dev, _special(r, n), kind)
    with np.errstate(invalid="ignore", over="ignore"):
        want = np.where(x > 0, _round(singa, dy + d1, kind), np.float32(0))
    _same_bits(singa.ReLUBackwardSum(dyt, d1t, xt).to_numpy(), want, "relu_bwd_add " + kind)
    with np.errstate(invalid="ignore", over="ignore"):
        _same_bits(singa.__add__(dyt, xt).to_numpy(), _round(singa, dy + x, kind), "add " + kind)
        _same_bits(singa.EltwiseMult(dyt, xt).to_numpy(), _round(singa, dy * x, kind), "mult " + kind)
        alpha = np.float32(-0.05)
        want = _round(singa, x + alpha * dy, kind)     # two fp32 roundings, then the storage rounding
        singa.Axpy(float(alpha), dyt, xt)              # xt += alpha * dyt
        _same_bits(xt.to_numpy(), want, "axpy " + kind)
    # in place accumulate (gradient fan-in)
    at, a = _to(singa, dev, r.standard_normal(n).astype(np.float32), kind)
    bt, b = _to(singa, dev, r.standard_normal(n).astype(np.float32), kind)
    at += bt
    _same_bits(at.to_numpy(), _round(singa, a + b, kind), "iadd " + kind)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("n", SIZES)
def test_relu_forward_16bit(singa, dev, kind, n):
    """ReLU on a half tensor (src/core/tensor/math_kernel.cu:242-251: in > 0 ? in : 0): a select on the
    stored values, so exact; -0.0, NaN and negative values give +0."""
    xt, x = _to(singa, dev, _special(rng(77 + n), n), kind)
    _same_bits(singa.ReLU(xt).to_numpy(), np.where(x > 0, x, np.float32(0)), "relu_fwd " + kind)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("batch,dim", [(1, 1), (3, 10), (128, 10), (64, 1000), (5, 4097)])
def test_softmax_cross_entropy_backward_16bit(singa, dev, kind, batch, dim):
    """SoftmaxCrossEntropyBwd on half probabilities (src/core/tensor/math_kernel.cu:588-611): the fp32
    oracle applied to the stored values, its result rounded once -- bit for bit; label handling as in fp32
    (index targets, array targets normalised by their row sum, out-of-range labels flagged and skipped)."""
    from oracle import cpu_oracle as O
    r = rng(batch * 31 + dim)
    logits = r.standard_normal((batch, dim)).astype(np.float32)
    p32 = np.exp(logits - logits.max(axis=1, keepdims=True))
    p32 = (p32 / p32.sum(axis=1, keepdims=True)).astype(np.float32)
    pt, p = _to(singa, dev, p32, kind)
    labels = r.integers(0, dim, size=batch).astype(np.int32)
    lt = singa.Tensor((batch,), dev, singa.kInt)
    lt.CopyIntDataFromHostPtr(labels)
    for scale in (1.0, 1.0 / batch):
        want = O.softmax_ce_bwd(p, labels) * np.float32(scale)
        _same_bits(singa.SoftmaxCrossEntropyBwd(pt, lt, scale).to_numpy(), _round(singa, want, kind),
                   "softmax-CE bwd, index target, " + kind)
    assert singa.LabelErrors(dev) == 0
    # array target (multi-hot rows, each normalised by its sum); with dim == 1 the reference cannot tell it from an
    # index target (int_target = t.Size() == batch, src/core/tensor/tensor.cc:1741-1758)
    if dim > 1:
        hot = (r.random((batch, dim)) < 0.3).astype(np.int32)
        hot[np.arange(batch), labels] = 1          # no empty row
        ht = singa.Tensor((batch, dim), dev, singa.kInt)
        ht.CopyIntDataFromHostPtr(hot)
        want = O.softmax_ce_bwd(p, hot)
        _same_bits(singa.SoftmaxCrossEntropyBwd(pt, ht).to_numpy(), _round(singa, want, kind),
                   "softmax-CE bwd, array target, " + kind)
    # a label out of range leaves its row as p and is counted
    if batch >= 3:
        bad = labels.copy()
        bad[1] = dim
        bad[2] = -1
        lt.CopyIntDataFromHostPtr(bad)
        got = singa.SoftmaxCrossEntropyBwd(pt, lt).to_numpy()
        _same_bits(got[1:3], p[1:3], "rows of out-of-range labels")
        assert singa.LabelErrors(dev) == 2


def _gemm_case(singa, dev, kind, M, N, K, tA, tB, r):
    """A (M x K) and B (K x N) as the stored matrices a transposed view reads: [K][M] / [N][K]."""
    a32 = (r.standard_normal((M, K)) / np.sqrt(max(K, 1))).astype(np.float32)
    b32 = r.standard_normal((K, N)).astype(np.float32)
    at, a = _to(singa, dev, np.ascontiguousarray(a32.T) if tA else a32, kind)
    bt, b = _to(singa, dev, np.ascontiguousarray(b32.T) if tB else b32, kind)
    A = at.T() if tA else at
    B = bt.T() if tB else bt
    got = singa.Mult(A, B)
    assert got.data_type() == at.data_type() and got.shape() == [M, N]
    want = (a.T if tA else a).astype(np.float64) @ (b.T if tB else b).astype(np.float64)
    return got, want


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (5, 7, 3), (64, 64, 32), (65, 63, 33), (128, 1000, 2048), (128, 2048, 1000),
                                   (2048, 1000, 128), (100, 10, 4096), (3, 130, 257)])
def test_gemm_16bit(singa, dev, kind, M, N, K):
    """Mult on half matrices (cublasHgemm in the reference, tensor_math_cuda.h:1163-1187) for the four
    transpose combinations: exact products of the stored values accumulated in fp32, one rounding -- held to
    1e-2 normalised L2 against float64 (observed: the rounding of the result, 3e-4 / 2.5e-3), and to the
    rounded float64 result within two units of the storage type's last place element by element."""
    from util import nl2
    r = rng(M * 7 + N * 3 + K)
    for tA in (False, True):
        for tB in (False, True):
            got, want = _gemm_case(singa, dev, kind, M, N, K, tA, tB, r)
            g = got.to_numpy().astype(np.float64)
            assert nl2(g, want) <= 1e-2, (tA, tB, nl2(g, want))
            ulp = (2.0 ** -10 if kind == "f16" else 2.0 ** -7) * np.maximum(np.abs(want), 1e-3)
            assert np.all(np.abs(g - want) <= 2 * ulp + 1e-4), (tA, tB, float(np.max(np.abs(g - want) / ulp)))
    # run-to-run identical, and a unit matrix reproduces the other operand bit for bit
    r = rng(5)
    eye = np.eye(64, dtype=np.float32)
    b32 = r.standard_normal((64, 96)).astype(np.float32)
    et, _ = _to(singa, dev, eye, kind)
    bt, b = _to(singa, dev, b32, kind)
    _same_bits(singa.Mult(et, bt).to_numpy(), b, "I * B")
    _same_bits(singa.Mult(et, bt).to_numpy(), singa.Mult(et, bt).to_numpy(), "run to run")


def test_gemm_16bit_alpha_beta_and_pitches(singa, dev):
    """The C ABI directly: alpha / beta in fp32, row pitches larger than the rows, unaligned pointers
    (the element-wise staging path) against float64."""
    import ctypes as C
    from singa_amd import _lib
    r = rng(9)
    M, N, K, lda, ldb, ldc = 37, 29, 45, 51, 33, 40
    A = r.standard_normal((M, lda)).astype(np.float16)
    B = r.standard_normal((K, ldb)).astype(np.float16)
    C0 = r.standard_normal((M, ldc)).astype(np.float16)
    # one leading element of padding makes every base pointer 2-byte aligned only
    def dev_of(a):
        t = singa.from_numpy(np.concatenate([[np.float16(0)], a.ravel()]).astype(np.float16), dev)
        return t, t.ptr + 2
    at, ap = dev_of(A)
    bt, bp = dev_of(B)
    ct, cp = dev_of(C0)
    _lib.check(_lib.lib().sgh_gemm_f16(0, 0, M, N, K, 0.5, ap, lda, bp, ldb, -2.0, cp, ldc, dev.stream), "sgh_gemm_f16")
    got = ct.to_numpy()[1:].reshape(M, ldc).astype(np.float64)
    want = 0.5 * (A[:, :K].astype(np.float64) @ B[:, :N].astype(np.float64)) - 2.0 * C0[:, :N].astype(np.float64)
    assert np.max(np.abs(got[:, :N] - want)) <= 2.0 ** -9 * np.max(np.abs(want)) + 1e-3
    # the padding columns of C are untouched
    assert np.array_equal(got[:, N:], C0[:, N:].astype(np.float64))
    # bad arguments are rejected on the host
    assert _lib.lib().sgh_gemm_f16(0, 0, M, N, K, 1.0, ap, K - 1, bp, ldb, 0.0, cp, ldc, dev.stream) < 0
    assert _lib.lib().sgh_gemm_f16(0, 0, M, N, K, 1.0, ap, lda, bp, ldb, 0.0, cp, N - 1, dev.stream) < 0


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(4, 3, 5, 6), (2, 5, 7, 7), (8, 64, 28, 28), (16, 32, 8, 8), (3, 7, 4, 2),
                                   (16, 24, 14, 14), (2, 8, 6, 6),    # these two: planes of 8-byte vectors
                                   (8, 128, 14, 14), (16, 256, 7, 7), (4, 130, 5, 6), (32, 128, 8, 8),   # one-pass backward
                                   (128, 8, 7, 7), (96, 16, 5, 5)])    # ... ragged planes, a channel in several slices
def test_batchnorm_16bit_storage(singa, dev, kind, shape):
    """BN forward-training / backward on 16-bit activations with fp32 parameters and statistics:
    the fp32 CPU oracle on the same (already rounded) inputs, outputs compared at the 16-bit
    tolerance of 1e-2 normalised L2; statistics and parameter gradients stay fp32 (1e-3)."""
    from oracle import cpu_oracle as O
    from util import nl2
    r = rng(sum(shape))
    N, C, H, W = shape
    xt, x = _to(singa, dev, (r.standard_normal(shape) * 2 + 0.5).astype(np.float32), kind)
    dyt, dy = _to(singa, dev, r.standard_normal(shape).astype(np.float32), kind)
    gamma = (1 + 0.1 * r.standard_normal(C)).astype(np.float32)
    beta = (0.1 * r.standard_normal(C)).astype(np.float32)
    h = singa.CudnnBatchNormHandle(0.9, xt)
    gd, bd = singa.from_numpy(gamma, dev), singa.from_numpy(beta, dev)
    rm, rv = singa.from_numpy(np.zeros(C, np.float32), dev), singa.from_numpy(np.ones(C, np.float32), dev)
    y, mean, var = singa.GpuBatchNormForwardTraining(h, xt, gd, bd, rm, rv)
    assert y.data_type() == xt.data_type() and mean.data_type() == singa.kFloat32
    y_o, mean_o, invstd_o = O.bn_fwd_train(x, gamma, beta, np.zeros(C, np.float32), np.ones(C, np.float32), 0.9, 1e-5)
    assert nl2(y.to_numpy(), y_o) < 1e-2
    np.testing.assert_allclose(mean.to_numpy(), mean_o, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(var.to_numpy(), invstd_o, rtol=1e-4)
    dx, ds, db = singa.GpuBatchNormBackward(h, dyt, xt, gd, mean, var)
    dx_o, ds_o, db_o = O.bn_bwd(dy, x, gamma, mean_o, invstd_o)
    assert dx.data_type() == xt.data_type()
    assert nl2(dx.to_numpy(), dx_o) < 1e-2
    assert nl2(ds.to_numpy(), ds_o) < 1e-3 and nl2(db.to_numpy(), db_o) < 1e-3


def _random_bn_shapes16(count, seed):
    """Seeded shapes for the 16-bit one-pass BatchNorm kernels: planes of whole 16-byte vectors (8 elements), of whole
    8-byte vectors only, and of neither (overlapping pieces); a thread's vectors stepping over several images or
    lying in one plane; one slice per channel and many."""
    r = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < count:
        C = int(r.choice([1, 3, 8, 24, 64, 130, 256, 300]))
        H = int(r.integers(1, 31))
        W = H if r.random() < 0.5 else int(r.integers(1, 31))
        N = int(r.integers(1, 65))
        if not 4000 <= N * C * H * W <= 4_000_000:
            continue
        shapes.append((N, C, H, W))
    return shapes


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("shape", _random_bn_shapes16(24, 20241126))
def test_batchnorm_16bit_shape_sweep(singa, dev, kind, shape):
    test_batchnorm_16bit_storage(singa, dev, kind, shape)


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(4, 3, 5, 6), (2, 5, 7, 7), (8, 64, 28, 28), (3, 7, 4, 2), (16, 24, 14, 14)])
def test_batchnorm_inference(singa, dev, kind, shape):
    """BatchNorm inference, y = gamma * (x - running_mean) / sqrt(running_var + 1e-5) + beta
    (cudnnBatchNormalizationForwardInference with CUDNN_BN_MIN_EPSILON, batchnorm.cc:352-360),
    against the formula in float64; and it reproduces the training-mode output when it is handed
    that batch's own statistics."""
    from util import nl2
    r = rng(sum(shape) + 9)
    N, C, H, W = shape
    x32 = (r.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    gamma = (1 + 0.1 * r.standard_normal(C)).astype(np.float32)
    beta = (0.1 * r.standard_normal(C)).astype(np.float32)
    rm = (0.3 * r.standard_normal(C)).astype(np.float32)
    rv = (0.5 + r.random(C)).astype(np.float32)
    if kind == "f32":
        xt, x = singa.from_numpy(x32, dev), x32
    else:
        xt, x = _to(singa, dev, x32, kind)
    gd, bd = singa.from_numpy(gamma, dev), singa.from_numpy(beta, dev)
    h = singa.CudnnBatchNormHandle(0.9, xt)
    y = singa.GpuBatchNormForwardInference(h, xt, gd, bd, singa.from_numpy(rm, dev), singa.from_numpy(rv, dev))
    assert y.data_type() == xt.data_type()
    c = (1, C, 1, 1)
    want = gamma.reshape(c).astype(np.float64) * (x.astype(np.float64) - rm.reshape(c)) / np.sqrt(
        rv.reshape(c).astype(np.float64) + 1e-5) + beta.reshape(c)
    assert nl2(y.to_numpy(), want) < (1e-6 if kind == "f32" else 1e-2)
    yt, mean, invstd = singa.GpuBatchNormForwardTraining(h, xt, gd, bd, None, None)
    var = 1.0 / invstd.to_numpy().astype(np.float64) ** 2 - 1e-5
    y2 = singa.GpuBatchNormForwardInference(h, xt, gd, bd, mean, singa.from_numpy(var.astype(np.float32), dev))
    assert nl2(y2.to_numpy(), yt.to_numpy()) < (1e-5 if kind == "f32" else 1e-2)


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(4, 3, 5, 6), (2, 5, 7, 7), (8, 64, 28, 28), (16, 32, 8, 8), (3, 7, 4, 2),
                                   (32, 64, 56, 56), (16, 24, 14, 14), (2, 8, 6, 6),
                                   # the one-pass backward (a channel fits in LDS, >= 128 channels)
                                   (8, 128, 14, 14), (16, 256, 7, 7), (4, 130, 5, 6), (32, 128, 8, 8), (128, 256, 14, 14),
                                   (128, 8, 7, 7), (96, 16, 5, 5)])
def test_fused_relu_batchnorm_backward(singa, dev, kind, shape):
    """The fused ReLU + BatchNorm backward equals ReLUBackward followed by GpuBatchNormBackward on
    the forward's own output BIT FOR BIT (the recomputed output selects the same elements as the
    stored one, zeros and 16-bit underflow included), in every storage type; and it matches the
    oracle's composition of the two ops."""
    from oracle import cpu_oracle as O
    from util import nl2
    r = rng(sum(shape) + 3)
    N, C, H, W = shape
    x32 = (r.standard_normal(shape) * 1.5 - 0.2).astype(np.float32)
    x32.ravel()[::17] = x32.ravel()[1]          # repeated values
    dy32 = r.standard_normal(shape).astype(np.float32)
    gamma = (1 + 0.3 * r.standard_normal(C)).astype(np.float32)
    beta = (0.2 * r.standard_normal(C)).astype(np.float32)
    gamma[0], beta[0] = 0.0, 0.0                # a channel whose output is exactly 0 everywhere: ReLU passes nothing
    if C > 1:
        gamma[1], beta[1] = 1e-6, 1e-8          # tiny outputs: underflow to zero in binary16
    if kind == "f32":
        xt, x, dyt, dy = singa.from_numpy(x32, dev), x32, singa.from_numpy(dy32, dev), dy32
    else:
        xt, x = _to(singa, dev, x32, kind)
        dyt, dy = _to(singa, dev, dy32, kind)
    gd, bd = singa.from_numpy(gamma, dev), singa.from_numpy(beta, dev)
    h = singa.CudnnBatchNormHandle(0.9, xt)
    y, mean, var = singa.GpuBatchNormForwardTraining(h, xt, gd, bd, None, None)
    two = singa.GpuBatchNormBackward(h, singa.ReLUBackward(dyt, y), xt, gd, mean, var)
    one = singa.GpuBatchNormReLUBackward(h, dyt, xt, gd, bd, mean, var)
    for a, b, what in zip(one, two, ("dx", "dscale", "dbias")):
        _same_bits(a.to_numpy(), b.to_numpy(), "fused vs separate " + what + " " + kind)
    y_o, mean_o, invstd_o = O.bn_fwd_train(x, gamma, beta, np.zeros(C, np.float32), np.ones(C, np.float32), 0.9, 1e-5)
    ynp = y.to_numpy()                          # the selection is made on the GPU's stored output
    dx_o, ds_o, db_o = O.bn_bwd(O.relu_bwd(dy, ynp), x, gamma, mean.to_numpy(), var.to_numpy())
    tol = 1e-3 if kind == "f32" else 1e-2
    assert nl2(one[0].to_numpy(), dx_o) < tol
    assert nl2(one[1].to_numpy(), ds_o) < 1e-3 and nl2(one[2].to_numpy(), db_o) < 1e-3


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(4, 3, 5, 6), (8, 64, 28, 28), (16, 24, 14, 14), (16, 256, 7, 7), (3, 7, 4, 2),
                                   (2, 5, 7, 7)])
def test_fused_forward_calls(singa, dev, kind, shape):
    """The forward fusions store the bits of the separate calls: GpuBatchNormReLUForwardTraining =
    ReLU(GpuBatchNormForwardTraining(...)) with the same saved and running statistics, AddReLU(a, b) =
    ReLU(a + b) (zeros, negative zeros of the sum and 16-bit underflow included); and a ReLU backward gated on
    the fused output equals the one gated on the ReLU's input."""
    r = rng(sum(shape) + 11)
    N, C, H, W = shape
    x32 = (r.standard_normal(shape) * 1.5 - 0.2).astype(np.float32)
    a32 = r.standard_normal(shape).astype(np.float32)
    a32.ravel()[::5] = -x32.ravel()[::5]        # sums that are exactly zero
    a32.ravel()[1::7] = 0.0
    dy32 = r.standard_normal(shape).astype(np.float32)
    gamma = (1 + 0.3 * r.standard_normal(C)).astype(np.float32)
    beta = (0.2 * r.standard_normal(C)).astype(np.float32)
    gamma[0], beta[0] = 0.0, 0.0                # outputs exactly 0
    if C > 1:
        gamma[1], beta[1] = 1e-6, 1e-8          # tiny outputs: underflow to zero in binary16
    if kind == "f32":
        xt, at, dyt = (singa.from_numpy(v, dev) for v in (x32, a32, dy32))
        relu = singa.ReLU
    else:
        xt, at, dyt = (_to(singa, dev, v, kind)[0] for v in (x32, a32, dy32))
        relu = lambda t: singa.ReLUBackward(t, t)   # the 16-bit tape's ReLU: t > 0 ? t : 0
    gd, bd = singa.from_numpy(gamma, dev), singa.from_numpy(beta, dev)
    stats = lambda: (singa.from_numpy(np.full(C, 0.25, np.float32), dev), singa.from_numpy(np.full(C, 2.0, np.float32), dev))
    h = singa.CudnnBatchNormHandle(0.9, xt)
    rm1, rv1 = stats()
    y, mean, var = singa.GpuBatchNormForwardTraining(h, xt, gd, bd, rm1, rv1)
    rm2, rv2 = stats()
    yr, mean2, var2 = singa.GpuBatchNormReLUForwardTraining(h, xt, gd, bd, rm2, rv2)
    _same_bits(yr.to_numpy(), relu(y).to_numpy(), "BatchNorm + ReLU forward " + kind)
    for got, want, what in ((mean2, mean, "mean"), (var2, var, "invstd"), (rm2, rm1, "running mean"), (rv2, rv1, "running var")):
        _same_bits(got.to_numpy(), want.to_numpy(), what + " " + kind)
    _same_bits(singa.ReLUBackward(dyt, yr).to_numpy(), singa.ReLUBackward(dyt, y).to_numpy(), "ReLU backward gated on the output " + kind)
    rm3, rv3 = stats()
    ysr, mean3, var3 = singa.GpuBatchNormAddReLUForwardTraining(h, xt, at, gd, bd, rm3, rv3)
    _same_bits(ysr.to_numpy(), relu(singa.__add__(y, at)).to_numpy(), "BatchNorm + Add + ReLU forward " + kind)
    for got, want, what in ((mean3, mean, "mean"), (var3, var, "invstd"), (rm3, rm1, "running mean"), (rv3, rv1, "running var")):
        _same_bits(got.to_numpy(), want.to_numpy(), what + " (with the sum) " + kind)
    s = singa.__add__(xt, at)
    sr = singa.AddReLU(xt, at)
    _same_bits(sr.to_numpy(), relu(s).to_numpy(), "Add + ReLU forward " + kind)
    _same_bits(singa.ReLUBackward(dyt, sr).to_numpy(), singa.ReLUBackward(dyt, s).to_numpy(), "ReLU backward gated on the sum's output " + kind)
    # unaligned operands take the scalar path
    n = xt.Size() - 1
    dt = {"f32": singa.kFloat32, "f16": singa.kFloat16, "bf16": singa.kBFloat16}[kind]
    views = [singa.from_device_pointer(t.ptr + (4 if kind == "f32" else 2), (n,), dev, dtype=dt, keepalive=t)
             for t in (xt, at)]
    _same_bits(singa.AddReLU(*views).to_numpy(), sr.to_numpy().ravel()[1:], "Add + ReLU, unaligned " + kind)


@pytest.mark.parametrize("kind,shape", [("f16", (64, 256, 56, 56)), ("f32", (32, 96, 28, 28))])
def test_recorded_batchnorm_forward_between_eager_backward_passes(singa, dev, kind, shape):
    """A recorded BatchNorm + Add + ReLU forward (graph mode) is replayed with eager backward passes on the same
    handle -- the same workspace -- in between: every replay stores the bits of the eager forward call.  (The
    one-pass forward kernel cuts a channel into other slices than the backward kernel; each keeps its exchange
    words in a part of the workspace that the other never writes.)"""
    r = rng(sum(shape) + 5)
    N, C, H, W = shape
    x32, z32, dy32 = (r.standard_normal(shape).astype(np.float32) for _ in range(3))
    if kind == "f32":
        xt, zt, dyt = (singa.from_numpy(v, dev) for v in (x32, z32, dy32))
    else:
        xt, zt, dyt = (_to(singa, dev, v, kind)[0] for v in (x32, z32, dy32))
    gd = singa.from_numpy((1 + 0.3 * r.standard_normal(C)).astype(np.float32), dev)
    bd = singa.from_numpy((0.2 * r.standard_normal(C)).astype(np.float32), dev)
    rm, rv = singa.from_numpy(np.zeros(C, np.float32), dev), singa.from_numpy(np.ones(C, np.float32), dev)
    h = singa.CudnnBatchNormHandle(0.9, xt)
    for _ in range(2):   # (the pool holds the blocks the recorded call will take)
        want, mean, var = singa.GpuBatchNormAddReLUForwardTraining(h, xt, zt, gd, bd, rm, rv)
        singa.GpuBatchNormBackward(h, dyt, xt, gd, mean, var)
    want_bits, want_mean = want.to_numpy(), mean.to_numpy()
    assert np.isfinite(want_bits.astype(np.float32)).all()
    del want
    dev.Sync()
    dev.EnableGraph(True)
    y, mean_g, var_g = singa.GpuBatchNormAddReLUForwardTraining(h, xt, zt, gd, bd, rm, rv)
    dev.EnableGraph(False)
    try:
        for i in range(5):
            y.SetFloatValue(0.0)
            dev.RunGraph()
            _same_bits(y.to_numpy(), want_bits, "replay %d of the recorded forward, %s" % (i, kind))
            _same_bits(mean_g.to_numpy(), want_mean, "saved mean of replay %d" % i)
            if i != 2:   # (also two replays in a row)
                dx, _, _ = singa.GpuBatchNormBackward(h, dyt, xt, gd, mean, var)
                assert np.isfinite(dx.to_numpy().astype(np.float32)).all()
    finally:
        dev.ResetGraph()


@pytest.mark.parametrize("kind,shape", [("f16", (128, 48, 7, 7)), ("bf16", (128, 96, 7, 7)), ("f32", (64, 24, 28, 28)),
                                        ("f16", (32, 16, 14, 14))])
def test_recorded_batchnorm_backward_between_eager_forward_passes(singa, dev, kind, shape):
    """The other direction: a recorded BatchNorm backward whose channels are cut into several slices (the one-pass
    kernel with exchange words) is replayed with eager FORWARD calls on the same handle in between.  On planes
    that are not whole vectors (7 x 7) the forward pass runs the two-pass kernels, which write their partial sums
    at the start of the workspace; the backward kernel's words lie in a part of their own behind them, so every
    replay finds all words of a channel in one state and stores the bits of the eager call."""
    r = rng(sum(shape) + 11)
    N, C, H, W = shape
    x32, dy32 = (r.standard_normal(shape).astype(np.float32) for _ in range(2))
    if kind == "f32":
        xt, dyt = (singa.from_numpy(v, dev) for v in (x32, dy32))
    else:
        xt, dyt = (_to(singa, dev, v, kind)[0] for v in (x32, dy32))
    gd = singa.from_numpy((1 + 0.3 * r.standard_normal(C)).astype(np.float32), dev)
    bd = singa.from_numpy((0.2 * r.standard_normal(C)).astype(np.float32), dev)
    rm, rv = singa.from_numpy(np.zeros(C, np.float32), dev), singa.from_numpy(np.ones(C, np.float32), dev)
    h = singa.CudnnBatchNormHandle(0.9, xt)
    for _ in range(2):   # (the pool holds the blocks the recorded call will take)
        y, mean, var = singa.GpuBatchNormForwardTraining(h, xt, gd, bd, rm, rv)
        want = [t.to_numpy() for t in singa.GpuBatchNormBackward(h, dyt, xt, gd, mean, var)]
    assert all(np.isfinite(np.asarray(w, np.float32)).all() for w in want)
    dev.Sync()
    dev.EnableGraph(True)
    dx, dg, db = singa.GpuBatchNormBackward(h, dyt, xt, gd, mean, var)
    dev.EnableGraph(False)
    try:
        for i in range(6):
            dx.SetFloatValue(0.0)
            dev.RunGraph()
            for got, w, what in zip((dx, dg, db), want, ("dx", "dgamma", "dbeta")):
                _same_bits(got.to_numpy(), w, "%s of replay %d of the recorded backward, %s" % (what, i, kind))
            if i != 3:   # (also two replays in a row)
                y2, _, _ = singa.GpuBatchNormForwardTraining(h, xt, gd, bd, rm, rv)
                _same_bits(y2.to_numpy(), y.to_numpy(), "eager forward between replays")
        dev.Sync()       # (no workgroup gave up: the wait reports nothing)
    finally:
        dev.ResetGraph()


def test_batchnorm_exchange_gives_up_visibly(singa, dev):
    """The one-pass kernels' bounded wait: with the spin limit forced down to one poll from the host, workgroups
    of a channel cut into many slices give up -- every kernel still ends normally, the channel's outputs are NaN,
    and the next wait on the device returns SGH_EEXCHANGE instead of 0 (once); sgh_bn_exchange_failures counts
    them.  With the default limit the same calls are clean and match the CPU oracle."""
    import ctypes as C
    from oracle import cpu_oracle as O
    from singa_amd import _lib
    from util import nl2
    L = _lib.lib()
    r = rng(77)
    N, Cn, H, W = 32, 8, 112, 112     # 8 channels on a whole chip: 64 slices per channel
    x = r.standard_normal((N, Cn, H, W)).astype(np.float32)
    dy = r.standard_normal((N, Cn, H, W)).astype(np.float32)
    g = (1 + 0.3 * r.standard_normal(Cn)).astype(np.float32)
    b = (0.2 * r.standard_normal(Cn)).astype(np.float32)
    xt, dyt, gd, bd = (singa.from_numpy(v, dev) for v in (x, dy, g, b))
    rm, rv = singa.from_numpy(np.zeros(Cn, np.float32), dev), singa.from_numpy(np.ones(Cn, np.float32), dev)
    h = singa.CudnnBatchNormHandle(0.9, xt)
    y, mean, var = singa.GpuBatchNormForwardTraining(h, xt, gd, bd, rm, rv)
    dev.Sync()
    L.sgh_bn_exchange_spin_limit(1)
    try:
        dx, dg, db = singa.GpuBatchNormBackward(h, dyt, xt, gd, mean, var)
        assert L.sgh_device_sync(dev._h) == _lib.SGH_EEXCHANGE          # the error code, not NaN-sniffing
        assert b"gave up" in L.sgh_error_string(_lib.SGH_EEXCHANGE)
        assert L.sgh_device_sync(dev._h) == 0                           # reported once
        assert np.isnan(dg.to_numpy()).any() and np.isnan(dx.to_numpy()).any()
        with pytest.raises(singa.SingaHipError, match="gave up"):
            singa.GpuBatchNormBackward(h, dyt, xt, gd, mean, var)
            dev.Sync()
        # the forward kernel likewise; counted by the explicit query
        singa.GpuBatchNormForwardTraining(h, xt, gd, bd, rm, rv)
        n = C.c_int(-1)
        _lib.check(L.sgh_bn_exchange_failures(dev.stream, C.byref(n)), "sgh_bn_exchange_failures")
        assert n.value > 0
        assert L.sgh_device_sync(dev._h) == 0                           # the query cleared the counter
    finally:
        L.sgh_bn_exchange_spin_limit(0)
    dx, dg, db = singa.GpuBatchNormBackward(h, dyt, xt, gd, mean, var)
    dev.Sync()
    n = C.c_int(-1)
    _lib.check(L.sgh_bn_exchange_failures(dev.stream, C.byref(n)), "sgh_bn_exchange_failures")
    assert n.value == 0
    dx_o, dg_o, db_o = O.bn_bwd(dy, x, g, mean.to_numpy(), var.to_numpy())
    assert nl2(dx.to_numpy(), dx_o) <= 1e-3 and nl2(dg.to_numpy(), dg_o) <= 1e-3 and nl2(db.to_numpy(), db_o) <= 1e-3


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("case", [
    (2, 3, 8, 8, (2, 2), (2, 2), (0, 0)),
    (2, 4, 17, 17, (3, 3), (2, 2), (1, 1)),
    (2, 16, 112, 112, (3, 3), (2, 2), (1, 1)),   # ResNet stem max-pool geometry (tiled kernel, 16-byte staging)
    (1, 2, 7, 5, (3, 2), (1, 2), (1, 0)),
    (3, 8, 14, 14, (3, 3), (1, 1), (1, 1)),
    (3, 40, 7, 7, (7, 7), (1, 1), (0, 0)),       # ResNet global pool geometry (whole-vector average backward)
    (1, 3, 5, 3, (5, 3), (1, 1), (0, 0)),        # ... planes of 15 elements: vectors across planes, scalar tail
])
def test_pooling_16bit_storage(singa, dev, kind, case):
    """Max pooling on 16-bit tensors routes the gradient like the CPU algorithm on the stored
    values (the 16-bit grid makes ties frequent: first maximum wins) and sums overlapping
    windows in fp32 with one rounding: bit-exact against the fp32 oracle on the same inputs,
    rounded once.  Average pooling: same rounding rule."""
    from oracle import cpu_oracle as O
    N, C, H, W, kernel, stride, pad = case
    r = rng(sum(case[:4]) + 3)
    xt, x = _to(singa, dev, np.round(r.standard_normal((N, C, H, W)) * 4).astype(np.float32) / 4, kind)  # many ties
    h = singa.CudnnPoolingHandle(xt, kernel, stride, pad, True)
    y = singa.GpuPoolingForward(h, xt)
    y_o, mask = O.pool_max_fwd(x, kernel, stride, pad)
    _same_bits(y.to_numpy(), y_o, "max-pool forward " + kind)       # a maximum of stored values is a stored value
    dyt, dy = _to(singa, dev, r.standard_normal(y_o.shape).astype(np.float32), kind)
    dx = singa.GpuPoolingBackward(h, dyt, xt, y)
    dx_o = O.pool_max_bwd(dy, mask, x.shape)
    _same_bits(dx.to_numpy(), _round(singa, dx_o, kind), "max-pool backward " + kind)
    ha = singa.CudnnPoolingHandle(xt, kernel, stride, pad, False)
    ya = singa.GpuPoolingForward(ha, xt)
    _same_bits(ya.to_numpy(), _round(singa, O.pool_avg_fwd(x, kernel, stride, pad, include_pad=False), kind),
               "avg-pool forward " + kind)
    dxa = singa.GpuPoolingBackward(ha, dyt, xt, ya)
    _same_bits(dxa.to_numpy(), _round(singa, O.pool_avg_bwd(dy, x.shape, kernel, stride, pad, include_pad=False), kind),
               "avg-pool backward " + kind)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("case", [
    (2, 64, 14, 14, 64, 3, 3, (1, 1), (1, 1), True),      # shared-tile kernels
    (2, 64, 14, 14, 128, 3, 3, (2, 2), (1, 1), False),    # stride-2 residue classes
    (2, 3, 32, 32, 64, 7, 7, (2, 2), (3, 3), False),      # stem kernels
    (3, 64, 8, 8, 128, 1, 1, (2, 2), (0, 0), False),      # pointwise
    (2, 5, 9, 7, 6, 3, 2, (2, 1), (1, 0), True),          # generic path
])
def test_conv_16bit_storage(singa, dev, kind, case):
    """Convolution passes on 16-bit tensors: operands widened to fp32, fp32 accumulation, one
    rounding of the result.  Checked against the fp32 CPU oracle on the same stored inputs at the
    16-bit tolerance (1e-2 normalised L2; the rounding of the result alone is about 3e-4 for
    binary16 and 2e-3 for bfloat16)."""
    from oracle import cpu_oracle as O
    from util import nl2
    N, C, H, W, K, R, S, stride, pad, bias = case
    r = rng(sum(case[:7]) + 11)
    xt, x = _to(singa, dev, r.standard_normal((N, C, H, W)).astype(np.float32), kind)
    wt, w = _to(singa, dev, (r.standard_normal((K, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32), kind)
    bt, b = _to(singa, dev, r.standard_normal(K).astype(np.float32), kind) if bias else (None, None)
    h = singa.CudnnConvHandle(xt, (R, S), stride, pad, C, K, bias)
    y = singa.GpuConvForward(xt, wt, bt, h)
    assert y.data_type() == xt.data_type()
    assert nl2(y.to_numpy(), O.conv_fwd(x, w, b, stride, pad)) < 1e-2
    dyt, dy = _to(singa, dev, r.standard_normal(y.shape()).astype(np.float32), kind)
    dx = singa.GpuConvBackwardx(dyt, wt, xt, h)
    dw = singa.GpuConvBackwardW(dyt, xt, wt, h)
    dx_o, dw_o = O.conv_bwd(dy, x, w, stride, pad)
    assert dx.data_type() == xt.data_type() and dw.data_type() == xt.data_type()
    assert nl2(dx.to_numpy(), dx_o) < 1e-2 and nl2(dw.to_numpy(), dw_o) < 1e-2
    if bias:
        db = singa.GpuConvBackwardb(dyt, bt, h)
        assert nl2(db.to_numpy(), O.conv_bgrad(dy)) < 1e-2


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("case", [
    # N, C, H = W, bias: the stem's forward kernel (7 x 7, stride 2, padding 3, 64 filters) at its four widths
    (3, 3, 32, True), (2, 1, 64, False), (2, 2, 128, True), (1, 3, 224, False),
])
def test_stem_forward_16bit(singa, dev, kind, case):
    """Forward convolution of the stem geometry on 16-bit tensors against the fp32 oracle on the same stored
    inputs (1e-2 normalised L2 as for every 16-bit convolution; the rounding of the result alone is about 3e-4
    for binary16 and 2e-3 for bfloat16, and the bound asserted here is 4e-3), borders included: every output
    row and column whose window reaches outside the image is compared on its own."""
    from oracle import cpu_oracle as O
    from util import nl2
    N, C, H, bias = case
    r = rng(H + 7 * C)
    xt, x = _to(singa, dev, r.standard_normal((N, C, H, H)).astype(np.float32), kind)
    wt, w = _to(singa, dev, (r.standard_normal((64, C, 7, 7)) * np.sqrt(2.0 / (C * 49))).astype(np.float32), kind)
    bt, b = _to(singa, dev, r.standard_normal(64).astype(np.float32), kind) if bias else (None, None)
    h = singa.CudnnConvHandle(xt, (7, 7), (2, 2), (3, 3), C, 64, bias)
    y = singa.GpuConvForward(xt, wt, bt, h).to_numpy()
    want = O.conv_fwd(x, w, b, (2, 2), (3, 3))
    assert y.shape == want.shape == (N, 64, H // 2, H // 2)
    assert nl2(y, want) < 4e-3
    for sl in (np.s_[:, :, :2, :], np.s_[:, :, -2:, :], np.s_[:, :, :, :2], np.s_[:, :, :, -2:]):
        assert nl2(y[sl], want[sl]) < 4e-3


def _grad16_cases(count, seed):
    """Seeded geometries for the 16-bit matrix-instruction gradient kernels: output rows of 1..3
    octets with partly empty last octets, odd and even widths (paired and single-pixel gradient
    loads), strides 1-2 with every residue class, channel counts around the 64 / 128 tile edges and
    K both below and above one 64-wide reduction chunk."""
    r = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        R = int(r.choice([1, 1, 3, 3, 3, 5, 7]))
        st = int(r.choice([1, 1, 2]))
        pd = int(r.integers(0, R // 2 + 1))
        C = int(r.choice([3, 16, 40, 64, 65, 128, 136]))
        K = int(r.choice([8, 24, 64, 72, 128, 136]))
        H = int(r.integers(max(R - 2 * pd, 2), 30))
        W = H if r.random() < 0.5 else int(r.integers(max(R - 2 * pd, 2), 36))
        N = int(r.integers(1, 5))
        P, Q = (H + 2 * pd - R) // st + 1, (W + 2 * pd - R) // st + 1
        if P < 1 or Q < 2 or N * K * P * Q * C * R * R > 3e8:
            continue
        cases.append((N, C, H, W, K, R, R, (st, st), (pd, pd)))
    return cases


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("case", _grad16_cases(40, 777) + [
    (2, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1)),      # ResNet stage-1 3x3
    (2, 256, 14, 14, 64, 1, 1, (1, 1), (0, 0)),     # bottleneck reduce: plane of 196 = 24.5 octets
    (3, 64, 7, 7, 256, 1, 1, (1, 1), (0, 0)),       # odd plane: single-pixel gradient loads
    (2, 128, 28, 28, 256, 1, 1, (2, 2), (0, 0)),    # downsample
    (1, 3, 64, 64, 64, 7, 7, (2, 2), (3, 3)),       # stem
    (2, 3, 224, 224, 64, 7, 7, (2, 2), (3, 3)),     # stem at full image size: seven column tiles per class row
    (2, 4, 40, 40, 96, 7, 7, (2, 2), (3, 3)),       # stem-like: four channels, three chunks of 32 gradient channels, a partial row band
    (2, 1, 24, 24, 32, 5, 5, (2, 2), (2, 2)),       # stem-like: one channel, 5x5 (three offsets per dimension)
    # 3x3 / stride 1 / padding 1 on the slab kernel (gradient slab shared by the nine taps):
    (3, 136, 12, 8, 136, 3, 3, (1, 1), (1, 1)),     # three chunks of gradient channels (the last partial), two channel tiles, 8-pixel groups
    (9, 256, 14, 14, 256, 3, 3, (1, 1), (1, 1)),    # planes of 196 pixels: 4-pixel groups, tiles that span images
    (5, 40, 30, 32, 72, 3, 3, (1, 1), (1, 1)),      # rows longer than a pixel group, two chunks, channel tile mostly empty
    (40, 128, 28, 28, 72, 3, 3, (1, 1), (1, 1)),    # many tiles of 256 positions across 40 images
    (2, 64, 10, 10, 64, 3, 3, (1, 1), (1, 1)),      # one chunk: the single-slab variant, groups of 4
    (1, 65, 16, 56, 64, 3, 3, (1, 1), (1, 1)),      # widest rows of the residual networks, 65 channels
])
def test_conv_gradients_16bit_matrix_kernels(singa, dev, kind, case):
    """dgrad / wgrad on the 16-bit MFMA kernels against the fp32 CPU oracle on the same stored
    inputs (1e-2 normalised L2), plus run-to-run identity of the split weight gradient."""
    from oracle import cpu_oracle as O
    from util import nl2
    N, C, H, W, K, R, S, stride, pad = case
    r = rng(sum(case[:7]) + 5)
    xt, x = _to(singa, dev, r.standard_normal((N, C, H, W)).astype(np.float32), kind)
    wt, w = _to(singa, dev, (r.standard_normal((K, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32), kind)
    h = singa.CudnnConvHandle(xt, (R, S), stride, pad, C, K, False)
    P, Q = (H + 2 * pad[0] - R) // stride[0] + 1, (W + 2 * pad[1] - S) // stride[1] + 1
    dyt, dy = _to(singa, dev, r.standard_normal((N, K, P, Q)).astype(np.float32), kind)
    dx = singa.GpuConvBackwardx(dyt, wt, xt, h)
    dw = singa.GpuConvBackwardW(dyt, xt, wt, h)
    dx_o, dw_o = O.conv_bwd(dy, x, w, stride, pad)
    e = nl2(dx.to_numpy(), dx_o), nl2(dw.to_numpy(), dw_o)
    print("16-bit gradients nl2: dx %.2e dw %.2e" % e)
    assert max(e) < 1e-2
    _same_bits(singa.GpuConvBackwardW(dyt, xt, wt, h).to_numpy(), dw.to_numpy(), "wgrad run-to-run")
    # the forward pass (stride 1: the data-gradient kernel on the channel-swapped, tap-reversed twin;
    # stride 2: fp32 kernels on widened copies), with and without bias
    bt, b = _to(singa, dev, r.standard_normal(K).astype(np.float32), kind)
    hb = singa.CudnnConvHandle(xt, (R, S), stride, pad, C, K, True)
    e = (nl2(singa.GpuConvForward(xt, wt, None, h).to_numpy(), O.conv_fwd(x, w, None, stride, pad)),
         nl2(singa.GpuConvForward(xt, wt, bt, hb).to_numpy(), O.conv_fwd(x, w, b, stride, pad)))
    print("16-bit forward nl2: %.2e, with bias %.2e" % e)
    assert max(e) < 1e-2
    # dx_old += dgrad on 16-bit tensors: the data gradient and a separate 16-bit add (two roundings)
    oldt, old = _to(singa, dev, r.standard_normal((N, C, H, W)).astype(np.float32), kind)
    got = singa.GpuConvBackwardxAccumulate(dyt, wt, xt, h, oldt)
    assert got is oldt
    _same_bits(got.to_numpy(), _round(singa, old + dx.to_numpy(), kind), "dx += dgrad")


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_conv_dgrad_16bit_with_batched_weight_relayout(singa, dev, kind):
    """GpuConvPrepareBackward on the seeded 16-bit geometries: one launch re-lays the weights of all
    layers that the 16-bit matrix kernel covers, the data gradients that follow give the same bits."""
    layers = []
    for i, case in enumerate(_grad16_cases(24, 9090) + [(2, 3, 32, 32, 64, 7, 7, (2, 2), (3, 3)),
                                                        (4, 512, 7, 7, 512, 3, 3, (1, 1), (1, 1))]):
        N, C, H, W, K, R, S, stride, pad = case
        r = rng(700 + i)
        P, Q = (H + 2 * pad[0] - R) // stride[0] + 1, (W + 2 * pad[1] - S) // stride[1] + 1
        xt, _ = _to(singa, dev, r.standard_normal((N, C, H, W)).astype(np.float32), kind)
        wt, _ = _to(singa, dev, r.standard_normal((K, C, R, S)).astype(np.float32), kind)
        dyt, _ = _to(singa, dev, r.standard_normal((N, K, P, Q)).astype(np.float32), kind)
        h = singa.CudnnConvHandle(xt, (R, S), stride, pad, C, K, False)
        layers.append((case, xt, wt, dyt, h, singa.GpuConvBackwardx(dyt, wt, xt, h).to_numpy()))
    singa.GpuConvPrepareBackward([(l[2], l[4]) for l in layers])
    prelaid = [bool(l[4].geom.prelaid_W) for l in layers]
    assert False in prelaid and prelaid.count(True) >= len(layers) // 2, prelaid
    for case, xt, wt, dyt, h, want in layers:
        _same_bits(singa.GpuConvBackwardx(dyt, wt, xt, h).to_numpy(), want, "prepared dgrad %r" % (case,))
    assert not any(l[4].geom.prelaid_W for l in layers)     # each note was used once
    # prepared, then the weights change (an update of the 16-bit tensor): the current weights are used
    case, xt, wt, dyt, h, want = layers[prelaid.index(True)]
    singa.GpuConvPrepareBackward([(wt, h)])
    singa.Axpy(0.5, wt, wt)
    fresh_h = singa.CudnnConvHandle(xt, (case[5], case[6]), case[7], case[8], case[1], case[4], False)
    _same_bits(singa.GpuConvBackwardx(dyt, wt, xt, h).to_numpy(), singa.GpuConvBackwardx(dyt, wt, xt, fresh_h).to_numpy(),
               "prepared dgrad after the weights changed")


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [
    (128, 64, 56, 64, 3, 1, 1),      # ResNet-50 stage 1, 3x3
    (128, 256, 56, 64, 1, 1, 0),     # bottleneck reduce
    (128, 128, 56, 128, 3, 2, 1),    # stage transition, stride 2
    (128, 1024, 14, 256, 1, 1, 0),   # plane of 196 pixels: 24.5 octets
    (128, 512, 7, 2048, 1, 1, 0),    # stage 4: bottleneck expand on 7 x 7 planes
    (128, 2048, 7, 512, 1, 1, 0),    # ... reduce
    (128, 512, 7, 512, 3, 1, 1),     # ... 3x3 on 49-pixel planes (pixel-major gradient copy)
    (128, 512, 14, 512, 3, 2, 1),    # ... its stride-2 opening layer
    (128, 256, 56, 512, 1, 2, 0),    # downsample convolutions: 1x1 stride 2 (one residue class, 2x2-block store)
    (128, 1024, 14, 2048, 1, 2, 0),
])
def test_conv_gradients_16bit_full_size_properties(singa, dev, kind, shape):
    """The 16-bit gradient kernels at the half-precision configuration's full batch (N = 128), too
    large for the CPU oracle inside a test: adjointness <x, dgrad(dy)> = <W, wgrad(dy)> (both equal
    <conv(x, W), dy>) on the stored values, the oracle on one image of the batch for dgrad, on a
    2-image sub-batch for wgrad (additive over images), and exact linearity under scaling by 2
    (wherever the result is a normal number of the storage type)."""
    from oracle import cpu_oracle as O
    from util import nl2
    N, C, H, K, R, st, pd = shape
    r = rng(sum(shape))
    xt, x = _to(singa, dev, r.standard_normal((N, C, H, H)).astype(np.float32), kind)
    wt, w = _to(singa, dev, (r.standard_normal((K, C, R, R)) * np.sqrt(2.0 / (C * R * R))).astype(np.float32), kind)
    h = singa.CudnnConvHandle(xt, (R, R), (st, st), (pd, pd), C, K, False)
    P = h.conv_height
    dy32 = r.standard_normal((N, K, P, P)).astype(np.float32)
    dyt, dy = _to(singa, dev, dy32, kind)
    dx = singa.GpuConvBackwardx(dyt, wt, xt, h).to_numpy()
    dw = singa.GpuConvBackwardW(dyt, xt, wt, h).to_numpy()
    a = float((x.astype(np.float64) * dx).sum()), float((w.astype(np.float64) * dw).sum())
    scale = float(np.sqrt((x.astype(np.float64) ** 2).sum() * (dx.astype(np.float64) ** 2).sum()))
    assert abs(a[0] - a[1]) < 1e-3 * scale      # both sides carry one 16-bit rounding per element
    dx5, _ = O.conv_bwd(dy[5:6], x[5:6], w, (st, st), (pd, pd), want_dw=False)
    assert nl2(dx[5:6], dx5) < 1e-2
    dys = dy.copy()
    dys[2:] = 0
    dw2 = singa.GpuConvBackwardW(_to(singa, dev, dys, kind)[0], xt, wt, h).to_numpy()
    _, dw2_o = O.conv_bwd(dy[:2], x[:2], w, (st, st), (pd, pd), want_dx=False)
    assert nl2(dw2, dw2_o) < 1e-2
    dx2 = singa.GpuConvBackwardx(_to(singa, dev, dy * 2, kind)[0], wt, xt, h).to_numpy()
    normal = np.abs(dx) >= 2.0 ** -13        # (binary16 subnormals have a coarser grid: 2x is not exact there)
    _same_bits(dx2[normal], dx[normal] * 2, "dgrad linearity " + kind)
    # the forward pass at the same size: <conv(x, W), dy> closes the adjointness triangle, and the
    # oracle on one image of the batch
    y = singa.GpuConvForward(xt, wt, None, h).to_numpy()
    a_y = float((y.astype(np.float64) * dy).sum())
    scale_y = float(np.sqrt((y.astype(np.float64) ** 2).sum() * (dy.astype(np.float64) ** 2).sum()))
    assert abs(a_y - a[0]) < 1e-3 * max(scale, scale_y)
    assert nl2(y[5:6], O.conv_fwd(x[5:6], w, None, (st, st), (pd, pd))) < 1e-2


def _sgd_ref(p, g, v, lr, mu, damp, wd, nesterov):
    """The four ops of SGD.apply in fp32, each product / sum rounded separately."""
    f = np.float32
    p, g, v = p.astype(f), g.astype(f), v.astype(f)
    if wd != 0:
        g = g + f(wd) * p
    if mu != 0:
        v = v * f(mu) + (f(1.0) - f(damp)) * g
        g = g + f(mu) * v if nesterov else v
    p = p + (f(0.0) - f(lr)) * g
    return p, v


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("hyper", [(0.05, 0.9, 0.0, 0.0, False), (0.1, 0.9, 0.0, 1e-4, True), (0.01, 0.0, 0.0, 5e-4, False),
                                   (0.05, 0.5, 0.1, 0.0, False)])
def test_sgd_on_16bit_gradients(singa, dev, kind, hyper):
    from singa_amd import opt
    lr, mu, damp, wd, nesterov = hyper
    r = rng(int(lr * 1000) + int(mu * 10))
    n = 70001
    # (a) everything 16-bit: two steps, p and v rounded once per step
    pt, p = _to(singa, dev, r.standard_normal(n).astype(np.float32), kind)
    sgd = opt.SGD(lr=lr, momentum=mu, dampening=damp, weight_decay=wd, nesterov=nesterov)
    v = np.zeros(n, np.float32)
    for _ in range(2):
        gt, g = _to(singa, dev, r.standard_normal(n).astype(np.float32), kind)
        sgd.apply("w", pt, gt)
        p, v = _sgd_ref(p, g, v, lr, mu, damp, wd, nesterov)
        p, v = _round(singa, p, kind), _round(singa, v, kind)
        _same_bits(pt.to_numpy(), p, "16-bit SGD p " + kind)
        if mu != 0:
            _same_bits(sgd.moments["w"].to_numpy(), v, "16-bit SGD v " + kind)
    # (b) fp32 master weights and momentum, 16-bit working copy
    pt, p = _to(singa, dev, r.standard_normal(n).astype(np.float32), kind)
    sgd = opt.SGD(lr=lr, momentum=mu, dampening=damp, weight_decay=wd, nesterov=nesterov)
    v = np.zeros(n, np.float32)
    for _ in range(3):
        gt, g = _to(singa, dev, r.standard_normal(n).astype(np.float32), kind)
        sgd.apply_master("w", pt, gt)
        p, v = _sgd_ref(p, g, v, lr, mu, damp, wd, nesterov)     # the master stays fp32 between steps
        _same_bits(sgd.masters["w"].to_numpy(), p, "master p " + kind)
        _same_bits(pt.to_numpy(), _round(singa, p, kind), "working copy " + kind)
        if mu != 0:
            _same_bits(sgd.moments["w"].to_numpy(), v, "master v " + kind)


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_set_value_on_16bit_tensors_stays_inside_the_tensor(singa, dev, kind):
    """Tensor::SetValue on a 16-bit tensor writes 2-byte elements: the neighbours of the filled
    range keep their contents (a float fill of the same element count would run over them), at
    every alignment of the range and for odd lengths; the value is rounded once to the storage type."""
    dt = singa.kFloat16 if kind == "f16" else singa.kBFloat16
    values = [0.1, -3.0, 65520.0, 1e-7, 2.0 ** -25 * 1.5, 1.00390625]
    for off, n, v in [(0, 1000, 0.1), (1, 1001, -3.0), (2, 7, 65520.0), (3, 1, 1e-7), (5, 64 * 1024 + 3, values[4]),
                      (8, 0, 1.0), (7, 2, values[5])]:
        total = off + n + 9
        sentinel = np.full(total, 0x7B7B, np.uint16)
        big = singa.Tensor((total,), dev, dt)
        big.CopyHalfDataFromHostPtr(sentinel.view(np.float16) if kind == "f16" else sentinel)   # (raw payloads)
        view = singa.from_device_pointer(big.ptr + 2 * off, (n,), dev, dt, keepalive=big)
        view.SetFloatValue(v)
        got = np.empty(total, np.uint16)
        from singa_amd._lib import check, lib
        check(lib().sgh_memcpy(dev._h, got.ctypes.data, big.ptr, got.nbytes, 2))
        want = sentinel.copy()
        if kind == "f16":
            with np.errstate(over="ignore"):
                want[off:off + n] = np.float32(v).astype(np.float16).view(np.uint16)
        else:
            want[off:off + n] = singa.float_to_bf16_bits(np.array([v], np.float32))[0]
        assert np.array_equal(got, want), (kind, off, n, v)


def test_fp32_only_functions_refuse_16bit_tensors(singa, dev):
    t = singa.Tensor((4, 8), dev, singa.kFloat16)
    t.SetFloatValue(1.0)
    for call in (lambda: singa.SoftMax(t), lambda: singa.Sum(t, 0), lambda: t.__imul__(2.0)):
        with pytest.raises(singa.SingaHipError):
            call()
