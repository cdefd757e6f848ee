"""GPU parity: tensor_math backward ops and the SGD update against the CPU oracle, through the
C ABI (singa_amd.singa_wrap -> ctypes -> libsinga_hip.so).

Tolerances: elementwise ops are compared bit for bit where the arithmetic is a single rounding
per op (ReLU, Add, Mult, softmax-CE backward, Axpy and SGD with contraction off); where a
library routine may legitimately round differently the bound is max relative error 1e-5."""
import numpy as np
import pytest

from oracle import cpu_oracle as O
from util import assert_bit_equal, max_rel_err, nl2, randn, rng

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 3, 4, 5, 255, 256, 1027, 4096, 100003, 1 << 20]


@pytest.fixture(scope="module")
def singa():
    from singa_amd import singa_wrap
    return singa_wrap


def test_relu_reference_vector(singa, dev, golden):
    g = golden["relu"]
    x = singa.from_numpy(np.array(g["x"], np.float32).reshape(g["x_shape"]), dev)
    dy = singa.from_numpy(np.array(g["dy"], np.float32).reshape(g["x_shape"]), dev)
    assert singa.ReLU(x).to_numpy().ravel().tolist() == [np.float32(v) for v in g["y"]]
    assert singa.ReLUBackward(dy, x).to_numpy().ravel().tolist() == g["dx"]


def test_relu_layer_reference_vector(singa, dev, golden):
    """The legacy Activation layer's ReLU vectors (test/singa/test_activation.cc:44-129)."""
    g = golden["relu_layer"]
    x, dy = singa.from_numpy(np.array(g["x"], np.float32), dev), singa.from_numpy(np.array(g["dy"], np.float32), dev)
    assert singa.ReLU(x).to_numpy().tolist() == g["y"]
    assert singa.ReLUBackward(dy, x).to_numpy().tolist() == g["dx"]


def test_dense_backward_reference_vector(singa, dev, golden):
    """Dense.Backward (test/singa/test_dense.cc:75-137) as autograd runs a Linear layer: db = Sum(dy, 0), the value the
    reference test asserts; dx = dy . W^T and dW = x^T . dy (python/singa/autograd.py:613-623) against the oracle."""
    g = golden["dense"]
    x = np.array(g["x"], np.float32).reshape(g["x_shape"])
    w = np.array(g["w"], np.float32).reshape(g["w_shape"])
    dy = np.array(g["dy"], np.float32).reshape(g["dy_shape"])
    xd, wd, dyd = (singa.from_numpy(v, dev) for v in (x, w, dy))
    db = singa.Sum(dyd, 0).to_numpy()
    for i, terms in enumerate(g["db_terms"]):
        np.testing.assert_allclose(db[i], sum(float(dy.ravel()[k]) for k in terms), rtol=5e-7)
    assert_bit_equal(singa.Mult(dyd, wd.T()).to_numpy(), O.sgemm(dy, w, transB=True), "dx = dy . W^T")
    assert_bit_equal(singa.Mult(xd.T(), dyd).to_numpy(), O.sgemm(x, dy, transA=True), "dW = x^T . dy")


@pytest.mark.parametrize("n", SIZES)
def test_relu_backward(singa, dev, n):
    r = rng(n + 1)
    x, dy = randn(r, n), randn(r, n)
    if n > 8:
        x[::7] = 0.0      # gradient at exactly zero is zero
        x[3::11] = -0.0
    dx = singa.ReLUBackward(singa.from_numpy(dy, dev), singa.from_numpy(x, dev)).to_numpy()
    assert_bit_equal(dx, O.relu_bwd(dy, x), "relu_bwd n=%d" % n)


@pytest.mark.parametrize("n", [1, 5, 1024, 4099, 1 << 20])
def test_relu_backward_of_two_summands(singa, dev, n):
    """ReLUBackwardSum(dy0, dy1, x) = ReLUBackward(dy0 + dy1, x) bit for bit (oracle: the fp32 sum,
    then the select), also through the scalar path of unaligned pointers."""
    r = rng(n + 77)
    x, d0, d1 = randn(r, n), randn(r, n), randn(r, n)
    x[::5] = 0.0
    want = O.relu_bwd(d0 + d1, x)
    t = [singa.from_numpy(a, dev) for a in (d0, d1, x)]
    assert_bit_equal(singa.ReLUBackwardSum(*t).to_numpy(), want, "relu_bwd_add n=%d" % n)
    if n > 1:
        views = [singa.from_device_pointer(a.ptr + 4, (n - 1,), dev, keepalive=a) for a in t]
        assert_bit_equal(singa.ReLUBackwardSum(*views).to_numpy(), want[1:], "relu_bwd_add unaligned")


def test_relu_backward_stage1_shape_and_unaligned(singa, dev):
    r = rng(99)
    shape = (8, 64, 56, 56)
    x, dy = randn(r, *shape), randn(r, *shape)
    dx = singa.ReLUBackward(singa.from_numpy(dy, dev), singa.from_numpy(x, dev)).to_numpy()
    assert_bit_equal(dx, O.relu_bwd(dy, x), "relu_bwd 4-D")
    # pointers that are not 16-byte aligned take the scalar path
    big = singa.from_numpy(np.concatenate([[0], x.ravel()[:1001]]).astype(np.float32), dev)
    bigdy = singa.from_numpy(np.concatenate([[0], dy.ravel()[:1001]]).astype(np.float32), dev)
    xs = singa.from_device_pointer(big.ptr + 4, (1001,), dev, keepalive=big)
    dys = singa.from_device_pointer(bigdy.ptr + 4, (1001,), dev, keepalive=bigdy)
    assert_bit_equal(singa.ReLUBackward(dys, xs).to_numpy(), O.relu_bwd(dy.ravel()[:1001], x.ravel()[:1001]), "unaligned")


def test_softmax_ce_reference_vector(singa, dev, golden):
    g = golden["softmax_ce"]
    p = singa.SoftMax(singa.from_numpy(np.array(g["p"], np.float32).reshape(g["p_shape"]), dev))
    for t in (np.array(g["t_index"], np.int32), np.array(g["t_onehot"], np.int32).reshape(2, 4)):
        tt = singa.from_numpy(t, dev)
        np.testing.assert_allclose(singa.CrossEntropyFwd(p, tt).to_numpy(), np.float32(-np.log(0.25)), rtol=4e-7)
        np.testing.assert_allclose(singa.SoftmaxCrossEntropyBwd(p, tt).to_numpy().ravel(),
                                   np.array(g["grad"], np.float32), rtol=4e-7)


@pytest.mark.parametrize("batch,dim", [(1, 1), (2, 4), (128, 10), (64, 1000), (7, 1025), (3, 70001)])
def test_softmax_ce_backward_bit_exact(singa, dev, batch, dim):
    r = rng(batch * 131 + dim)
    p = O.softmax(randn(r, batch, dim) * 3)
    t = r.integers(0, dim, size=batch).astype(np.int32)
    pd = singa.from_numpy(p, dev)
    g = singa.SoftmaxCrossEntropyBwd(pd, singa.from_numpy(t, dev)).to_numpy()
    assert_bit_equal(g, O.softmax_ce_bwd(p, t), "index target")
    assert_bit_equal(pd.to_numpy(), p, "p must not be modified")
    # fused /N (multiply by the fp32 reciprocal like the reference's Div)
    scale = float(np.float32(1.0) / np.float32(batch))
    g = singa.SoftmaxCrossEntropyBwd(pd, singa.from_numpy(t, dev), scale=scale).to_numpy()
    assert_bit_equal(g, O.softmax_ce_bwd(p, t, div_by=batch), "index target, /N")
    if 1 < dim <= 1025:  # with dim == 1 a [batch, dim] target is indistinguishable from an index target
        multi = np.eye(dim, dtype=np.int32)[t]
        multi[:, 0] += 2
        g = singa.SoftmaxCrossEntropyBwd(pd, singa.from_numpy(multi, dev)).to_numpy()
        assert_bit_equal(g, O.softmax_ce_bwd(p, multi), "array target")


def test_softmax_ce_label_edges(singa, dev):
    p = O.softmax(randn(rng(5), 4, 6))
    t = np.array([0, 5, 5, 0], np.int32)  # first and last class
    g = singa.SoftmaxCrossEntropyBwd(singa.from_numpy(p, dev), singa.from_numpy(t, dev)).to_numpy()
    assert_bit_equal(g, O.softmax_ce_bwd(p, t))
    assert singa.LabelErrors(dev) == 0
    bad = np.array([0, 6, -1, 1], np.int32)  # out of range: row left as p, error counted
    g = singa.SoftmaxCrossEntropyBwd(singa.from_numpy(p, dev), singa.from_numpy(bad, dev)).to_numpy()
    assert_bit_equal(g[1:3], p[1:3])
    assert singa.LabelErrors(dev) == 2
    assert singa.LabelErrors(dev) == 0


def test_softmax_and_ce_forward(singa, dev):
    r = rng(6)
    x = randn(r, 64, 1000) * 5
    p = singa.SoftMax(singa.from_numpy(x, dev))
    assert max_rel_err(p.to_numpy(), O.softmax(x), floor=1e-12) < 1e-5
    t = r.integers(0, 1000, size=64).astype(np.int32)
    loss = singa.CrossEntropyFwd(p, singa.from_numpy(t, dev)).to_numpy()
    assert max_rel_err(loss, O.cross_entropy_fwd(p.to_numpy(), t)) < 1e-5


@pytest.mark.parametrize("n", SIZES)
def test_axpy_mult_add(singa, dev, n):
    r = rng(n + 17)
    x, y = randn(r, n), randn(r, n)
    yd = singa.from_numpy(y, dev)
    singa.Axpy(0.37, singa.from_numpy(x, dev), yd)
    exp = y.copy()
    O.axpy(0.37, x, exp)
    assert_bit_equal(yd.to_numpy(), exp, "Axpy scalar")
    # Tensor alpha (1-element device tensor, as opt.SGD passes it)
    alpha = singa.from_numpy(np.array([-0.05], np.float32), dev)
    singa.Axpy(alpha, singa.from_numpy(x, dev), yd)
    O.axpy(-0.05, x, exp)
    assert_bit_equal(yd.to_numpy(), exp, "Axpy tensor alpha")
    assert_bit_equal(singa.EltwiseMult(singa.from_numpy(x, dev), singa.from_numpy(y, dev)).to_numpy(),
                     O.eltwise_mult(x, y), "EltwiseMult")
    if n > 1:
        buf = singa.from_numpy(x, dev)
        buf *= singa.from_numpy(np.array([0.9], np.float32), dev)  # stride-0 broadcast of opt.py:299-300
        assert_bit_equal(buf.to_numpy(), O.eltwise_mult(x, np.array([0.9], np.float32)), "buf *= mom")
    acc = singa.from_numpy(x, dev)
    acc += singa.from_numpy(y, dev)
    assert_bit_equal(acc.to_numpy(), O.add(x, y), "+=")


@pytest.mark.parametrize("op_by_op", [False, True])
def test_sgd_reference_cases(singa, dev, golden, op_by_op):
    """op_by_op: the reference's own sequence of tensor ops (Axpy with device scalars, the in-place product with the
    momentum tensor) instead of the fused kernel -- what unchanged python/singa/opt.py runs on this library."""
    from singa_amd import opt
    g = golden["sgd"]
    shape = tuple(g["shape"])
    for c in g["cases"]:
        sgd = opt.SGD(lr=c["lr"], momentum=c["mu"], weight_decay=c["wd"], nesterov=bool(c["nesterov"]), op_by_op=op_by_op)
        w = singa.from_numpy(np.full(shape, c["w0"], np.float32), dev)
        wo, vo = np.full(shape, c["w0"], np.float32), np.zeros(shape, np.float32)
        for _ in range(c["steps"]):
            grad = np.full(shape, c["g"], np.float32)
            sgd.apply("w", w, singa.from_numpy(grad, dev))
            sgd.step()
            O.sgd_momentum(wo, grad, vo, c["lr"], mu=c["mu"], wd=c["wd"], nesterov=bool(c["nesterov"]))
            assert_bit_equal(w.to_numpy(), wo, c["name"])


@pytest.mark.parametrize("n", [1, 5, 4096, 100003, 2359296])
@pytest.mark.parametrize("cfg", [(0.05, 0.9, 0.0, 0.0, False), (0.1, 0.9, 0.1, 1e-4, False), (0.01, 0.8, 0.0, 5e-4, True),
                                 (0.05, 0.0, 0.0, 0.0, False)])
@pytest.mark.parametrize("op_by_op", [False, True])
def test_sgd_momentum_fused(singa, dev, n, cfg, op_by_op):
    lr, mu, damp, wd, nesterov = cfg
    from singa_amd import opt
    r = rng(n)
    p, v = randn(r, n), randn(r, n)
    sgd = opt.SGD(lr=lr, momentum=mu, dampening=damp, weight_decay=wd, nesterov=nesterov, op_by_op=op_by_op)
    pd = singa.from_numpy(p, dev)
    if mu != 0:
        sgd.moments["p"] = singa.from_numpy(v, dev)
    for step in range(2):
        g = randn(r, n)
        sgd.apply("p", pd, singa.from_numpy(g, dev))
        O.sgd_momentum(p, g, v, lr, mu=mu, damp=damp, wd=wd, nesterov=nesterov)
    assert_bit_equal(pd.to_numpy(), p, "p")
    if mu != 0:
        assert_bit_equal(sgd.moments["p"].to_numpy(), v, "v")


def test_sgd_multi_tensor_matches_per_tensor(singa, dev):
    from singa_amd import opt
    r = rng(77)
    sizes = [1, 7, 64, 1000, 2048, 4099, 36864, 147456, 10]
    ps = [randn(r, n) for n in sizes]
    gs = [randn(r, n) for n in sizes]
    a = opt.SGD(lr=0.05, momentum=0.9)
    b = opt.SGD(lr=0.05, momentum=0.9)
    pa = [singa.from_numpy(p, dev) for p in ps]
    pb = [singa.from_numpy(p, dev) for p in ps]
    for step in range(2):
        for i, n in enumerate(sizes):
            a.apply("p%d" % i, pa[i], singa.from_numpy(gs[i], dev))
        b.apply_all([("p%d" % i, pb[i], singa.from_numpy(gs[i], dev)) for i in range(len(sizes))])
    for i in range(len(sizes)):
        assert_bit_equal(pa[i].to_numpy(), pb[i].to_numpy(), "multi p%d" % i)
        assert_bit_equal(a.moments["p%d" % i].to_numpy(), b.moments["p%d" % i].to_numpy(), "multi v%d" % i)


@pytest.mark.parametrize("M,N,K", [(128, 784, 1000), (128, 1000, 10), (64, 512, 1000), (1, 1, 1), (65, 129, 33),
                                   (300, 260, 515), (70, 90, 516), (128, 2048, 1000), (33, 31, 256)])
def test_linear_backward_gemms(singa, dev, M, N, K):
    """Matmul.backward: dx = dy * W^T, dW = x^T * dy (python/singa/autograd.py:613-623)."""
    r = rng(M + N + K)
    x, W, dy = randn(r, M, N), randn(r, N, K), randn(r, M, K)
    xd, Wd, dyd = (singa.from_numpy(a, dev) for a in (x, W, dy))
    dx = singa.Mult(dyd, singa.DefaultTranspose(Wd)).to_numpy()
    dW = singa.Mult(singa.DefaultTranspose(xd), dyd).to_numpy()
    y = singa.Mult(xd, Wd).to_numpy()
    assert nl2(dx, O.sgemm(dy, W, transB=True)) < 1e-5
    assert nl2(dW, O.sgemm(x, dy, transA=True)) < 1e-5
    assert nl2(y, O.sgemm(x, W)) < 1e-5
    tt = singa.Mult(singa.DefaultTranspose(xd), singa.DefaultTranspose(singa.from_numpy(randn(r, K, M), dev)))
    assert tt.shape() == [N, K]
    db = singa.Sum(dyd, 0).to_numpy()
    assert max_rel_err(db, O.sum_rows(dy), floor=1e-3) < 1e-5
    in_row_order = np.zeros(K, np.float32)
    for row in dy:          # the kernel adds the rows in ascending order, one fp32 addition each
        in_row_order += row
    assert_bit_equal(db, in_row_order, "column sums in row order")


@pytest.mark.parametrize("M,N,K", [(128, 512, 1000), (70, 90, 516), (5, 40, 300), (128, 96, 64)])
def test_gemm_alpha_beta_with_contiguous_reductions(singa, dev, M, N, K):
    """sgh_gemm_f32 as C = alpha * A * B^T + beta * C (cublasSgemm's contract, src/core/tensor/tensor_math_cuda.h:
    GEMM): few output tiles with a long reduction run on the kernel that splits the reduction over a workgroup's
    wavefronts; checked against float64, with beta = 0 not reading C (NaN in it), and run twice for identical bits."""
    from singa_amd._lib import check, lib
    r = rng(M * 3 + N * 5 + K)
    a, b, c = randn(r, M, K), randn(r, N, K), randn(r, M, N)
    ad, bd = singa.from_numpy(a, dev), singa.from_numpy(b, dev)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    outs = []
    for alpha, beta in ((1.0, 0.0), (0.5, -2.0), (1.0, 0.0)):
        c0 = np.full((M, N), np.nan, np.float32) if beta == 0.0 else c
        cd = singa.from_numpy(c0, dev)
        check(lib().sgh_gemm_f32(0, 1, M, N, K, alpha, ad.ptr, K, bd.ptr, K, beta, cd.ptr, N, dev.stream), "sgh_gemm_f32")
        got = cd.to_numpy()
        ref = alpha * want + (beta * c.astype(np.float64) if beta != 0.0 else 0.0)
        assert nl2(got, ref.astype(np.float32)) < 1e-5, (alpha, beta)
        outs.append(got)
    assert_bit_equal(outs[0], outs[2], "two runs")


def test_pool_reuses_freed_blocks(singa, dev):
    before = dev.PoolStats()["driver_allocs"]
    for _ in range(20):
        t = singa.Tensor((1 << 16,), dev)
        t.SetFloatValue(1.0)
        del t
    assert dev.PoolStats()["driver_allocs"] - before <= 1


def test_profiling_records_and_their_release(singa, dev):
    """sgh_prof_enable / count / get / clear: a bracketed launch leaves a record with its tag, a positive
    duration and its work; records outlive sgh_prof_enable(0) until sgh_prof_clear drops them; clearing
    while records are still being taken is refused."""
    import ctypes as C
    from singa_amd import _lib
    lib = _lib.lib()
    m = 5000
    x = singa.Tensor((m,), dev); x.SetFloatValue(1.0)
    dy = singa.Tensor((m,), dev); dy.SetFloatValue(2.0)
    n = C.c_int(-1)
    assert lib.sgh_prof_enable(1) == 0
    assert lib.sgh_prof_count(C.byref(n)) == 0 and n.value == 0
    dx = singa.ReLUBackward(dy, x)
    dev.Sync()
    assert lib.sgh_prof_clear() == -1                       # still enabled
    assert lib.sgh_prof_count(C.byref(n)) == 0 and n.value >= 1
    taken = n.value
    buf = C.create_string_buffer(64)
    ms, work = C.c_float(), C.c_double()
    assert lib.sgh_prof_get(0, buf, 64, C.byref(ms), C.byref(work)) == 0
    assert buf.value.decode().startswith("relu_bwd/") and ms.value > 0
    assert work.value == 3.0 * m * 4
    assert lib.sgh_prof_get(taken, buf, 64, C.byref(ms), C.byref(work)) == -1
    assert lib.sgh_prof_enable(0) == 0
    assert lib.sgh_prof_count(C.byref(n)) == 0 and n.value == taken   # kept for the reader
    assert lib.sgh_prof_clear() == 0
    assert lib.sgh_prof_count(C.byref(n)) == 0 and n.value == 0
    assert lib.sgh_prof_clear() == 0                        # idempotent
    assert (dx.to_numpy() == 2.0).all()


def test_no_profiling_records_inside_a_recording(singa, dev):
    """While the device records a graph no profiling record is taken (events inside a recording have no
    times); the recorded kernel replays with the right result, and records are taken again afterwards."""
    import ctypes as C
    from singa_amd import _lib
    lib = _lib.lib()
    m = 70000
    x = singa.from_numpy(np.linspace(-1, 1, m, dtype=np.float32), dev)
    dy = singa.Tensor((m,), dev); dy.SetFloatValue(3.0)
    n = C.c_int(-1)
    assert lib.sgh_prof_enable(1) == 0
    try:
        dev.EnableGraph(True)
        dx = singa.ReLUBackward(dy, x)
        dev.EnableGraph(False)
        assert lib.sgh_prof_count(C.byref(n)) == 0 and n.value == 0
        dev.RunGraph()
        dev.Sync()
        assert lib.sgh_prof_count(C.byref(n)) == 0 and n.value == 0
        want = np.where(np.linspace(-1, 1, m, dtype=np.float32) > 0, np.float32(3.0), np.float32(0.0))
        assert (dx.to_numpy() == want).all()
        dx2 = singa.ReLUBackward(dy, x)     # eager again: one record, with a duration
        dev.Sync()
        assert lib.sgh_prof_count(C.byref(n)) == 0 and n.value == 1
        buf = C.create_string_buffer(64)
        ms, work = C.c_float(), C.c_double()
        assert lib.sgh_prof_get(0, buf, 64, C.byref(ms), C.byref(work)) == 0 and ms.value > 0
        assert (dx2.to_numpy() == want).all()
    finally:
        dev.ResetGraph()
        lib.sgh_prof_enable(0)
        lib.sgh_prof_clear()


def test_upload_without_waiting(singa, dev):
    """sgh_upload_async: the host buffer may be overwritten as soon as the call returns, copies land
    in stream order (more uploads than staging slots in a row), oversize copies take the blocking path."""
    import ctypes as C
    from singa_amd import _lib
    lib = _lib.lib()
    host = np.zeros(3000, np.float32)
    tensors = []
    for i in range(20):
        host[:] = np.arange(3000, dtype=np.float32) + 1000 * i
        t = singa.Tensor((3000,), dev)
        _lib.check(lib.sgh_upload_async(dev._h, t.ptr, host.ctypes.data, host.nbytes), "sgh_upload_async")
        tensors.append(t)
    host[:] = -1
    for i, t in enumerate(tensors):
        assert_bit_equal(t.to_numpy(), np.arange(3000, dtype=np.float32) + 1000 * i, "upload %d" % i)
    big = np.arange(40000, dtype=np.float32)   # 160 KB: beyond a staging slot
    t = singa.Tensor((40000,), dev)
    _lib.check(lib.sgh_upload_async(dev._h, t.ptr, big.ctypes.data, big.nbytes), "sgh_upload_async")
    assert_bit_equal(t.to_numpy(), big, "large upload")
    assert lib.sgh_upload_async(dev._h, None, big.ctypes.data, 16) == -1
    assert lib.sgh_upload_async(dev._h, t.ptr, big.ctypes.data, 0) == 0


def test_pool_keeps_blocks_of_the_auxiliary_stream_until_the_join(singa, dev):
    """A block that work on the auxiliary stream uses may be freed right after that work was enqueued
    (SINGA's Graph does so): the pool hands it out again only once the main stream has been ordered
    behind the auxiliary one (Join / Sync), never to main-stream work that could overtake it."""
    from singa_amd._lib import lib
    n = (1 << 18) + 4096
    dev.Sync()

    def grab(k):     # k live tensors of the size class (whatever the pool has cached comes out first)
        return [singa.Tensor((n,), dev) for _ in range(k)]

    aux = dev.Fork()
    a = singa.Tensor((n,), dev)
    pa = a.ptr
    dev.UsedOn(aux, a)
    assert lib().sgh_memset_f32(pa, 3.0, n, aux) == 0      # work on the auxiliary stream writes the block
    cached0 = dev.PoolStats()["cached"]
    del a                                                  # freed while that work may still be running
    assert dev.PoolStats()["cached"] == cached0            # not back in the pool
    held = grab(12)
    assert pa not in [t.ptr for t in held]                 # and not handed to anyone
    held[0].SetFloatValue(7.0)
    cached1 = dev.PoolStats()["cached"]
    dev.Join()
    assert dev.PoolStats()["cached"] - cached1 >= 4 * n    # back in the pool after the join
    more = grab(64)
    assert pa in [t.ptr for t in more]                     # and handed out again
    assert (held[0].to_numpy() == 7.0).all()
    c = [t for t in more if t.ptr == pa][0]
    del more, held
    # marks are for this device's own blocks and streams only
    assert lib().sgh_block_used_on(dev._h, pa + 64, aux) == -1
    assert lib().sgh_block_used_on(dev._h, pa, 0xdead0) == -1
    assert lib().sgh_block_used_on(dev._h, pa, dev.stream) == 0
    # without a join, Sync releases what waited
    dev.Fork()
    dev.UsedOn(aux, c)
    del c
    held = grab(80)
    assert pa not in [t.ptr for t in held]
    dev.Sync()
    assert pa in [t.ptr for t in grab(8)]


@pytest.mark.parametrize("n", [1, 5, 1000, 4099, 1 << 20])
def test_elementwise_functions_around_the_path(singa, dev, n):
    """Sub, Div, Add/Mult/Div by a scalar: each is one IEEE operation per element, so NumPy's fp32
    result is the reference result bit for bit (Div by a scalar multiplies by the fp32 reciprocal
    as the reference does)."""
    r = rng(n + 7)
    a, b = randn(r, n), randn(r, n) + np.float32(3.0)
    ad, bd = singa.from_numpy(a, dev), singa.from_numpy(b, dev)
    assert_bit_equal(singa.__sub__(ad, bd).to_numpy(), a - b, "Sub")
    assert_bit_equal(singa.__div__(ad, bd).to_numpy(), a / b, "Div")
    assert_bit_equal(singa.AddFloat(ad, 1.25).to_numpy(), a + np.float32(1.25), "Add scalar")
    assert_bit_equal(singa.MultFloat(ad, -0.3).to_numpy(), a * np.float32(-0.3), "Mult scalar")
    assert_bit_equal(singa.DivFloat(ad, 64).to_numpy(), a * (np.float32(1.0) / np.float32(64)), "Div scalar")


# ---- the remaining Tensor functions: Transform / Broadcast, RowMax, Dot, SumAll, Uniform, Gaussian

def test_transform_and_broadcast(singa, dev):
    r = rng(31)
    m = randn(r, 37, 53)
    t = singa.from_numpy(m, dev)
    assert_bit_equal(singa.Transform(t.T()).to_numpy(), m.T.copy(), "transposed view made dense")
    assert singa.Transform(t) is t
    for src, shape in [((53,), (37, 53)), ((37, 1), (37, 53)), ((1,), (5, 4, 3)), ((4, 1, 3), (2, 4, 6, 3)),
                       ((2, 1, 1, 1, 3, 1, 1, 2), (2, 3, 2, 2, 3, 2, 2, 2))]:
        a = randn(r, *src)
        want = np.broadcast_to(a, shape)
        assert_bit_equal(singa.Broadcast(singa.from_numpy(a, dev), shape).to_numpy(), want, "broadcast %r -> %r" % (src, shape))
        assert_bit_equal(O.transform(a.ravel(), shape, [0 if s == 0 else s // 4 for s in want.strides]), want)
    with pytest.raises(singa.SingaHipError):
        singa.Broadcast(t, (37, 54))


def test_eltwise_ops_on_broadcast_and_transposed_operands(singa, dev):
    """Tensor *= / + with operands that are not dense: NumPy's result, as in the reference
    (src/core/tensor/tensor.cc:481-503 Broadcast, then the dense op)."""
    r = rng(32)
    a, row, col = randn(r, 12, 33), randn(r, 33), randn(r, 12, 1)
    ad, rowd, cold = (singa.from_numpy(v, dev) for v in (a, row, col))
    assert_bit_equal(singa.EltwiseMult(ad, rowd).to_numpy(), a * row, "matrix * row")
    assert_bit_equal(singa.__add__(cold, ad).to_numpy(), col + a, "column + matrix")
    b = randn(r, 33, 12)
    assert_bit_equal(singa.EltwiseMult(ad, singa.from_numpy(b, dev).T()).to_numpy(), a * b.T, "matrix * transposed view")
    assert_bit_equal(singa.__add__(rowd, cold).to_numpy(), row + col, "outer sum of a row and a column")
    with pytest.raises(singa.SingaHipError):
        singa.__add__(ad, singa.from_numpy(randn(r, 12, 32), dev))


def test_row_max_dot_and_sum(singa, dev):
    r = rng(33)
    for rows, cols in [(1, 1), (3, 7), (128, 1000), (17, 4097)]:
        m = randn(r, rows, cols)
        m[0] = -np.abs(m[0]) - 1          # an all-negative row, where the reference's two backends differ
        md = singa.from_numpy(m, dev)
        # the CPU function seeds the maximum with 0 (tensor_math_cpp.h:1132): the oracle's rule
        assert_bit_equal(singa.RowMax(md, cpu_rule=True).to_numpy(), O.row_max(m), "row max, CPU rule")
        assert singa.RowMax(md, cpu_rule=True).to_numpy()[0] == 0.0
        # the accelerator kernel seeds it with the row's first element (math_kernel.cu:488-499): the true
        # maximum, which is the default here
        assert_bit_equal(singa.RowMax(md).to_numpy(), m.max(axis=1), "row max, accelerator rule")
        assert singa.RowMax(md).to_numpy()[0] < 0.0
    for n in (1, 100, 4096, 4097, 1 << 20, 5 * (1 << 20) + 3):
        a, b = randn(r, n), randn(r, n)
        ad, bd = singa.from_numpy(a, dev), singa.from_numpy(b, dev)
        scale = float(np.abs(a.astype(np.float64) * b).sum())
        got = float(singa.Dot(ad, bd).to_numpy()[0])
        assert abs(got - float(a.astype(np.float64) @ b.astype(np.float64))) <= 1e-6 * scale + 1e-12
        assert abs(got - O.dot(a, b)) <= 1e-5 * scale + 1e-12          # the CPU function sums in another order
        assert got == float(singa.Dot(ad, bd).to_numpy()[0])           # run-to-run identical
        s = singa.SumAll(ad)
        assert abs(s - float(a.astype(np.float64).sum())) <= 1e-6 * float(np.abs(a).sum()) + 1e-12
        assert abs(s - O.sum_all(a)) <= 1e-5 * float(np.abs(a).sum()) + 1e-12


def test_uniform_and_gaussian_fills(singa, dev):
    """The device fills against the CPU twin of the same counter-based generator: uniform numbers
    bit for bit, Gaussian ones to the last place of the device's double-precision log / cos."""
    from singa_amd import rng as host
    dev.SetRandSeed(0x5167A123)
    n = 100003
    t = singa.Tensor((n,), dev)
    singa.Uniform(-2.0, 3.0, t)
    assert_bit_equal(t.to_numpy(), O.rng_uniform(0x5167A123, n, -2.0, 3.0), "uniform")
    singa.Uniform(0.0, 1.0, t)                                  # the stream continues where the last fill ended
    assert_bit_equal(t.to_numpy(), host.uniform(0x5167A123, (n,), offset=n), "uniform, continued")
    singa.Gaussian(0.5, 2.0, t)
    want = O.rng_normal(0x5167A123, n, 0.5, 2.0, offset=2 * n)
    got = t.to_numpy()
    assert int((got.view(np.uint32) != want.view(np.uint32)).sum()) <= n // 1000
    assert float(np.abs(got - want).max()) <= 1e-6 * 8
    dev.SetRandSeed(0x5167A123)                                 # the same seed replays the stream
    u = singa.Tensor((10,), dev)
    singa.Uniform(-2.0, 3.0, u)
    assert_bit_equal(u.to_numpy(), O.rng_uniform(0x5167A123, 10, -2.0, 3.0))


def test_clamp_and_the_half_precision_trip_of_a_gradient(singa, dev):
    from singa_amd import opt
    r = rng(34)
    g = (randn(r, 100003) * 60).astype(np.float32)
    g[:4] = [np.nan, np.inf, -np.inf, 100.0]
    gd = singa.from_numpy(g, dev)
    got = singa.Clamp(-100.0, 100.0, gd).to_numpy()
    want = np.where(g < -100, -100, np.where(g > 100, 100, g)).astype(np.float32)
    assert np.array_equal(got[1:], want[1:]) and np.isnan(got[0])
    sgd = opt.SGD(lr=0.1)
    out = sgd.through_half(gd, clipping=True, clip_value=100).to_numpy()
    with np.errstate(invalid="ignore"):
        assert np.array_equal(out[1:], want[1:].astype(np.float16).astype(np.float32))
    big = singa.from_numpy(np.array([70000.0, -1e-9, 3.0], np.float32), dev)
    assert np.array_equal(sgd.through_half(big).to_numpy(), np.array([np.inf, -0.0, 3.0], np.float32))   # no clipping: overflow


def test_int_float_casts(singa, dev):
    """AsType between float and int tensors (CastCopy<float, int> / <int, float>,
    src/core/tensor/math_kernel.cu:280-292): (int)x truncates toward zero, (float)i rounds to nearest even."""
    r = rng(41)
    for n in (1, 5, 4097, 1 << 20):
        f = (r.standard_normal(n) * 1000).astype(np.float32)
        f[: min(n, 6)] = [0.5, -0.5, 1.999, -1.999, -0.0, 2147483520.0][: min(n, 6)]
        it = singa.from_numpy(f, dev).AsType(singa.kInt)
        assert it.data_type() == singa.kInt
        assert np.array_equal(it.to_numpy(), np.trunc(f.astype(np.float64)).astype(np.int64).astype(np.int32))
        i = r.integers(-2 ** 31, 2 ** 31 - 1, size=n, dtype=np.int64).astype(np.int32)
        i[: min(n, 4)] = [0, -1, 16777217, -2 ** 31][: min(n, 4)]
        t = singa.Tensor((n,), dev, singa.kInt)
        t.CopyIntDataFromHostPtr(i)
        assert_bit_equal(t.AsType(singa.kFloat32).to_numpy(), i.astype(np.float32), "int -> float")
    # out of range saturates, NaN becomes 0 (the conversion instruction's rule; C leaves both undefined)
    edge = np.array([3e9, -3e9, np.inf, -np.inf, np.nan], dtype=np.float32)
    got = singa.from_numpy(edge, dev).AsType(singa.kInt).to_numpy()
    assert got.tolist() == [2 ** 31 - 1, -2 ** 31, 2 ** 31 - 1, -2 ** 31, 0]
