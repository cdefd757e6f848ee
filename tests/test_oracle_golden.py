"""The CPU oracle against every vector the reference's own tests hold for the backward path
(tests/golden/reference_vectors.json; each entry names its source file:line)."""
import numpy as np
import pytest

from oracle import cpu_oracle as O


def _a(v, shape=None):
    a = np.array(v, dtype=np.float32)
    return a.reshape(shape) if shape is not None else a


def test_conv_forward(golden):
    g = golden["conv"]
    y = O.conv_fwd(_a(g["x"], g["x_shape"]), _a(g["w"], g["w_shape"]), _a(g["bias"]), g["stride"], g["pad"])
    assert y.shape == (2, 1, 2, 2)
    assert np.array_equal(y.ravel(), _a(g["y"]))  # EXPECT_EQ in the reference


def test_conv_backward(golden):
    g = golden["conv"]
    x, w, dy = _a(g["x"], g["x_shape"]), _a(g["w"], g["w_shape"]), _a(g["dy"], g["dy_shape"])
    dx, dw = O.conv_bwd(dy, x, w, g["stride"], g["pad"])
    db = O.conv_bgrad(dy)
    dyf, wf, xf = dy.ravel(), w.ravel(), x.ravel()
    for i, terms in enumerate(g["dx_terms"]):
        exp = np.float32(0)
        for a, b in terms:
            exp = np.float32(exp + np.float32(dyf[a] * wf[b]))
        assert dx.ravel()[i] == exp, ("dx", i)  # EXPECT_EQ: exact
    np.testing.assert_allclose(db[0], sum(float(dyf[i]) for i in g["db_terms"]), rtol=4e-7)
    for i, terms in enumerate(g["dw_terms"]):
        exp = sum(float(dyf[a]) * float(xf[b]) for a, b in terms)
        np.testing.assert_allclose(dw.ravel()[i], exp, rtol=5e-7)  # EXPECT_FLOAT_EQ = 4 ulp


def test_max_pool(golden):
    g = golden["pool_max"]
    x, dy = _a(g["x"], g["x_shape"]), _a(g["dy"], g["dy_shape"])
    y, mask = O.pool_max_fwd(x, g["kernel"], g["stride"], g["pad"])
    assert np.array_equal(y.ravel(), _a(g["y"]))
    dx = O.pool_max_bwd(dy, mask, x.shape)
    assert np.array_equal(dx.ravel(), _a(g["dx"]))  # EXPECT_EQ: exact


def test_pool_api_vectors(golden):
    g = golden["pool_api"]
    x, dy = _a(g["x"], g["x_shape"]), _a(g["dy"], g["dy_shape"])
    y, mask = O.pool_max_fwd(x, g["kernel"], g["stride"], g["pad"])
    assert np.array_equal(y.ravel(), _a(g["max_y"]))
    assert np.array_equal(O.pool_max_bwd(dy, mask, x.shape).ravel(), _a(g["max_dx"]))
    for inc in (False, True):  # no padding: both divisor conventions agree
        ya = O.pool_avg_fwd(x, g["kernel"], g["stride"], g["pad"], include_pad=inc)
        np.testing.assert_allclose(ya.ravel(), _a(g["avg_y"]), atol=1e-6)
        dxa = O.pool_avg_bwd(dy, x.shape, g["kernel"], g["stride"], g["pad"], include_pad=inc)
        np.testing.assert_allclose(dxa.ravel(), _a(g["avg_dx"]), atol=1e-6)


def test_softmax_cross_entropy(golden):
    g = golden["softmax_ce"]
    p = O.softmax(_a(g["p"], g["p_shape"]))  # the legacy loss layer applies SoftMax first
    np.testing.assert_allclose(p, 0.25, rtol=1e-6)
    for t in (np.array(g["t_index"], dtype=np.int32), np.array(g["t_onehot"], dtype=np.int32).reshape(2, 4)):
        loss = O.cross_entropy_fwd(p, t)
        np.testing.assert_allclose(loss, np.float32(-np.log(0.25)), rtol=4e-7)
        grad = O.softmax_ce_bwd(p, t)
        np.testing.assert_allclose(grad.ravel(), _a(g["grad"]), rtol=4e-7)


def test_negative_label_is_rejected():
    p = np.full((2, 4), 0.25, dtype=np.float32)
    with pytest.raises(ValueError):
        O.softmax_ce_bwd(p, np.array([0, -1], dtype=np.int32))
    with pytest.raises(ValueError):
        O.softmax_ce_bwd(p, np.array([4, 0], dtype=np.int32))


def test_bn_forward_cudnn_vector(golden):
    g = golden["bn_cudnn"]
    x = _a(g["x"], g["x_shape"])
    rm, rv = np.zeros(2, np.float32), np.zeros(2, np.float32)
    y, mean, invstd = O.bn_fwd_train(x, _a(g["gamma"]), _a(g["beta"]), rm, rv, factor=0.9)
    np.testing.assert_allclose(y.ravel(), _a(g["y"]), atol=g["tol"])
    xs = x.astype(np.float64)
    np.testing.assert_allclose(mean, xs.mean(axis=(0, 2, 3)), rtol=1e-6)
    np.testing.assert_allclose(invstd, 1 / np.sqrt(xs.var(axis=(0, 2, 3)) + 1e-5), rtol=1e-6)
    # running = (1 - factor) * running + factor * batch, unbiased variance, from zero
    np.testing.assert_allclose(rm, 0.9 * xs.mean(axis=(0, 2, 3)), rtol=1e-5)
    np.testing.assert_allclose(rv, 0.9 * xs.var(axis=(0, 2, 3)) * 16 / 15, rtol=1e-5)


def test_bn_backward_cudnn_vector(golden):
    g = golden["bn_cudnn"]
    x, dy = _a(g["x"], g["x_shape"]), _a(g["dy"], g["x_shape"])
    # the reference layer's Forward recomputes the statistics; the mean_/var_ arrays its test
    # declares are never used (see the fixture's note)
    _, mean, invstd = O.bn_fwd_train(x, _a(g["gamma"]), _a(g["beta"]))
    dx, dg, db = O.bn_bwd(dy, x, _a(g["gamma"]), mean, invstd)
    np.testing.assert_allclose(dx.ravel(), _a(g["dx"]), atol=g["tol"])
    np.testing.assert_allclose(dg, _a(g["dgamma"]), atol=g["tol"])
    np.testing.assert_allclose(db, _a(g["dbeta"]), atol=g["tol"])
    # tighter: the vector carries ~6 significant digits
    np.testing.assert_allclose(dx.ravel(), _a(g["dx"]), rtol=1e-4, atol=5e-7)
    np.testing.assert_allclose(dg, _a(g["dgamma"]), rtol=1e-5)
    np.testing.assert_allclose(db, _a(g["dbeta"]), rtol=1e-5)


def test_bn_backward_api_vector(golden):
    g = golden["bn_api"]
    x, dy = _a(g["x"], g["x_shape"]), _a(g["dy"], g["x_shape"])
    gamma = _a(g["gamma"])
    _, mean, invstd = O.bn_fwd_train(x, gamma, np.zeros(3, np.float32))
    dx, _, _ = O.bn_bwd(dy, x, gamma, mean, invstd)
    # dy == x here, so dx is pure cancellation (~1e-5); the reference asserts 6 decimals
    np.testing.assert_allclose(dx.ravel(), _a(g["dx"]), atol=1e-6)


def test_relu(golden):
    g = golden["relu"]
    x, dy = _a(g["x"], g["x_shape"]), _a(g["dy"], g["x_shape"])
    assert np.array_equal(O.relu_fwd(x).ravel(), _a(g["y"]))
    assert np.array_equal(O.relu_bwd(dy, x).ravel(), _a(g["dx"]))
    # gradient at exactly zero is zero (strict '>')
    assert O.relu_bwd(np.ones(3, np.float32), np.array([0.0, -0.0, 1e-30], np.float32)).tolist() == [0, 0, 1]


def test_bn_2d_layer_vectors(golden):
    """The legacy BatchNorm layer on a [batch, features] input (test/singa/test_batchnorm.cc:44-129): every
    feature normalised over the batch, i.e. the 4-D case with planes of one element."""
    g = golden["bn_2d"]
    x, dy = _a(g["x"], g["x_shape"]), _a(g["dy"], g["x_shape"])
    y, _, _ = O.bn_fwd_train(x, _a(g["fwd_gamma"]), _a(g["fwd_beta"]))
    np.testing.assert_allclose(y.ravel(), _a(g["y"]), atol=g["tol"])
    _, mean, invstd = O.bn_fwd_train(x, _a(g["bwd_gamma"]), _a(g["bwd_beta"]))
    dx, dg, db = O.bn_bwd(dy, x, _a(g["bwd_gamma"]), mean, invstd)
    np.testing.assert_allclose(dx.ravel(), _a(g["dx"]), atol=g["tol"])
    np.testing.assert_allclose(dg, _a(g["dgamma"]), atol=g["tol"])
    np.testing.assert_allclose(db, _a(g["dbeta"]), atol=g["tol"])
    # the same numbers through the 4-D entry: [N, C] is [N, C, 1, 1]
    dx4, dg4, db4 = O.bn_bwd(dy.reshape(2, 2, 1, 1), x.reshape(2, 2, 1, 1), _a(g["bwd_gamma"]), mean, invstd)
    assert np.array_equal(dx4.ravel(), dx.ravel()) and np.array_equal(dg4, dg) and np.array_equal(db4, db)


def test_dense_bias_gradient_vector(golden):
    """Dense.Backward's bias gradient (test/singa/test_dense.cc:75-137): column sums of dy, the one thing the
    reference test asserts; dx and dW (its assertions are commented out) against float64 instead."""
    g = golden["dense"]
    x, w, dy = _a(g["x"], g["x_shape"]), _a(g["w"], g["w_shape"]), _a(g["dy"], g["dy_shape"])
    db = O.sum_rows(dy)
    for i, terms in enumerate(g["db_terms"]):
        exp = np.float32(0)
        for k in terms:
            exp = np.float32(exp + dy.ravel()[k])
        np.testing.assert_allclose(db[i], exp, rtol=5e-7)   # EXPECT_FLOAT_EQ
    dx = O.sgemm(dy, w, transB=True)      # dy . W^T  (python/singa/autograd.py:613-623)
    dw = O.sgemm(x, dy, transA=True)      # x^T . dy
    np.testing.assert_allclose(dx, dy.astype(np.float64) @ w.astype(np.float64).T, rtol=1e-6)
    np.testing.assert_allclose(dw, x.astype(np.float64).T @ dy.astype(np.float64), rtol=1e-6)


def test_relu_layer_vectors(golden):
    g = golden["relu_layer"]
    x, dy = _a(g["x"]), _a(g["dy"])
    y, dx = O.relu_fwd(x), O.relu_bwd(dy, x)
    for i in g["asserted_dx_elements"]:      # what the reference test checks (EXPECT_FLOAT_EQ)
        assert y[i] == np.float32(g["y"][i]) and dx[i] == np.float32(g["dx"][i])
    assert np.array_equal(y, _a(g["y"])) and np.array_equal(dx, _a(g["dx"]))


def test_sgd_reference_cases(golden):
    g = golden["sgd"]
    shape = tuple(g["shape"])
    for c in g["cases"]:
        w = np.full(shape, c["w0"], np.float32)
        grad0 = np.full(shape, c["g"], np.float32)
        v = np.zeros(shape, np.float32)
        f32 = np.float32
        lr, mu, wd = f32(c["lr"]), f32(c["mu"]), f32(c["wd"])
        # expected values with the test's own formulas (float32 tensor arithmetic)
        if c["name"] == "const_lr":
            exp = [f32(c["w0"]) - lr * f32(c["g"])]
        elif c["name"] == "momentum":
            w1 = f32(c["w0"]) - lr * f32(c["g"])
            buf = f32(c["g"]) + f32(c["g"]) * mu
            exp = [w1, w1 - lr * buf]
        elif c["name"] == "weight_decay":
            exp = [f32(c["w0"]) - lr * (f32(c["g"]) + wd * f32(c["w0"]))]
        else:
            exp = [f32(c["w0"]) - lr * (f32(c["g"]) + mu * f32(c["g"]))]
        for step in range(c["steps"]):
            grad = grad0.copy()
            O.sgd_momentum(w, grad, v, c["lr"], mu=c["mu"], wd=c["wd"], nesterov=bool(c["nesterov"]))
            np.testing.assert_array_almost_equal(w, np.full(shape, exp[step]), decimal=5)
