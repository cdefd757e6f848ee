"""GPU parity: operation entry points (conv dgrad/wgrad/bias-grad, BatchNorm, pooling) against
the CPU oracle, through the C ABI.

Tolerances: max-pool routing and average pooling are bit-exact; conv and BatchNorm reductions
are compared with the normalised L2 error ||gpu - cpu|| / ||cpu|| <= 1e-3 (fp32), the bound the
task states for reductions whose summation order differs from the CPU's by construction."""
import os

import numpy as np
import pytest

from oracle import cpu_oracle as O
from util import assert_bit_equal, nl2, randn, rng

pytestmark = pytest.mark.gpu

TOL = 1e-3   # stated bound; the observed error is printed and is typically < 1e-6


@pytest.fixture(scope="module")
def singa():
    from singa_amd import singa_wrap
    return singa_wrap


def run_conv(singa, dev, x, w, b, dy, stride, pad):
    N, C, H, W = x.shape
    K, _, R, S = w.shape
    xd, wd, dyd = singa.from_numpy(x, dev), singa.from_numpy(w, dev), singa.from_numpy(dy, dev)
    h = singa.CudnnConvHandle(xd, (R, S), stride, pad, C, K, b is not None)
    dx = singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy()
    dw = singa.GpuConvBackwardW(dyd, xd, wd, h).to_numpy()
    db = singa.GpuConvBackwardb(dyd, singa.from_numpy(b, dev), h).to_numpy() if b is not None else None
    return h, dx, dw, db


def test_conv_reference_vector(singa, dev, golden):
    g = golden["conv"]
    x = np.array(g["x"], np.float32).reshape(g["x_shape"])
    w = np.array(g["w"], np.float32).reshape(g["w_shape"])
    b = np.array(g["bias"], np.float32)
    dy = np.array(g["dy"], np.float32).reshape(g["dy_shape"])
    xd, wd, bd = singa.from_numpy(x, dev), singa.from_numpy(w, dev), singa.from_numpy(b, dev)
    h = singa.CudnnConvHandle(xd, (3, 3), g["stride"], g["pad"], 1, 1, True)
    assert (h.conv_height, h.conv_width, h.col_height, h.col_width) == (2, 2, 9, 4)
    y = singa.GpuConvForward(xd, wd, bd, h).to_numpy()
    np.testing.assert_allclose(y.ravel(), np.array(g["y"], np.float32), rtol=1e-6)
    _, dx, dw, db = run_conv(singa, dev, x, w, b, dy, g["stride"], g["pad"])
    dyf, wf, xf = dy.ravel(), w.ravel(), x.ravel()
    for i, terms in enumerate(g["dx_terms"]):
        np.testing.assert_allclose(dx.ravel()[i], sum(float(dyf[a]) * float(wf[c]) for a, c in terms), rtol=1e-6, atol=1e-7)
    for i, terms in enumerate(g["dw_terms"]):
        np.testing.assert_allclose(dw.ravel()[i], sum(float(dyf[a]) * float(xf[c]) for a, c in terms), rtol=1e-6)
    np.testing.assert_allclose(db[0], float(dyf.sum()), rtol=1e-6)


CONV_CASES = [
    # N, C, H, W, K, R, S, stride, pad, bias
    (2, 3, 7, 6, 4, 3, 3, (1, 1), (1, 1), True),
    (2, 3, 9, 8, 5, 3, 3, (2, 2), (1, 1), False),
    (2, 2, 6, 7, 3, 3, 2, (2, 1), (0, 1), True),          # non-square kernel / stride / pad
    (3, 16, 8, 8, 32, 1, 1, (2, 2), (0, 0), False),       # 1x1 stride-2 downsample
    (2, 3, 32, 32, 32, 5, 5, (1, 1), (2, 2), True),       # small-CNN conv1
    (2, 32, 16, 16, 64, 5, 5, (1, 1), (2, 2), True),      # small-CNN conv2
    (2, 3, 64, 64, 64, 7, 7, (2, 2), (3, 3), False),      # ResNet stem (reduced image)
    (2, 64, 14, 14, 64, 3, 3, (1, 1), (1, 1), True),      # stage-1 class (forward: shared-tile kernel with bias)
    (2, 64, 14, 14, 128, 3, 3, (2, 2), (1, 1), False),    # stage transition
    (2, 128, 7, 7, 128, 3, 3, (1, 1), (1, 1), True),      # odd spatial size (forward bias added by the split reduction)
    (1, 130, 9, 9, 70, 3, 3, (1, 1), (1, 1), False),      # channel counts that are not tile multiples
    (4, 8, 5, 5, 8, 3, 3, (1, 1), (0, 0), False),         # no padding
    (1, 1, 3, 3, 1, 3, 3, (1, 1), (2, 2), False),         # pad wider than half the kernel
    (2, 40, 9, 11, 24, 3, 3, (2, 2), (1, 1), False),      # stride 2, odd image: residue classes of unequal size
    (2, 34, 10, 10, 20, 3, 3, (3, 3), (1, 1), False),     # stride 3: nine residue classes
    (3, 64, 8, 8, 128, 1, 1, (2, 2), (0, 0), False),      # 1x1 stride 2: three classes receive no tap at all
    (1, 32, 12, 12, 16, 5, 5, (2, 2), (2, 2), False),
    (2, 32, 8, 8, 32, 2, 2, (2, 2), (0, 0), False),       # kernel == stride
    (1, 32, 7, 7, 16, 1, 1, (3, 3), (0, 0), False),       # kernel smaller than stride
    (2, 36, 9, 7, 33, 3, 2, (2, 1), (1, 0), True),        # mixed strides, non-square kernel
    (2, 4, 12, 12, 8, 3, 3, (2, 2), (1, 1), False),       # few input channels: column-GEMM + gather path, strided
    (2, 32, 12, 12, 64, 3, 3, (1, 1), (0, 0), False),     # shared-slab wgrad without padding
    (2, 64, 10, 10, 64, 3, 3, (1, 1), (2, 2), False),     # ... with padding 2 (output larger than input)
    (2, 32, 13, 13, 128, 3, 3, (2, 2), (1, 1), False),    # ... stride 2 on an odd image (dgrad: residue-class GEMMs)
    (2, 32, 16, 16, 128, 3, 3, (2, 2), (0, 0), True),     # ... stride 2 without padding
    (1, 32, 62, 62, 64, 3, 3, (1, 1), (1, 1), False),     # widest rows the 64-column slab holds
    (1, 64, 30, 30, 64, 3, 3, (1, 1), (1, 1), False),     # widest rows the 32-column slab holds
    (3, 96, 9, 20, 160, 3, 3, (1, 1), (1, 1), False),     # non-square image, channel tails in both tile dimensions
    (1, 64, 56, 56, 128, 3, 3, (2, 2), (1, 1), False),    # stage transitions at full spatial size: four residue
    (2, 128, 28, 28, 64, 3, 3, (2, 2), (1, 1), False),    #   classes per workgroup, tiles crossing image boundaries
    (5, 68, 14, 14, 48, 3, 3, (2, 2), (1, 1), True),      #   (7x7 class grid: up to 3 crossings), ragged channel counts
    (1, 3, 224, 224, 64, 7, 7, (2, 2), (3, 3), False),    # ResNet stem at full image size
    (3, 3, 40, 40, 96, 7, 7, (2, 2), (3, 3), True),       # stem-like, output channels over two 64-row tiles (second partial)
    (2, 2, 24, 24, 40, 7, 7, (1, 1), (3, 3), False),      # few-channel large-filter path at stride 1
    (2, 4, 24, 24, 16, 5, 5, (2, 2), (2, 2), False),      # direct few-channel dgrad: 5x5 (three offsets per dimension), C = 4
    (2, 1, 16, 16, 8, 7, 7, (2, 2), (3, 3), True),        # direct few-channel dgrad: one channel
    (32, 96, 57, 57, 32, 1, 1, (2, 2), (0, 0), False),    # 1x1 stride 2, 64 x 64 wavefront tiles: ragged channel tile, odd image
    (2, 48, 11, 11, 64, 1, 1, (3, 3), (0, 0), False),     # 1x1 stride 3 on the matrix-instruction-from-global-memory kernel
    (3, 40, 28, 28, 96, 1, 1, (2, 2), (0, 0), True),      # 1x1 stride 2, rows of 14: pointwise weight gradient, ragged tiles
    (2, 64, 56, 56, 130, 1, 1, (2, 2), (0, 0), False),    # ... rows of 28, a second (nearly empty) row tile
    (5, 33, 14, 14, 160, 1, 1, (2, 2), (0, 0), False),    # ... rows of 7 (odd: zero column behind the pixels)
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_backward_vs_oracle(singa, dev, case):
    N, C, H, W, K, R, S, stride, pad, bias = case
    r = rng(abs(hash(case)) % 2**31)
    x = randn(r, N, C, H, W)
    w = (randn(r, K, C, R, S) * np.sqrt(2.0 / (C * R * S))).astype(np.float32)
    b = randn(r, K) if bias else None
    P, Q = (H + 2 * pad[0] - R) // stride[0] + 1, (W + 2 * pad[1] - S) // stride[1] + 1
    dy = randn(r, N, K, P, Q)
    h, dx, dw, db = run_conv(singa, dev, x, w, b, dy, stride, pad)
    dx_o, dw_o = O.conv_bwd(dy, x, w, stride, pad)
    e_dx, e_dw = nl2(dx, dx_o), nl2(dw, dw_o)
    print("dgrad nl2 %.2e  wgrad nl2 %.2e" % (e_dx, e_dw))
    assert e_dx < TOL and e_dw < TOL
    if bias:
        assert nl2(db, O.conv_bgrad(dy)) < TOL
    # forward, which produces the activations the backward consumes
    xd, wd = singa.from_numpy(x, dev), singa.from_numpy(w, dev)
    y = singa.GpuConvForward(xd, wd, singa.from_numpy(b, dev) if bias else None, h).to_numpy()
    assert nl2(y, O.conv_fwd(x, w, b, stride, pad)) < TOL


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", [
    (2, 64, 14, 14, 64, 3, 3, (1, 1), (1, 1), 2, True),      # two groups of a shared-tile layer
    (3, 32, 9, 11, 48, 3, 3, (2, 2), (1, 1), 4, False),      # stride 2, ragged image, 8 -> 12 channels per group
    (2, 24, 12, 12, 24, 3, 3, (1, 1), (1, 1), 24, True),     # depthwise (the first half of SeparableConv2d)
    (4, 16, 8, 8, 40, 1, 1, (1, 1), (0, 0), 8, False),       # pointwise, 2 -> 5 channels per group
    (1, 6, 7, 5, 9, 5, 3, (2, 1), (2, 1), 3, True),          # generic path
])
def test_grouped_conv_vs_oracle(singa, dev, kind, case):
    """Grouped convolution (CudnnConvHandle's `groups`): forward, data, weight and bias gradient against the
    per-group oracle, fp32 at the reduction bar and on 16-bit tensors (stored values, 1e-2)."""
    N, C, H, W, K, R, S, stride, pad, G, bias = case
    r = rng(sum(case[:7]) + 31 * G)
    dt = {"f32": singa.kFloat32, "f16": singa.kFloat16, "bf16": singa.kBFloat16}[kind]
    tol = TOL if kind == "f32" else 1e-2

    def to(a):
        t = singa.from_numpy(a.astype(np.float32), dev)
        if kind != "f32":
            t = t.AsType(dt)
        return t, (t.AsType(singa.kFloat32) if kind != "f32" else t).to_numpy()
    xt, x = to(randn(r, N, C, H, W))
    wt, w = to(randn(r, K, C // G, R, S) * np.sqrt(2.0 * G / (C * R * S)))
    bt, b = to(randn(r, K)) if bias else (None, None)
    h = singa.CudnnConvHandle(xt, (R, S), stride, pad, C, K, bias, G)
    assert h.group == G and h.channels_per_filter == C // G
    y = singa.GpuConvForward(xt, wt, bt, h)
    y_o = O.conv_fwd_grouped(x, w, b, stride, pad, G)
    assert y.shape() == list(y_o.shape) and nl2(y.to_numpy(), y_o) < tol
    dyt, dy = to(randn(r, *y_o.shape))
    dx_o, dw_o = O.conv_bwd_grouped(dy, x, w, stride, pad, G)
    dx = singa.GpuConvBackwardx(dyt, wt, xt, h)
    dw = singa.GpuConvBackwardW(dyt, xt, wt, h)
    e = nl2(dx.to_numpy(), dx_o), nl2(dw.to_numpy(), dw_o)
    print("grouped conv %s: dx %.2e dw %.2e" % (kind, e[0], e[1]))
    assert dw.shape() == [K, C // G, R, S] and max(e) < tol
    if bias:
        assert nl2(singa.GpuConvBackwardb(dyt, bt, h).to_numpy(), O.conv_bgrad(dy)) < tol
        if kind == "f32":
            dW2, db2 = singa.GpuConvBackwardWb(dyt, xt, wt, bt, h)
            assert_bit_equal(dW2.to_numpy(), dw.to_numpy(), "grouped dW with bias")
            assert nl2(db2.to_numpy(), O.conv_bgrad(dy)) < tol
    # the tensors outside the slices stay untouched: a second call gives the same bits
    assert_bit_equal(singa.GpuConvBackwardx(dyt, wt, xt, h).to_numpy(), dx.to_numpy(), "grouped dx again")


@pytest.mark.parametrize("case", [c for c in CONV_CASES if c[-1]] + [
    (4, 32, 16, 16, 64, 5, 5, (1, 1), (2, 2), True),      # generic kernel, split reduction: db rides along as a column of ones
    (1, 20, 6, 6, 40, 5, 5, (1, 1), (2, 2), True),        # ... without a split (one chunk range): written straight to db
    (2, 32, 9, 9, 16, 2, 2, (1, 1), (0, 0), True),        # C*R*S = 128, a whole number of column tiles: the reduction kernel instead
])
def test_conv_weight_and_bias_gradient_in_one_call(singa, dev, case):
    """GpuConvBackwardWb: dW bit-identical to GpuConvBackwardW (same kernel, the extra column changes no
    other sum), db within the reduction bar of the CPU oracle and of GpuConvBackwardb."""
    N, C, H, W, K, R, S, stride, pad, _ = case
    r = rng(abs(hash(case)) % 2**31 + 5)
    x, w, b = randn(r, N, C, H, W), randn(r, K, C, R, S), randn(r, K)
    P, Q = (H + 2 * pad[0] - R) // stride[0] + 1, (W + 2 * pad[1] - S) // stride[1] + 1
    dy = (randn(r, N, K, P, Q) + 0.25).astype(np.float32)    # (a mean, so that db is not a sum that cancels)
    xd, wd, bd, dyd = (singa.from_numpy(a, dev) for a in (x, w, b, dy))
    h = singa.CudnnConvHandle(xd, (R, S), stride, pad, C, K, True)
    dW, db = singa.GpuConvBackwardWb(dyd, xd, wd, bd, h)
    assert_bit_equal(dW.to_numpy(), singa.GpuConvBackwardW(dyd, xd, wd, h).to_numpy(), "dW")
    want = O.conv_bgrad(dy)
    e = (nl2(db.to_numpy(), want), nl2(db.to_numpy(), singa.GpuConvBackwardb(dyd, bd, h).to_numpy()))
    print("db nl2 vs oracle %.2e, vs the separate kernel %.2e" % e)
    assert max(e) < TOL
    dW2, db2 = singa.GpuConvBackwardWb(dyd, xd, wd, bd, h)     # run-to-run identical
    assert_bit_equal(db2.to_numpy(), db.to_numpy(), "db again")


def test_conv_dgrad_with_batched_weight_relayout(singa, dev):
    """GpuConvPrepareBackward re-lays the weights of all CONV_CASES layers in one launch; the data
    gradients (plain and accumulating) that follow skip their own re-layout and must give the same
    bits; layers whose kernel reads W as it is are left alone; a prepared layer's note is used once."""
    layers = []
    for i, case in enumerate(CONV_CASES):
        N, C, H, W, K, R, S, stride, pad, _ = case
        r = rng(2000 + i)
        P, Q = (H + 2 * pad[0] - R) // stride[0] + 1, (W + 2 * pad[1] - S) // stride[1] + 1
        xd, wd = singa.from_numpy(randn(r, N, C, H, W), dev), singa.from_numpy(randn(r, K, C, R, S), dev)
        dyd = singa.from_numpy(randn(r, N, K, P, Q), dev)
        h = singa.CudnnConvHandle(xd, (R, S), stride, pad, C, K, False)
        old = randn(r, N, C, H, W)
        want = singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy()
        want_acc = singa.GpuConvBackwardxAccumulate(dyd, wd, xd, h, singa.from_numpy(old, dev)).to_numpy()
        layers.append((case, xd, wd, dyd, h, old, want, want_acc))
    singa.GpuConvPrepareBackward([(l[2], l[4]) for l in layers])
    prelaid = [bool(l[4].geom.prelaid_W) for l in layers]
    assert False in prelaid and prelaid.count(True) >= 6, prelaid
    for case, xd, wd, dyd, h, old, want, want_acc in layers:
        assert_bit_equal(singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy(), want, "prepared dgrad %r" % (case,))
        assert not h.geom.prelaid_W            # a note is used once
    singa.GpuConvPrepareBackward([(l[2], l[4]) for l in layers])
    for case, xd, wd, dyd, h, old, want, want_acc in layers:
        got = singa.GpuConvBackwardxAccumulate(dyd, wd, xd, h, singa.from_numpy(old, dev)).to_numpy()
        assert_bit_equal(got, want_acc, "prepared accumulating dgrad %r" % (case,))
        assert not h.geom.prelaid_W


def test_prepared_weights_are_never_stale(singa, dev):
    """What a caller can do wrong after GpuConvPrepareBackward, and still gets the gradient of the
    CURRENT weights: (1) the weights change before the data gradient (an optimizer update, an upload
    into the tensor, the caller's own write announced by ConvWeightsChanged); (2) another pass of
    the same handle overwrites the workspace; (3) a different weight tensor is handed in."""
    from singa_amd import opt
    N, C, H, W, K = 2, 64, 14, 14, 64
    r = rng(77)
    x, w, w2, dy = randn(r, N, C, H, W), randn(r, K, C, 3, 3), randn(r, K, C, 3, 3), randn(r, N, K, H, W)
    xd, dyd = singa.from_numpy(x, dev), singa.from_numpy(dy, dev)
    h = singa.CudnnConvHandle(xd, (3, 3), (1, 1), (1, 1), C, K, False)
    ref_h = singa.CudnnConvHandle(xd, (3, 3), (1, 1), (1, 1), C, K, False)

    def fresh(wt):
        return singa.GpuConvBackwardx(dyd, wt, xd, ref_h).to_numpy()

    # (1a) an optimizer update between prepare and data gradient
    wd = singa.from_numpy(w, dev)
    singa.GpuConvPrepareBackward([(wd, h)])
    assert h.geom.prelaid_W == wd.ptr
    sgd = opt.SGD(lr=0.1, momentum=0.9)
    sgd.apply("w", wd, singa.from_numpy(w2, dev))
    assert_bit_equal(singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy(), fresh(wd), "after an update")
    # (1b) new values uploaded into the same tensor
    singa.GpuConvPrepareBackward([(wd, h)])
    wd.CopyFloatDataFromHostPtr(w2)
    assert_bit_equal(singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy(), fresh(wd), "after an upload")
    # (1c) the caller's own write, announced
    singa.GpuConvPrepareBackward([(wd, h)])
    other = singa.from_numpy(w, dev)
    singa.ConvWeightsChanged()
    assert_bit_equal(singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy(), fresh(wd), "after ConvWeightsChanged")
    # (2) the weight gradient / the forward pass of the same handle ran on the prepared workspace
    for other_pass in (lambda: singa.GpuConvBackwardW(dyd, xd, wd, h), lambda: singa.GpuConvForward(xd, wd, None, h)):
        singa.GpuConvPrepareBackward([(wd, h)])
        other_pass()
        assert not h.geom.prelaid_W
        assert_bit_equal(singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy(), fresh(wd), "after another pass")
    # (3) prepared for one weight tensor, called with another
    singa.GpuConvPrepareBackward([(wd, h)])
    assert_bit_equal(singa.GpuConvBackwardx(dyd, other, xd, h).to_numpy(), fresh(other), "another weight tensor")
    # (1d) in-place tensor arithmetic on the weight: `W *= s` (EltwiseMult with a scalar tensor on the right, the
    # optimizer's own idiom, python/singa/opt.py:299-300) and `W += t`; the same ops on OTHER tensors leave the
    # note alone (a backward pass runs many of them between the prepare and its data gradients)
    half = singa.from_numpy(np.array([0.5], np.float32), dev)
    acts, acts2, w2d = singa.from_numpy(x, dev), singa.from_numpy(x, dev), singa.from_numpy(w2, dev)
    singa.GpuConvPrepareBackward([(wd, h)])
    acts *= half
    acts += acts2
    wd *= half
    assert_bit_equal(singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy(), fresh(wd), "after W *= s")
    singa.GpuConvPrepareBackward([(wd, h)])
    wd += w2d
    assert_bit_equal(singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy(), fresh(wd), "after W += t")
    # (1e) a replayed recording that holds an update: the library cannot see inside it
    g = singa.from_numpy(w2, dev)
    sgd2 = opt.SGD(lr=0.05, momentum=0.0)
    sgd2.apply("w", wd, g)
    dev.Sync()
    dev.EnableGraph(True)
    sgd2.apply("w", wd, g)
    dev.EnableGraph(False)
    try:
        singa.GpuConvPrepareBackward([(wd, h)])
        dev.RunGraph()
        assert_bit_equal(singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy(), fresh(wd), "after a replayed update")
    finally:
        dev.ResetGraph()


def test_conv_wgrad_is_deterministic(singa, dev):
    r = rng(4)
    x, dy = randn(r, 8, 64, 28, 28), randn(r, 8, 64, 28, 28)
    w = randn(r, 64, 64, 3, 3)
    xd, wd, dyd = singa.from_numpy(x, dev), singa.from_numpy(w, dev), singa.from_numpy(dy, dev)
    h = singa.CudnnConvHandle(xd, (3, 3), (1, 1), (1, 1), 64, 64, False)
    a = singa.GpuConvBackwardW(dyd, xd, wd, h).to_numpy()
    for _ in range(3):
        assert_bit_equal(singa.GpuConvBackwardW(dyd, xd, wd, h).to_numpy(), a, "split-K reduction order")


@pytest.mark.parametrize("n,c,hw,k,r,stride,pad", [
    (40, 64, 56, 64, 3, 1, 1),    # shared remainder tiles: whole-tile stores and the fix-up pass both add
    (16, 256, 14, 256, 3, 1, 1),  # every tile shared
    (16, 64, 28, 128, 3, 2, 1),   # residue-class kernel
    (3, 64, 9, 64, 3, 1, 1),      # odd image, tiles straddle images
    (4, 64, 16, 128, 1, 2, 0),    # not covered by the accumulating kernels: the two-step fallback
    (2, 8, 12, 16, 5, 1, 2),      # generic path: fallback
])
def test_conv_dgrad_accumulate(singa, dev, n, c, hw, k, r, stride, pad):
    """dx += dgrad (the residual fan-in folded into the data gradient) equals the separate data
    gradient followed by "+=" bit for bit, on the kernels that add in their store and on the
    fallback alike."""
    rg = rng(23)
    p = (hw + 2 * pad - r) // stride + 1
    x, dy = randn(rg, n, c, hw, hw), randn(rg, n, k, p, p)
    w, base = randn(rg, k, c, r, r), randn(rg, n, c, hw, hw)
    xd, wd, dyd = singa.from_numpy(x, dev), singa.from_numpy(w, dev), singa.from_numpy(dy, dev)
    h = singa.CudnnConvHandle(xd, (r, r), (stride, stride), (pad, pad), c, k, False)
    want = singa.from_numpy(base, dev)
    want += singa.GpuConvBackwardx(dyd, wd, xd, h)
    acc = singa.from_numpy(base, dev)
    got = singa.GpuConvBackwardxAccumulate(dyd, wd, xd, h, acc)
    assert got is acc
    assert_bit_equal(got.to_numpy(), want.to_numpy(), "accumulating dgrad")


@pytest.mark.parametrize("n,c,hw,k,stride", [
    (40, 64, 56, 64, 1),     # 980 tiles: three whole rounds of tiles plus a shared remainder
    (16, 256, 14, 256, 1),   # fewer tiles than CUs: every tile is shared between workgroups
    (16, 64, 28, 128, 2),    # residue-class kernel, four partial classes per shared tile
])
def test_conv_dgrad_is_deterministic(singa, dev, n, c, hw, k, stride):
    """Tiles shared between workgroups are summed in a fixed order: repeated runs agree bit for bit,
    and one image of the batch agrees with the oracle."""
    r = rng(11)
    p = hw // stride
    x, dy = randn(r, n, c, hw, hw), randn(r, n, k, p, p)
    w = randn(r, k, c, 3, 3)
    xd, wd, dyd = singa.from_numpy(x, dev), singa.from_numpy(w, dev), singa.from_numpy(dy, dev)
    h = singa.CudnnConvHandle(xd, (3, 3), (stride, stride), (1, 1), c, k, False)
    a = singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy()
    for _ in range(3):
        assert_bit_equal(singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy(), a, "shared-tile summation order")
    dx_o, _ = O.conv_bwd(dy[-1:], x[-1:], w, (stride, stride), (1, 1), want_dw=False)
    assert nl2(a[-1:], dx_o) < TOL


@pytest.mark.parametrize("shape", [
    (64, 64, 56, 64, 3, 1, 1),     # the single-convolution benchmark configuration
    (64, 3, 224, 64, 7, 2, 3),     # ResNet stem: few-channel wgrad / direct dgrad kernels
    (64, 64, 56, 128, 3, 2, 1),    # stage transition: residue-class shared-tile dgrad, stride-2 slab wgrad
    (64, 256, 14, 512, 1, 2, 0),   # downsample: pointwise dgrad with dilating store
    (64, 64, 56, 128, 1, 2, 0),    # first downsample: 64 x 64 wavefront tiles
    (64, 128, 28, 128, 3, 1, 1),   # the 3x3 layers of stages 2-4 at the full batch: shared-tile kernels on 28 x 28,
    (64, 256, 14, 256, 3, 1, 1),   # 14 x 14 (tiles that straddle images, every tile shared between workgroups)
    (64, 512, 7, 512, 3, 1, 1),    # and 7 x 7 planes (49 pixels: a tile covers 2.6 images)
    (64, 128, 28, 256, 3, 2, 1),   # the stride-2 layers that open stages 3 and 4
    (64, 256, 14, 512, 3, 2, 1),
    (64, 128, 28, 256, 1, 2, 0),   # second downsample
])
def test_conv_full_size_properties(singa, dev, shape):
    """Convolutions at the benchmark's full batch are too large for the CPU oracle inside a test,
    so parity is checked through size-independent properties: adjointness
    <conv(x,W),dy> = <x,dgrad(dy,W)> = <W,wgrad(dy,x)>, linearity in dy, and the oracle on one image
    of the batch (dgrad is per-image; wgrad of a 2-image batch)."""
    r = rng(2024)
    N, C, H, K, R, st, pd = shape
    x = randn(r, N, C, H, H)
    w = (randn(r, K, C, R, R) * np.sqrt(2.0 / (C * R * R))).astype(np.float32)
    xd, wd = singa.from_numpy(x, dev), singa.from_numpy(w, dev)
    h = singa.CudnnConvHandle(xd, (R, R), (st, st), (pd, pd), C, K, True)
    P = h.conv_height
    dy = randn(r, N, K, P, P)
    dyd = singa.from_numpy(dy, dev)
    y = singa.GpuConvForward(xd, wd, None, h).to_numpy().astype(np.float64)
    dx = singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy()
    dw = singa.GpuConvBackwardW(dyd, xd, wd, h).to_numpy()
    db = singa.GpuConvBackwardb(dyd, singa.from_numpy(np.zeros(K, np.float32), dev), h).to_numpy()
    lhs = float((y * dy).sum())
    scale = float(np.sqrt((y * y).sum() * (dy.astype(np.float64) ** 2).sum()))  # |<y,dy>| can be small: bound by norms
    assert abs(lhs - float((x.astype(np.float64) * dx).sum())) < 1e-5 * scale
    assert abs(lhs - float((w.astype(np.float64) * dw).sum())) < 1e-5 * scale
    np.testing.assert_allclose(db, dy.astype(np.float64).sum(axis=(0, 2, 3)), rtol=1e-4, atol=1e-2)
    # oracle on image 5 (dgrad) and on a 2-image sub-batch (wgrad is additive over images)
    dx5, _ = O.conv_bwd(dy[5:6], x[5:6], w, (st, st), (pd, pd), want_dw=False)
    assert nl2(dx[5:6], dx5) < TOL
    dys = dy.copy()
    dys[2:] = 0
    dw2 = singa.GpuConvBackwardW(singa.from_numpy(dys, dev), xd, wd, h).to_numpy()
    _, dw2_o = O.conv_bwd(dy[:2], x[:2], w, (st, st), (pd, pd), want_dx=False)
    assert nl2(dw2, dw2_o) < TOL
    # linearity: dgrad(2*dy) == 2*dgrad(dy) exactly (scaling by a power of two)
    dx2 = singa.GpuConvBackwardx(singa.from_numpy(dy * 2, dev), wd, xd, h).to_numpy()
    assert_bit_equal(dx2, dx * 2, "dgrad linearity")


_TILE_ORDER_CHILD = r'''
import hashlib, sys, numpy as np
sys.path.insert(0, sys.argv[1])
from singa_amd import singa_wrap as singa
dev = singa.create_hip_gpu_on(0)
r = np.random.default_rng(99)
for (N, C, H, K, st) in [(64, 64, 56, 64, 1), (64, 128, 28, 128, 1), (64, 64, 56, 128, 2), (8, 512, 7, 512, 1)]:
    x = r.standard_normal((N, C, H, H)).astype(np.float32)
    w = r.standard_normal((K, C, 3, 3)).astype(np.float32)
    dy = r.standard_normal((N, K, H // st, H // st)).astype(np.float32)
    xd, wd, dyd = singa.from_numpy(x, dev), singa.from_numpy(w, dev), singa.from_numpy(dy, dev)
    h = singa.CudnnConvHandle(xd, (3, 3), (st, st), (1, 1), C, K, False)
    dx = singa.GpuConvBackwardx(dyd, wd, xd, h).to_numpy()
    dw = singa.GpuConvBackwardW(dyd, xd, wd, h).to_numpy()
    print(hashlib.sha256(dx.tobytes()).hexdigest(), hashlib.sha256(dw.tobytes()).hexdigest(), flush=True)
'''


def test_conv_tile_order_per_xcd_changes_no_bit(tmp_path):
    """The fp32 3x3 gradient kernels deal their tiles to workgroups per XCD (runs of eight neighbouring tiles in the
    data gradient, the tiles of one reduction split in the weight gradient); SGH_CONV_XCD_OFF deals them in launch
    order.  The switch is read once per process, so two child processes compute the same seeded gradients at full
    size (enough tiles for whole rounds of the chip, where the order differs) and their results agree bit for bit."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = tmp_path / "tile_order_child.py"
    script.write_text(_TILE_ORDER_CHILD)
    outs = []
    for off in (False, True):
        env = dict(os.environ)
        env.pop("SGH_CONV_XCD_OFF", None)
        if off:
            env["SGH_CONV_XCD_OFF"] = "1"
        outs.append(subprocess.check_output([sys.executable, str(script), root], env=env, timeout=300).decode().split())
    assert len(outs[0]) == 8 and outs[0] == outs[1]


def test_conv_argument_checks(singa, dev):
    x = singa.from_numpy(np.zeros((2, 3, 8, 8), np.float32), dev)
    with pytest.raises(singa.SingaHipError):
        singa.CudnnConvHandle(x, (3, 3), (1, 1), (1, 1), 4, 8, False)  # channel mismatch
    h = singa.CudnnConvHandle(x, (3, 3), (1, 1), (1, 1), 3, 8, False)
    w = singa.from_numpy(np.zeros((8, 3, 3, 3), np.float32), dev)
    with pytest.raises(singa.SingaHipError):
        singa.GpuConvBackwardx(singa.from_numpy(np.zeros((2, 8, 7, 7), np.float32), dev), w, x, h)


# ---------------------------------------------------------------------------------- pooling

POOL_CASES = [
    # N, C, H, W, kernel, stride, pad
    (2, 3, 8, 8, (2, 2), (2, 2), (0, 0)),
    (2, 4, 17, 17, (3, 3), (2, 2), (1, 1)),
    (4, 64, 112, 112, (3, 3), (2, 2), (1, 1)),   # ResNet stem max-pool geometry (reduced batch)
    (8, 32, 32, 32, (2, 2), (2, 2), (0, 0)),     # small-CNN pool 1
    (1, 2, 7, 5, (3, 2), (1, 2), (1, 0)),
    (2, 2, 6, 6, (2, 2), (3, 3), (0, 0)),        # stride > kernel: inputs outside every window
    (4, 512, 7, 7, (7, 7), (1, 1), (0, 0)),      # ResNet global pool geometry
    (1, 3, 5, 3, (5, 3), (1, 1), (0, 0)),        # global pool, planes of 15: vectors across planes and a scalar tail
    (3, 5, 12, 8, (3, 3), (2, 2), (1, 1)),       # window-column kernel: one partial wavefront strip
    (2, 3, 60, 16, (3, 3), (2, 2), (1, 1)),      # ... two bands (28 + 2 block rows)
    (1, 2, 6, 256, (3, 3), (2, 2), (1, 1)),      # ... 128 window columns: three column groups of 63
]


def test_pool_reference_vectors(singa, dev, golden):
    g = golden["pool_max"]
    x = np.array(g["x"], np.float32).reshape(g["x_shape"])
    dy = np.array(g["dy"], np.float32).reshape(g["dy_shape"])
    xd = singa.from_numpy(x, dev)
    h = singa.CudnnPoolingHandle(xd, g["kernel"], g["stride"], g["pad"], True)
    y = singa.GpuPoolingForward(h, xd)
    assert y.to_numpy().ravel().tolist() == g["y"]
    dx = singa.GpuPoolingBackward(h, singa.from_numpy(dy, dev), xd, y).to_numpy()
    assert_bit_equal(dx.ravel(), np.array(g["dx"], np.float32), "test_pooling.cc vector")
    g = golden["pool_api"]
    x = np.array(g["x"], np.float32).reshape(g["x_shape"])
    dy = np.array(g["dy"], np.float32).reshape(g["dy_shape"])
    xd, dyd = singa.from_numpy(x, dev), singa.from_numpy(dy, dev)
    for is_max, ky, kdx in ((True, "max_y", "max_dx"), (False, "avg_y", "avg_dx")):
        h = singa.CudnnPoolingHandle(xd, g["kernel"], g["stride"], g["pad"], is_max)
        y = singa.GpuPoolingForward(h, xd)
        assert_bit_equal(y.to_numpy().ravel(), np.array(g[ky], np.float32), ky)
        assert_bit_equal(singa.GpuPoolingBackward(h, dyd, xd, y).to_numpy().ravel(), np.array(g[kdx], np.float32), kdx)


@pytest.mark.parametrize("case", POOL_CASES)
@pytest.mark.parametrize("ties", [False, True])
def test_max_pool_bit_exact(singa, dev, case, ties):
    N, C, H, W, kernel, stride, pad = case
    r = rng(H * 31 + W)
    x = randn(r, N, C, H, W)
    if ties:
        x = np.round(x * 2).astype(np.float32)  # heavy ties: first maximum in row-major order wins
    y_o, mask = O.pool_max_fwd(x, kernel, stride, pad)
    dy = randn(r, *y_o.shape)
    xd = singa.from_numpy(x, dev)
    h = singa.CudnnPoolingHandle(xd, kernel, stride, pad, True)
    y = singa.GpuPoolingForward(h, xd)
    assert_bit_equal(y.to_numpy(), y_o, "max-pool forward")
    dx = singa.GpuPoolingBackward(h, singa.from_numpy(dy, dev), xd, y).to_numpy()
    assert_bit_equal(dx, O.pool_max_bwd(dy, mask, x.shape), "max-pool routing")


def test_max_pool_backward_keeps_the_sign_of_zero_sums(singa, dev):
    """A dx element that receives only -0.0 gradients is +0.0 on the CPU (its sum starts at +0.0)."""
    r = rng(5)
    x = randn(r, 2, 3, 16, 16)
    y_o, mask = O.pool_max_fwd(x, (3, 3), (2, 2), (1, 1))
    dy = np.where(r.random(y_o.shape) < 0.5, np.float32(-0.0), randn(r, *y_o.shape)).astype(np.float32)
    xd = singa.from_numpy(x, dev)
    h = singa.CudnnPoolingHandle(xd, (3, 3), (2, 2), (1, 1), True)
    y = singa.GpuPoolingForward(h, xd)
    dx = singa.GpuPoolingBackward(h, singa.from_numpy(dy, dev), xd, y).to_numpy()
    assert_bit_equal(dx, O.pool_max_bwd(dy, mask, x.shape), "max-pool routing with -0.0 gradients")


@pytest.mark.parametrize("case", POOL_CASES)
def test_avg_pool_bit_exact(singa, dev, case):
    N, C, H, W, kernel, stride, pad = case
    r = rng(H * 37 + W)
    x = randn(r, N, C, H, W)
    xd = singa.from_numpy(x, dev)
    h = singa.CudnnPoolingHandle(xd, kernel, stride, pad, False)
    y = singa.GpuPoolingForward(h, xd)
    y_o = O.pool_avg_fwd(x, kernel, stride, pad, include_pad=False)
    assert nl2(y.to_numpy(), y_o) < 1e-6  # forward sums the window in the same order; division is IEEE
    dy = randn(r, *y_o.shape)
    dx = singa.GpuPoolingBackward(h, singa.from_numpy(dy, dev), xd, y).to_numpy()
    assert_bit_equal(dx, O.pool_avg_bwd(dy, x.shape, kernel, stride, pad, include_pad=False), "avg-pool backward")


@pytest.mark.parametrize("case", [
    # N, C, H = W, bias: the stem's forward kernel (7 x 7, stride 2, padding 3, 64 filters) at its four widths
    (3, 3, 32, True), (2, 1, 64, False), (2, 2, 128, True), (1, 3, 224, False),
])
def test_stem_forward_fp32(singa, dev, case):
    """Forward convolution of the stem geometry against the CPU oracle (1e-3 normalised L2 as for every fp32
    convolution; asserted here: 1e-5), the border rows and columns on their own, and an infinity next to a
    window staying out of it."""
    N, C, H, bias = case
    r = rng(H + 7 * C)
    x = randn(r, N, C, H, H)
    w = (randn(r, 64, C, 7, 7) * np.sqrt(2.0 / (C * 49))).astype(np.float32)
    b = randn(r, 64) if bias else None
    xd, wd = singa.from_numpy(x, dev), singa.from_numpy(w, dev)
    bd = singa.from_numpy(b, dev) if bias else None
    h = singa.CudnnConvHandle(xd, (7, 7), (2, 2), (3, 3), C, 64, bias)
    y = singa.GpuConvForward(xd, wd, bd, h).to_numpy()
    want = O.conv_fwd(x, w, b, (2, 2), (3, 3))
    assert y.shape == want.shape == (N, 64, H // 2, H // 2)
    assert nl2(y, want) < 1e-5
    for sl in (np.s_[:, :, :2, :], np.s_[:, :, -2:, :], np.s_[:, :, :, :2], np.s_[:, :, :, -2:]):
        assert nl2(y[sl], want[sl]) < 1e-5
    # window (p, q) covers rows 2 p - 3 .. 2 p + 3 and columns 2 q - 3 .. 2 q + 3: an infinity at (9, 12) belongs to
    # the windows p = 3..6, q = 5..7 and to no other (column 12 is the one in front of window q = 8)
    x2 = x.copy()
    x2[0, 0, 9, 12] = np.inf
    y2 = singa.GpuConvForward(singa.from_numpy(x2, dev), wd, bd, h).to_numpy()
    hit = np.zeros(y2.shape, bool)
    hit[0, :, 3:7, 5:8] = True
    assert not np.isfinite(y2[hit]).any() and np.isfinite(y2[~hit]).all()


# ---------------------------------------------------------------------------------- batch norm

def test_bn_reference_vectors(singa, dev, golden):
    g = golden["bn_cudnn"]
    x = np.array(g["x"], np.float32).reshape(g["x_shape"])
    dy = np.array(g["dy"], np.float32).reshape(g["x_shape"])
    xd = singa.from_numpy(x, dev)
    h = singa.CudnnBatchNormHandle(0.9, xd)
    gamma, beta = singa.from_numpy(np.ones(2, np.float32), dev), singa.from_numpy(np.zeros(2, np.float32), dev)
    rm, rv = singa.from_numpy(np.zeros(2, np.float32), dev), singa.from_numpy(np.zeros(2, np.float32), dev)
    y, mean, var = singa.GpuBatchNormForwardTraining(h, xd, gamma, beta, rm, rv)
    np.testing.assert_allclose(y.to_numpy().ravel(), np.array(g["y"], np.float32), atol=g["tol"])
    dx, ds, db = singa.GpuBatchNormBackward(h, singa.from_numpy(dy, dev), xd, gamma, mean, var)
    np.testing.assert_allclose(dx.to_numpy().ravel(), np.array(g["dx"], np.float32), atol=g["tol"])
    np.testing.assert_allclose(ds.to_numpy(), np.array(g["dgamma"], np.float32), atol=g["tol"])
    np.testing.assert_allclose(db.to_numpy(), np.array(g["dbeta"], np.float32), atol=g["tol"])
    g = golden["bn_api"]
    x = np.array(g["x"], np.float32).reshape(g["x_shape"])
    xd = singa.from_numpy(x, dev)
    h = singa.CudnnBatchNormHandle(0.1, xd)
    gamma, beta = singa.from_numpy(np.ones(3, np.float32), dev), singa.from_numpy(np.zeros(3, np.float32), dev)
    y, mean, var = singa.GpuBatchNormForwardTraining(h, xd, gamma, beta, None, None)
    dx, _, _ = singa.GpuBatchNormBackward(h, xd, xd, gamma, mean, var)
    np.testing.assert_allclose(dx.to_numpy().ravel(), np.array(g["dx"], np.float32), atol=1e-6)


def test_bn_2d_reference_vectors(singa, dev, golden):
    """The reference's 2-D BatchNorm layer test (test/singa/test_batchnorm.cc:44-129) through the handle built from a
    [batch, features] tensor (CudnnBatchNormHandle's is_2d case, src/model/operation/batchnorm.cc:27-43)."""
    g = golden["bn_2d"]
    x = np.array(g["x"], np.float32).reshape(g["x_shape"])
    dy = np.array(g["dy"], np.float32).reshape(g["x_shape"])
    xd = singa.from_numpy(x, dev)
    h = singa.CudnnBatchNormHandle(1.0, xd)
    assert h.is_2d and (h.height, h.width) == (1, 1)
    mk = lambda v: singa.from_numpy(np.array(v, np.float32), dev)
    rm, rv = mk(g["fwd_beta"]), mk(g["fwd_beta"])        # (the test seeds the running statistics with beta)
    y, _, _ = singa.GpuBatchNormForwardTraining(h, xd, mk(g["fwd_gamma"]), mk(g["fwd_beta"]), rm, rv)
    assert y.shape() == g["x_shape"]
    np.testing.assert_allclose(y.to_numpy().ravel(), np.array(g["y"], np.float32), atol=g["tol"])
    gamma = mk(g["bwd_gamma"])
    _, mean, var = singa.GpuBatchNormForwardTraining(h, xd, gamma, mk(g["bwd_beta"]), None, None)
    dx, ds, db = singa.GpuBatchNormBackward(h, singa.from_numpy(dy, dev), xd, gamma, mean, var)
    assert dx.shape() == g["x_shape"] and ds.shape() == [2] and db.shape() == [2]
    np.testing.assert_allclose(dx.to_numpy().ravel(), np.array(g["dx"], np.float32), atol=g["tol"])
    np.testing.assert_allclose(ds.to_numpy(), np.array(g["dgamma"], np.float32), atol=g["tol"])
    np.testing.assert_allclose(db.to_numpy(), np.array(g["dbeta"], np.float32), atol=g["tol"])


@pytest.mark.parametrize("shape", [(4, 3, 5, 6), (2, 5, 7, 7), (8, 64, 56, 56), (64, 512, 7, 7), (16, 128, 28, 28),
                                   (2, 64, 112, 112), (32, 10),
                                   # a channel fits in LDS and there are >= 128 of them: the one-pass backward
                                   (8, 128, 14, 14), (16, 256, 7, 7), (4, 130, 5, 6), (64, 256, 14, 14), (3, 300, 1, 1),
                                   # planes that are not whole vectors, a channel in several slices
                                   (128, 8, 7, 7), (96, 16, 5, 5)])
def test_bn_vs_oracle(singa, dev, shape):
    r = rng(sum(shape))
    x = (randn(r, *shape) * 2 + 0.5).astype(np.float32)
    dy = randn(r, *shape)
    C = shape[1]
    gamma, beta = (randn(r, C) * 0.2 + 1).astype(np.float32), randn(r, C)
    rm, rv = randn(r, C), np.abs(randn(r, C))
    rm_o, rv_o = rm.copy(), rv.copy()
    y_o, mean_o, inv_o = O.bn_fwd_train(x, gamma, beta, rm_o, rv_o, factor=0.9)
    dx_o, dg_o, db_o = O.bn_bwd(dy, x, gamma, mean_o, inv_o)
    xd, gd, bd = singa.from_numpy(x, dev), singa.from_numpy(gamma, dev), singa.from_numpy(beta, dev)
    rmd, rvd = singa.from_numpy(rm, dev), singa.from_numpy(rv, dev)
    h = singa.CudnnBatchNormHandle(0.9, xd)
    y, mean, var = singa.GpuBatchNormForwardTraining(h, xd, gd, bd, rmd, rvd)
    assert nl2(y.to_numpy(), y_o) < TOL
    assert nl2(mean.to_numpy(), mean_o) < 1e-4 and nl2(var.to_numpy(), inv_o) < 1e-4
    assert nl2(rmd.to_numpy(), rm_o) < 1e-4 and nl2(rvd.to_numpy(), rv_o) < 1e-4
    # backward fed with the ORACLE's saved statistics, so only the backward kernel is under test
    dx, ds, db = singa.GpuBatchNormBackward(h, singa.from_numpy(dy, dev), xd, gd, singa.from_numpy(mean_o, dev),
                                            singa.from_numpy(inv_o, dev))
    e = (nl2(dx.to_numpy(), dx_o), nl2(ds.to_numpy(), dg_o), nl2(db.to_numpy(), db_o))
    print("bn bwd nl2 dx %.2e dgamma %.2e dbeta %.2e" % e)
    assert max(e) < TOL
    # run-to-run identical
    dx2, ds2, db2 = singa.GpuBatchNormBackward(h, singa.from_numpy(dy, dev), xd, gd, singa.from_numpy(mean_o, dev),
                                               singa.from_numpy(inv_o, dev))
    assert_bit_equal(dx2.to_numpy(), dx.to_numpy())
    assert_bit_equal(ds2.to_numpy(), ds.to_numpy())


def _random_bn_shapes(count, seed):
    """Seeded shapes aimed at the planning and indexing of the one-pass BatchNorm kernels: plane sizes that are
    and are not whole 16-byte vectors, fewer / more vectors per plane than a workgroup has threads (so that a
    thread's vectors step over several images, or several of them lie in one plane), channels in one slice and
    in many, channel counts below and above the number of CUs."""
    r = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < count:
        C = int(r.choice([1, 2, 3, 8, 24, 64, 130, 256, 300]))
        H = int(r.integers(1, 31))
        W = H if r.random() < 0.5 else int(r.integers(1, 31))
        N = int(r.integers(1, 49))
        if not 2000 <= N * C * H * W <= 4_000_000:
            continue
        shapes.append((N, C, H, W))
    return shapes


@pytest.mark.parametrize("shape", _random_bn_shapes(36, 20241125))
def test_bn_shape_sweep(singa, dev, shape):
    test_bn_vs_oracle(singa, dev, shape)


def _random_conv_cases(count, seed):
    """Seeded geometry sweep aimed at the planning logic of the specialised kernels: channel counts
    around the 32 / 64 / 128 tile edges, image sizes around the 16 / 32 / 64-column slab limits,
    strides 1-2, 1x1 / 3x3 / 5x5 / 7x7 filters, every legal padding."""
    r = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        R = int(r.choice([1, 3, 3, 3, 5, 7]))
        st = int(r.choice([1, 1, 2]))
        pd = int(r.integers(0, R // 2 + 2))
        C = int(r.choice([1, 3, 4, 16, 31, 32, 33, 48, 64, 65, 96, 128, 130]))
        K = int(r.choice([8, 16, 32, 48, 63, 64, 65, 96, 128, 144]))
        H = int(r.integers(max(R - 2 * pd, 1), 34)) if r.random() < 0.7 else int(r.choice([56, 58, 62, 63]))
        W = H if r.random() < 0.6 else int(r.integers(max(R - 2 * pd, 1), 40))
        if H + 2 * pd < R or W + 2 * pd < R:
            continue
        N = int(r.integers(1, 4))
        P, Q = (H + 2 * pd - R) // st + 1, (W + 2 * pd - R) // st + 1
        if N * K * P * Q * C * R * R > 4e8:   # keep the CPU oracle quick
            continue
        cases.append((N, C, H, W, K, R, R, (st, st), (pd, pd), bool(r.random() < 0.3)))
    return cases


@pytest.mark.parametrize("case", _random_conv_cases(48, 20240607))
def test_conv_geometry_sweep(singa, dev, case):
    test_conv_backward_vs_oracle(singa, dev, case)


def _shared_tile_cases(count, seed):
    """3x3 pad-1 geometries the shared-tile kernels accept (C >= 64, K a multiple of 16), over image
    sizes that move the slab pitch / rows-per-tile choices and make tiles straddle images."""
    r = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        st = int(r.choice([1, 1, 2]))
        C = int(r.choice([64, 68, 96, 128, 192, 256]))
        K = int(r.choice([64, 80, 96, 128, 160, 256]))
        H = int(r.integers(2, 32)) * (2 if st == 2 else 1)
        W = int(r.integers(2, 32)) * (2 if st == 2 else 1)
        if st == 1 and r.random() < 0.5:
            H, W = int(r.integers(2, 63)), int(r.integers(2, 63))
        N = int(r.integers(1, 6))
        P, Q = (H + 2 - 3) // st + 1, (W + 2 - 3) // st + 1
        if N * K * P * Q * C * 9 > 6e8:
            continue
        cases.append((N, C, H, W, K, 3, 3, (st, st), (1, 1), bool(r.random() < 0.3)))
    return cases


@pytest.mark.parametrize("case", _shared_tile_cases(40, 777))
def test_conv_shared_tile_sweep(singa, dev, case):
    test_conv_backward_vs_oracle(singa, dev, case)
