"""The whole-step drivers replayed on the CPU oracle alone (no GPU): the tape must reproduce the
NumPy restatement of an MLP training step that the reference's own integration test uses
(test/python/test_model.py:368-411), and the model graphs must have the reference's shapes."""
import numpy as np

from oracle.ops import OracleOps
from singa_amd import workloads as wl


def test_mlp_step_matches_reference_numpy_restatement():
    ops = OracleOps()
    net = wl.build("mlp", ops, lr=0.05, momentum=0.0)
    x, labels = wl.make_inputs("mlp", 16)
    W0, B0, W1, B1 = (np.array(p, np.float64) for _, p in net.params())
    net.forward(ops.from_numpy(x), ops.from_numpy(labels))
    net.backward_and_update(keep_grads=True)
    # test_model.py:370-411, in float64
    x1 = x @ W0 + B0
    x3 = np.maximum(x1, 0)
    out = x3 @ W1 + B1
    e = np.exp(out - out.max(axis=-1, keepdims=True))
    sm = e / e.sum(axis=-1, keepdims=True)
    onehot = np.eye(10)[labels]
    dloss = (sm - onehot) / sm.shape[0]
    db1 = dloss.sum(0)
    dx4 = dloss @ W1.T
    dw1 = x3.T @ dloss
    dx3 = dx4 * (x3 > 0)
    db0 = dx3.sum(0)
    dw0 = x.T.astype(np.float64) @ dx3
    exp = [W0 - 0.05 * dw0, B0 - 0.05 * db0, W1 - 0.05 * dw1, B1 - 0.05 * db1]
    for (name, p), e_ in zip(net.params(), exp):
        np.testing.assert_allclose(p, e_, rtol=2e-4, atol=2e-6, err_msg=name)


def test_resnet18_graph_shapes():
    ops = OracleOps()
    net = wl.build("resnet18_small", ops)
    names = [n for n, _ in net.params()]
    # 20 convolutions, 20 BatchNorms (scale + bias each), fc W + b = 62 parameter tensors
    assert len(names) == 62
    assert sum(1 for n in names if n.endswith(".W") and "fc" not in n) == 20
    shapes = {n: p.shape for n, p in net.params()}
    assert shapes["conv1.W"] == (64, 3, 7, 7)
    assert shapes["layer2.0.downsample.conv.W"] == (128, 64, 1, 1)
    assert shapes["layer4.1.conv2.W"] == (512, 512, 3, 3)
    f = wl.resnet18_flops(64)
    assert f["convs"] == 20
    assert abs(f["wgrad"] / 1e9 - 232.1) < 0.2  # algorithmic GFLOP of all wgrads at N=64
    full = wl.build("resnet18", ops)
    assert sum(p.size for _, p in full.params()) == 11689512  # torchvision's ResNet-18 parameter count


def test_small_resnet_step_runs_and_learns():
    ops = OracleOps()
    net = wl.build("resnet18_small", ops, lr=0.05, momentum=0.9)
    x, labels = wl.make_inputs("resnet18_small", 2)
    xs, ls = ops.from_numpy(x), ops.from_numpy(labels)
    l0 = float(np.mean(net.forward(xs, ls)))
    for _ in range(3):
        dxin = net.backward_and_update()
        l1 = float(np.mean(net.forward(xs, ls)))
    assert dxin.shape == x.shape          # the stem's dgrad is computed like SINGA does
    assert np.isfinite(l1) and l1 < l0    # three steps on one batch reduce its loss


def test_bf16_host_rounding():
    """float_to_bf16_bits is the reference rounding the GPU tests compare with: ties to even,
    carries into the exponent, infinities and NaN preserved."""
    from singa_amd.singa_wrap import bf16_bits_to_float, float_to_bf16_bits
    a = np.array([1.0, 1.00390625, 1.01171875, 3.4e38, -0.0, np.inf, -np.inf], np.float32)
    b = float_to_bf16_bits(a)
    assert list(b[:3]) == [0x3F80, 0x3F80, 0x3F82]          # tie -> even (down), tie -> even (up)
    assert b[3] == 0x7F80 and b[4] == 0x8000 and b[5] == 0x7F80 and b[6] == 0xFF80   # overflow rounds to inf
    assert np.isnan(bf16_bits_to_float(float_to_bf16_bits(np.array([np.nan], np.float32)))).all()
    x = np.random.default_rng(0).standard_normal(1000).astype(np.float32)
    y = bf16_bits_to_float(float_to_bf16_bits(x))
    assert np.abs(y - x).max() <= np.abs(x).max() * 2.0 ** -8
