"""GPU parity of whole backward+update steps (the benchmark configurations) against the CPU
oracle replaying the same tape on the same seeded inputs.

Metric: normalised L2 error per gradient / updated parameter tensor, bound 1e-3 (fp32 conv / BN
reductions).  The backward kernels are compared on the oracle's activations; the GPU's own
forward is compared separately (loss, logits)."""
import numpy as np
import pytest

from oracle.ops import OracleOps
from rounding_oracle import UNIT_ROUNDOFF, RoundingOracleOps, errors_against_truth, saved_inputs, store_fn
from singa_amd import workloads as wl
from torch_ref import TorchNet
from util import nl2

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _report(res, top=5):
    # loss / logits come from each side's OWN forward and own (already updated) parameters; the
    # backward kernels are judged on gradients and updated parameters
    bwd = {k: v for k, v in res["errors"].items() if ".grad." in k or ".param." in k}
    fwd = {k: v for k, v in res["errors"].items() if k not in bwd}
    worst = sorted(bwd.items(), key=lambda kv: -kv[1])[:top]
    print("worst:", ", ".join("%s=%.2e" % kv for kv in worst), "| forward:", ", ".join("%s=%.2e" % kv for kv in fwd.items()))
    assert max(fwd.values()) < 1e-2
    return worst[0][1]


@pytest.mark.parametrize("name,batch,steps", [("smoke_cnn", 4, 2), ("mlp", 128, 2), ("cnn", 128, 1),
                                              ("resnet18_small", 2, 2), ("resnet18", 2, 1)])
def test_backward_update_step(dev, name, batch, steps):
    res = wl.run_parity_case(name, dev, OracleOps(), batch=batch, steps=steps)
    assert len(res["errors"]) > 4
    assert _report(res) < TOL


def test_resnet18_own_forward_end_to_end(dev):
    """No shared activations: GPU forward + GPU backward vs the oracle's forward + backward.
    ReLU masks / max-pool winners may flip on near-ties, so the bound is looser (1e-2)."""
    res = wl.run_parity_case("resnet18_small", dev, OracleOps(), batch=2, share_activations=False)
    assert _report(res) < 1e-2


def test_fused_update_equals_per_parameter_update(dev):
    hip = wl.HipOps(dev)
    x, labels = wl.make_inputs("resnet18_small", 2)
    outs = []
    for fused in (False, True):
        net = wl.build("resnet18_small", hip)
        for _ in range(2):
            net.forward(hip.from_numpy(x), hip.from_numpy(labels))
            net.backward_and_update(fused_update=fused)
        outs.append([hip.to_numpy(p) for _, p in net.params()])
    for a, b in zip(*outs):
        assert np.array_equal(a, b)


def test_resnet18_full_batch_properties(dev):
    """ResNet-18 at the benchmark's full size (N=64, 224x224) is beyond the CPU oracle inside a
    test; parity at that size is checked through properties that do not depend on size:
    (1) images are independent in every layer but BatchNorm and the weight gradients, so the
        softmax-CE gradient and fc dgrad rows of image i depend only on image i;
    (2) the whole step is run-to-run deterministic (fixed-order split-K and BN reductions);
    (3) sum over classes of the logits gradient is 0 for every image."""
    hip = wl.HipOps(dev)
    x, labels = wl.make_inputs("resnet18", 64)
    runs = []
    for _ in range(2):
        net = wl.build("resnet18", hip)
        loss = net.forward(hip.from_numpy(x), hip.from_numpy(labels))
        net.backward_and_update(keep_grads=True)
        runs.append((hip.to_numpy(loss), {k: hip.to_numpy(v) for k, v in net.grad_log.items()},
                     [hip.to_numpy(p) for _, p in net.params()]))
    assert np.isfinite(runs[0][0]).all()
    for k in runs[0][1]:
        assert np.array_equal(runs[0][1][k], runs[1][1][k]), k
    for a, b in zip(runs[0][2], runs[1][2]):
        assert np.array_equal(a, b)
    g = runs[0][1]["logits"]
    assert g.shape == (64, 1000)
    assert np.abs(g.sum(axis=1)).max() < 1e-6
    assert runs[0][1]["input"].shape == (64, 3, 224, 224)
    assert all(np.isfinite(v).all() for v in runs[0][1].values())


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_resnet50_bottleneck_16bit_step(dev, kind):
    """The half-precision configuration on a narrow ResNet-50 (stages [3, 4, 6, 3], widths 16..128,
    64x64 images): 16-bit activations / gradients / convolution weights, fp32 BatchNorm statistics
    and parameters, fp32 master weights.

    Error model.  Truth is float64 arithmetic between the tape's rounding points (PyTorch autograd
    on an independently written graph, one rounding per stored 16-bit tensor; tests/torch_ref.py) on
    the same stored activations.  The GPU step and the fp32 CPU oracle that rounds at the same
    points are each measured against it, per gradient and updated parameter, in the normalised L2
    norm; the BatchNorm parameter gradients, sums of terms that largely cancel, are measured against
    the sum of |terms|.  Asserted:
      * the GPU's error is at most twice the oracle's plus one unit roundoff of the storage type
        (2^-11 / 2^-8): the kernels add nothing beyond what fp32 accumulation order does;
      * binary16: every tensor within the stated 1e-2;
      * bfloat16: within 5e-2 -- the oracle itself is 2e-2 from the truth on the first stage's
        weight gradients, last-place flips of stored bfloat16 gradients compounding over the 53
        layers behind them (test_tape_vs_torch.py); the 1e-2 bar is held per operation
        (test_gpu_half.py)."""
    from singa_amd import singa_wrap as singa
    dt = singa.kFloat16 if kind == "f16" else singa.kBFloat16
    name, lr, mu = "resnet50_small", 0.05, 0.9
    hip, orc = wl.HalfHipOps(dev, dt), RoundingOracleOps(kind)
    gpu, cpu = wl.build(name, hip, lr=lr, momentum=mu), wl.build(name, orc, lr=lr, momentum=mu)
    x, labels = wl.make_inputs(name, 4)
    p0 = {k: np.array(p) for k, p in cpu.params()}
    for k, p in gpu.params():
        assert np.array_equal(hip.to_numpy(p), p0[k]), k          # both start from the same stored weights
    losses = [np.asarray(n.ops.to_numpy(n.forward(n.ops.from_numpy(x), n.ops.from_numpy(labels)))) for n in (gpu, cpu)]
    # (each side's own 53-layer forward pass: not what this test judges -- the 16-bit forward ops are held
    # to 1e-2 one by one in test_gpu_half.py; here only a sanity bound, the numbers are printed)
    print(kind, "own forward: loss nl2 %.2e, logits nl2 %.2e" % (nl2(losses[0], losses[1]),
                                                                 nl2(hip.to_numpy(gpu.logits), cpu.logits)))
    assert nl2(losses[0], losses[1]) < 1e-1
    gpu.adopt_saved_tensors(cpu)
    truth = TorchNet(name, p0, lr, mu, store=store_fn(kind), adopt=saved_inputs(cpu))
    gpu.backward_and_update(keep_grads=True)
    cpu.backward_and_update(keep_grads=True)
    out = truth.step(orc.from_numpy(x), labels)
    e_gpu = errors_against_truth({k: hip.to_numpy(v) for k, v in gpu.grad_log.items()},
                                 {k: hip.to_numpy(p) for k, p in gpu.params()}, out, truth.bn_abs, lr)
    e_cpu = errors_against_truth(cpu.grad_log, dict(cpu.params()), out, truth.bn_abs, lr)
    assert set(e_gpu) == set(e_cpu) and len(e_gpu) > 300
    u = UNIT_ROUNDOFF[kind]
    ratio = sorted(((e_gpu[k] / (2 * e_cpu[k] + u), k) for k in e_gpu), reverse=True)
    worst = sorted(e_gpu.items(), key=lambda kv: -kv[1])[:4]
    print(kind, "GPU vs float64 model, worst:", ", ".join("%s=%.2e (oracle %.2e)" % (k, v, e_cpu[k]) for k, v in worst))
    print(kind, "largest GPU error / (2 x oracle error + u):", ", ".join("%s=%.2f" % (k, r) for r, k in ratio[:4]))
    assert ratio[0][0] <= 1.0, ratio[:4]
    # the stated bar, tensor by tensor: 1e-2 for every gradient and updated parameter.  In bfloat16 (unit roundoff
    # 2^-8) the fp32 oracle itself, rounding at the same points, does not hold it on some tensors -- last-place
    # flips of stored gradients that compound over the layers behind them -- so a tensor may exceed 1e-2 only where
    # the oracle's own distance from the float64 model is at least half the bar, and then stays within
    # 2 x oracle + u (above) and 5e-2.  The set is printed and counted.
    over = sorted(k for k, v in e_gpu.items() if v >= 1e-2)
    print(kind, "%d of %d tensors above 1e-2: %s" % (len(over), len(e_gpu), ", ".join("%s=%.2e (oracle %.2e)" % (k, e_gpu[k], e_cpu[k]) for k in over)))
    if kind == "f16":
        assert not over, over
    else:
        assert all(e_cpu[k] >= 5e-3 for k in over), [(k, e_gpu[k], e_cpu[k]) for k in over if e_cpu[k] < 5e-3]
        assert all(e_gpu[k] < 5e-2 for k in over)
        assert len(over) <= len(e_gpu) // 4, len(over)


@pytest.mark.parametrize("config,kind", [("resnet18_small", "f32"), ("resnet18_small", "f32-sum-in-relu"),
                                         ("resnet50_small", "f16"), ("resnet50_small", "bf16")])
def test_fused_tape_equals_reference_tape(dev, config, kind):
    """The tape with its cross-op fusions on -- ReLU backward folded into BatchNorm backward; the
    residual "+=" folded into the data gradient (fp32) or into the ReLU backward that reads the sum
    (16-bit storage) -- leaves bit-identical parameters and input gradient to the tape that makes
    one call per reference op.  (On 16-bit tensors with every kernel on one stream: a 16-bit weight gradient
    on the auxiliary stream plans its split reduction for the shared chip, i.e. sums in another order; that
    pair of tapes is compared in test_two_stream_tape_at_full_size.)"""
    from singa_amd import singa_wrap as singa
    x, labels = wl.make_inputs(config, 2)
    outs = []
    for fuse in (False, True):
        if kind.startswith("f32"):
            hip = wl.HipOps(dev)
            if kind == "f32-sum-in-relu":   # the 16-bit tape's choice of fusions on the fp32 ops
                hip.fusions = wl.HalfHipOps.fusions
        else:
            hip = wl.HalfHipOps(dev, singa.kFloat16 if kind == "f16" else singa.kBFloat16)
        hip.set_fusion(fuse)
        assert hip.fuse_bn_relu == fuse and (hip.fuse_dgrad_add or hip.fuse_add_relu) == fuse
        net = wl.build(config, hip)
        assert hip.overlap_wgrad == fuse and hip.batch_relayout == fuse
        if not kind.startswith("f32"):
            hip.overlap_wgrad = False
        for _ in range(2):
            net.forward(hip.from_numpy(x), hip.from_numpy(labels))
            # the fused tape also updates all parameters in one launch at the end, which lets it run
            # the weight gradients on the auxiliary stream
            dx = net.backward_and_update(fused_update=fuse)
        outs.append([hip.to_numpy(dx)] + [hip.to_numpy(p) for _, p in net.params()])
    for a, b in zip(*outs):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("config,batch,kind", [("resnet18", 64, "f32"), ("resnet50", 32, "f16")])
def test_two_stream_tape_at_full_size(dev, config, batch, kind):
    """The weight gradients on the auxiliary stream at the benchmark's layer sizes, where the two
    chains really run side by side for milliseconds: three steps leave bit-identical parameters and
    input gradient to the same tape with every kernel on one stream.  On 16-bit tensors a weight gradient
    on the auxiliary stream splits its reduction for the shared chip (fewer, longer splits: another summation
    order before the one rounding), so the one-stream tape is told to use that plan as well
    (sgh_conv_wgrad16_split_mode); with each tape on its own plan the first step's input gradient (which
    depends on no weight gradient) is still bit-identical and the parameters after one step agree to the
    last place (normalised L2 below 1e-3).  Later steps are no measure across plans: through fifty layers at
    random initialisation a perturbation of one unit in the last place of a few weights decorrelates the
    gradients within two steps."""
    from singa_amd import _lib
    from util import nl2
    from singa_amd import singa_wrap as singa
    x, labels = wl.make_inputs(config, batch)
    outs = []
    def run(overlap, steps, split_mode):
        _lib.lib().sgh_conv_wgrad16_split_mode(split_mode)
        try:
            hip = wl.HipOps(dev) if kind == "f32" else wl.HalfHipOps(dev, singa.kFloat16)
            hip.overlap_wgrad = overlap
            net = wl.build(config, hip, lr=0.01)
            for _ in range(steps):
                net.forward(hip.from_numpy(x), hip.from_numpy(labels))
                dx = net.backward_and_update(fused_update=True)
            return [hip.to_numpy(dx)] + [hip.to_numpy(p) for _, p in net.params()]
        finally:
            _lib.lib().sgh_conv_wgrad16_split_mode(-1)
    outs = [run(False, 3, 1), run(True, 3, -1)]
    for a, b in zip(*outs):
        assert np.array_equal(a, b)
    assert all(np.isfinite(a).all() for a in outs[0])     # the input gradient included
    if kind != "f32":   # each tape on its own plan, one step
        one, two = run(False, 1, -1), run(True, 1, -1)
        assert np.array_equal(one[0], two[0])
        worst = max(nl2(a, b) for a, b in zip(one[1:], two[1:]))
        print("parameters after one step, full-chip against shared-chip split plan: nl2 <= %.2e" % worst)
        assert worst < 1e-3


def test_resnet50_half_precision_tape_at_full_batch(dev):
    """The half-precision configuration at its own size (ResNet-50, N = 128, binary16 storage) as one whole tape --
    beyond the CPU oracle inside a test, so through what does not depend on size: every gradient and parameter
    finite; the logits gradient of every image sums to 0 over the classes (softmax-CE) and its rows are those of
    (p - onehot) / N computed from the tape's own probabilities; the step is run-to-run identical; and the input
    gradient of the first step, which depends on no weight gradient, is bit-equal between the one-stream and the
    two-stream tape."""
    from singa_amd import singa_wrap as singa
    x, labels = wl.make_inputs("resnet50", 128)

    def run(overlap):
        hip = wl.HalfHipOps(dev, singa.kFloat16)
        hip.overlap_wgrad = overlap
        net = wl.build("resnet50", hip, lr=0.01)
        net.forward(hip.from_numpy(x), hip.from_numpy(labels))
        p = hip.to_numpy(net.p).astype(np.float64)
        dx = net.backward_and_update(keep_grads=True, fused_update=True)
        grads = {k: np.asarray(hip.to_numpy(v), np.float32) for k, v in net.grad_log.items()}
        return hip.to_numpy(dx), grads, [np.asarray(hip.to_numpy(q), np.float32) for _, q in net.params()], p

    dx_a, grads_a, params_a, p = run(True)
    assert dx_a.shape == (128, 3, 224, 224) and len(grads_a) > 160
    assert np.isfinite(np.asarray(dx_a, np.float32)).all()
    assert all(np.isfinite(v).all() for v in grads_a.values()) and all(np.isfinite(v).all() for v in params_a)
    g = grads_a["logits"].astype(np.float64)
    assert g.shape == (128, 1000) and np.abs(g.sum(axis=1)).max() < 1e-6
    want = p.copy()
    want[np.arange(128), labels] -= 1.0
    assert nl2(g, want / 128) < 1e-6
    dx_b, grads_b, params_b, _ = run(True)                      # run to run
    assert np.array_equal(dx_a, dx_b)
    assert all(np.array_equal(grads_a[k], grads_b[k]) for k in grads_a)
    assert all(np.array_equal(a, b) for a, b in zip(params_a, params_b))
    dx_c, grads_c, _, _ = run(False)                            # every kernel on one stream
    assert np.array_equal(dx_a, dx_c)
    # (the 16-bit weight gradients plan their split reduction by the stream they run on: last-place differences)
    worst = max(nl2(grads_a[k], grads_c[k]) for k in grads_a)
    print("gradients, two-stream against one-stream tape: nl2 <= %.2e" % worst)
    assert worst < 1e-2


@pytest.mark.parametrize("two_streams", [False, True])
def test_graph_replay_of_the_step(dev, two_streams):
    """Graph mode (EnableGraph / RunGraph): one recorded backward+update step, replayed several
    times with eager work and synchronisations in between, leaves after every replay exactly the
    parameters of a network that ran the same number of eager steps.  `two_streams`: the recording holds
    the weight gradients as a branch on the auxiliary stream (fork / join while recording), in groups of
    three layers; the eager steps it is compared with fork once per layer."""
    hip = wl.HipOps(dev)
    hip.graph_overlap, hip.graph_wgrad_group = two_streams, 3
    x, labels = wl.make_inputs("resnet18_small", 2)
    nets = []
    for _ in range(2):
        net = wl.build("resnet18_small", hip, lr=0.002)
        net.forward(hip.from_numpy(x), hip.from_numpy(labels))
        nets.append(net)
    eager, replayed = nets
    for _ in range(2):   # momentum buffers, kernel attributes and the pool are set up by eager steps
        eager.backward_and_update(fused_update=True)
        replayed.backward_and_update(fused_update=True)
    dev.Sync()
    before = [hip.to_numpy(p) for _, p in replayed.params()]
    dev.EnableGraph(True)
    assert dev.graph_enabled()
    replayed.backward_and_update(fused_update=True)
    dev.EnableGraph(False)
    for a, (_, p) in zip(before, replayed.params()):
        assert np.isfinite(a).all() and np.array_equal(a, hip.to_numpy(p)), "recording must not execute"
    for i in range(4):
        eager.backward_and_update(fused_update=True)
        dev.RunGraph()
        t = hip.from_numpy(np.full(100000, i, np.float32))   # eager work on the same stream and pool
        t += t
        assert np.array_equal(hip.to_numpy(t), np.full(100000, 2 * i, np.float32))
        for (k, a), (_, b) in zip(eager.params(), replayed.params()):
            assert np.array_equal(hip.to_numpy(a), hip.to_numpy(b)), (i, k)
    dev.ResetGraph()
    eager.backward_and_update(fused_update=True)   # the device is back in eager mode
    replayed.backward_and_update(fused_update=True)
    for (k, a), (_, b) in zip(eager.params(), replayed.params()):
        assert np.array_equal(hip.to_numpy(a), hip.to_numpy(b)), k


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_mixed_precision_fused_update_equals_per_parameter_update(dev, kind):
    """One launch over all parameters of the mixed-precision network (fp32 BatchNorm / classifier
    parameters, 16-bit convolution weights with fp32 masters) leaves bit-identical parameters and
    masters to the per-parameter updates."""
    from singa_amd import singa_wrap as singa
    dt = singa.kFloat16 if kind == "f16" else singa.kBFloat16
    x, labels = wl.make_inputs("resnet50_small", 4)
    outs = []
    for fused in (False, True):
        hip = wl.HalfHipOps(dev, dt)
        net = wl.build("resnet50_small", hip, lr=0.01)
        for _ in range(2):
            net.forward(hip.from_numpy(x), hip.from_numpy(labels))
            net.backward_and_update(fused_update=fused)
        outs.append([hip.to_numpy(p) for _, p in net.params()] +
                    [net.sgd.masters[k].to_numpy() for k in sorted(net.sgd.masters)])
        assert len(net.sgd.masters) == 53
    for a, b in zip(*outs):
        assert np.array_equal(a, b)
