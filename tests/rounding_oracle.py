"""The fp32 CPU oracle as a model of 16-bit storage, and the float64 truth it is judged against.

``RoundingOracleOps``: fp32 arithmetic (the oracle's), with every 4-D array -- inputs, convolution
weights, activations, activation and weight gradients -- rounded to the storage type once, where
the GPU tape stores it; the gradient that re-enters the 16-bit part of the network behind the fp32
classifier head is rounded too.

``store_fn(kind)``: the same rounding for tests/torch_ref.TorchNet, which computes in float64
between the same rounding points.  An implementation's error is its distance from that model; the
oracle's own distance from it says how much of that is inherent to fp32 accumulation order and the
last-place flips it causes in the stored 16-bit values (which later layers amplify)."""
import numpy as np

from oracle.ops import OracleOps

# unit roundoff of the storage types (half a unit in the last place, relative)
UNIT_ROUNDOFF = {"f16": 2.0 ** -11, "bf16": 2.0 ** -8}


def round_to(kind, a):
    from singa_amd import singa_wrap as singa
    a = np.asarray(a, np.float32)
    if kind == "f16":
        with np.errstate(over="ignore"):
            return a.astype(np.float16).astype(np.float32)
    return singa.bf16_bits_to_float(singa.float_to_bf16_bits(a)).reshape(a.shape)


def store_fn(kind):
    import torch
    dt = torch.float16 if kind == "f16" else torch.bfloat16
    return lambda t: t.to(dt).to(torch.float64)


class RoundingOracleOps(OracleOps):
    ROUNDED = ("from_numpy", "conv_fwd", "bn_fwd_train", "pool_fwd", "relu", "add", "relu_bwd", "pool_bwd", "bn_bwd",
               "conv_bwd_x", "conv_bwd_w", "accumulate")

    def __init__(self, kind):
        self.kind = kind

    def _round(self, a):
        if isinstance(a, (tuple, list)):
            return type(a)(self._round(v) for v in a)
        if not isinstance(a, np.ndarray) or a.ndim != 4 or a.dtype.kind != "f":
            return a
        return round_to(self.kind, a)

    # precision boundary in front of the classifier head (workloads.Cast)
    def to_compute(self, x):
        return x

    def to_storage(self, x):
        return round_to(self.kind, x)

    def __getattribute__(self, name):
        attr = OracleOps.__getattribute__(self, name)
        if name in RoundingOracleOps.ROUNDED:
            return lambda *args, **kw: self._round(attr(*args, **kw))
        return attr


def saved_inputs(net):
    """{leaf layer name: the input the layer's backward will read}, as NumPy arrays."""
    from singa_amd import workloads as wl
    return {l.name: np.array(net.ops.to_numpy(l.x), copy=True) for l in net.leaf_layers()
            if hasattr(l, "x") and not isinstance(l, wl.Flatten)}


def errors_against_truth(grads, params, truth_out, bn_abs, lr):
    """Per-tensor normalised L2 distance from the float64 model: ||a - t|| / ||t||, except for the
    BatchNorm parameter gradients -- sums over a channel of terms that largely cancel -- whose
    error is measured against the size of what was summed, ||a - t|| / ||sum |terms| ||; the updated
    BatchNorm parameters (old value - lr * that sum) likewise against max(||t||, lr * ||sum |terms| ||)."""
    out = {}
    for k, g in grads.items():
        t = truth_out["grad." + k]
        d = np.linalg.norm(np.asarray(g, np.float64).ravel() - t.ravel())
        n = np.linalg.norm(bn_abs[k]) if k in bn_abs else np.linalg.norm(t)
        out["grad." + k] = float(d / (n if n > 0 else 1.0))
    for k, p in params.items():
        t = truth_out["param." + k]
        n = max(np.linalg.norm(t), lr * np.linalg.norm(bn_abs[k])) if k in bn_abs else np.linalg.norm(t)
        out["param." + k] = float(np.linalg.norm(np.asarray(p, np.float64).ravel() - t.ravel()) / (n if n > 0 else 1.0))
    return out
