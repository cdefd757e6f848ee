"""An independent restatement of the benchmark networks on PyTorch CPU autograd in float64, used
by the tests to pin the hand-written backward tapes of ``singa_amd/workloads.py``.

Nothing here shares code with the tape: the graphs are written from the reference's model files
(examples/cnn/model/resnet.py:27-185, the small CNN of the benchmark description), the backward
pass is torch's autograd, the update is the momentum rule of python/singa/opt.py:269-310 written
out by hand.  A wiring mistake in the tape (a dropped branch, a residual added twice, the wrong
tensor handed to a BatchNorm) therefore shows up as a difference against this model.

Two optional hooks make the same model serve as the float64 "truth" of the 16-bit tapes:

* ``store``: the rounding a tensor undergoes where the tape stores it in 16 bits (applied to the
  forward value and to the gradient of every stored 4-D tensor, and to weight gradients);
* ``adopt``: {leaf layer name: input array} -- the forward value at a layer's input is replaced by
  the given array (another implementation's stored activation), so that ReLU masks, max-pool
  winners and BatchNorm statistics are taken from identical inputs and only the backward
  arithmetic differs.  The value the model itself computed is kept in ``self.fwd_seen`` so the
  forward pass can be compared as well.
"""
import numpy as np
import torch
import torch.nn.functional as F


class _Point(torch.autograd.Function):
    """Forward: `value` (already a tensor) stands in for x; backward: the gradient as stored."""

    @staticmethod
    def forward(ctx, x, value, rnd):
        ctx.rnd = rnd
        return value.clone() if value is not None else x.clone()

    @staticmethod
    def backward(ctx, g):
        return (ctx.rnd(g) if ctx.rnd is not None else g), None, None


GRAPHS = {
    # name: (kind, options)
    "smoke_cnn": ("cnn", {}),
    "cnn": ("cnn", {}),
    "resnet18_small": ("resnet", {"block": "basic", "blocks": (2, 2, 2, 2), "final_pool": 2}),
    "resnet18": ("resnet", {"block": "basic", "blocks": (2, 2, 2, 2), "final_pool": 7}),
    "resnet50_small": ("resnet", {"block": "bottleneck", "blocks": (3, 4, 6, 3), "final_pool": 2}),
    "resnet50": ("resnet", {"block": "bottleneck", "blocks": (3, 4, 6, 3), "final_pool": 7}),
}


class TorchNet(object):
    def __init__(self, graph, params, lr, momentum, store=None, adopt=None, eps=1e-5):
        """`params`: {name: ndarray} with the tape's parameter names ("layer1.0.conv1.W", "bn1.scale", ...)."""
        self.kind, self.opt = GRAPHS[graph]
        self.p = {k: torch.tensor(np.asarray(v, np.float64), dtype=torch.float64, requires_grad=True)
                  for k, v in params.items()}
        self.lr, self.mu, self.eps = float(lr), float(momentum), eps
        self.store = store                 # tensor -> tensor rounding, or None
        self.adopt = adopt or {}
        self.moments = {}
        self.fwd_seen = {}
        self.bn_in = {}                    # BatchNorm name -> (input, output) tensors, for sum-of-|terms| norms

    # ---- stored-tensor points
    def _rnd(self, t):
        return self.store(t) if (self.store is not None and t.dim() == 4) else t

    def _at(self, name, x):
        """The input of leaf layer `name`: what the tape keeps in memory for it."""
        rnd = self._rnd if self.store is not None else None
        value = None
        if name in self.adopt:
            self.fwd_seen[name] = x.detach().numpy().copy()
            value = torch.tensor(np.asarray(self.adopt[name], np.float64).reshape(tuple(x.shape)))
        elif rnd is not None:
            value = rnd(x.detach())
        return _Point.apply(x, value, rnd)

    def _w(self, name):
        """A convolution weight: its gradient is stored like the weight."""
        w = self.p[name]
        return _Point.apply(w, None, self.store) if (self.store is not None and w.dim() == 4) else w

    # ---- leaf layers
    def conv(self, name, x, stride, pad):
        x = self._at(name, x)
        b = self.p.get(name + ".b")
        return F.conv2d(x, self._w(name + ".W"), b, stride=stride, padding=pad)

    def bn(self, name, x):
        x = self._at(name, x)
        y = F.batch_norm(x, None, None, self.p[name + ".scale"], self.p[name + ".bias"], training=True, eps=self.eps)
        y.retain_grad()
        self.bn_in[name] = (x, y)
        return y

    def relu(self, name, x):
        return F.relu(self._at(name, x))

    def maxpool(self, name, x, k, s, p):
        return F.max_pool2d(self._at(name, x), k, s, p)

    def avgpool(self, name, x, k):
        return F.avg_pool2d(self._at(name, x), k, 1, 0, count_include_pad=False)

    def linear(self, name, x):
        x = self._at(name, x)
        return x @ self.p[name + ".W"] + self.p[name + ".b"]

    # ---- graphs
    def _cnn(self, x):
        x = self.maxpool("pool1", self.relu("relu1", self.conv("conv1", x, 1, 2)), 2, 2, 0)
        x = self.maxpool("pool2", self.relu("relu2", self.conv("conv2", x, 1, 2)), 2, 2, 0)
        return self.linear("linear", x.flatten(1))

    def _entry(self, name, x):
        # the gradient of a block's input is one stored tensor: the sum of what the branches send back
        return _Point.apply(x, None, self._rnd) if self.store is not None else x

    def _basic(self, name, x, stride):
        x = self._entry(name, x)
        out = self.relu(name + ".relu1", self.bn(name + ".bn1", self.conv(name + ".conv1", x, stride, 1)))
        out = self.bn(name + ".bn2", self.conv(name + ".conv2", out, 1, 1))
        res = x
        if name + ".downsample.conv.W" in self.p:
            res = self.bn(name + ".downsample.bn", self.conv(name + ".downsample.conv", x, stride, 0))
        return self.relu(name + ".relu2", out + res)

    def _bottleneck(self, name, x, stride):
        x = self._entry(name, x)
        out = self.relu(name + ".relu1", self.bn(name + ".bn1", self.conv(name + ".conv1", x, 1, 0)))
        out = self.relu(name + ".relu2", self.bn(name + ".bn2", self.conv(name + ".conv2", out, stride, 1)))
        out = self.bn(name + ".bn3", self.conv(name + ".conv3", out, 1, 0))
        res = x
        if name + ".downsample.conv.W" in self.p:
            res = self.bn(name + ".downsample.bn", self.conv(name + ".downsample.conv", x, stride, 0))
        return self.relu(name + ".relu3", out + res)

    def _resnet(self, x):
        o = self.opt
        x = self.relu("relu", self.bn("bn1", self.conv("conv1", x, 2, 3)))
        x = self.maxpool("maxpool", x, 3, 2, 1)
        block = self._basic if o["block"] == "basic" else self._bottleneck
        for si, nb in enumerate(o["blocks"]):
            for bi in range(nb):
                x = block("layer%d.%d" % (si + 1, bi), x, 2 if (si > 0 and bi == 0) else 1)
        x = self.avgpool("avgpool", x, o["final_pool"]).flatten(1)
        if self.store is not None:   # the classifier head works in fp32; its input gradient is stored in 16 bits
            x = _Point.apply(x, None, self.store)
        return self.linear("fc", x)

    # ---- one training step
    def step(self, x, labels):
        """Forward, backward, update.  Returns {"loss", "logits", "grad.<name>", "param.<name>"} as
        float64 arrays; "grad.input" and "grad.logits" are the gradients of the mean loss."""
        for v in self.p.values():
            v.grad = None
        self.fwd_seen, self.bn_in = {}, {}
        xin = torch.tensor(np.asarray(x, np.float64), requires_grad=True)
        logits = (self._cnn if self.kind == "cnn" else self._resnet)(xin)
        logits.retain_grad()
        loss = F.cross_entropy(logits, torch.tensor(np.asarray(labels, np.int64)), reduction="mean")
        loss.backward()
        out = {"loss": float(loss.detach()), "logits": logits.detach().numpy().copy(),
               "grad.logits": logits.grad.numpy().copy(), "grad.input": xin.grad.numpy().copy()}
        # sums of |terms| of the two BatchNorm parameter-gradient sums (per channel), for normalising
        # errors of those heavily cancelling sums
        self.bn_abs = {}
        for name, (bx, by) in self.bn_in.items():
            dy = by.grad
            dims = [0] + list(range(2, bx.dim()))
            mean = bx.detach().mean(dim=dims, keepdim=True)
            var = bx.detach().var(dim=dims, unbiased=False, keepdim=True)
            xhat = (bx.detach() - mean) / torch.sqrt(var + self.eps)
            self.bn_abs[name + ".bias"] = dy.abs().sum(dim=dims).numpy().copy()
            self.bn_abs[name + ".scale"] = (dy * xhat).abs().sum(dim=dims).numpy().copy()
        with torch.no_grad():
            for k, p in self.p.items():
                g = p.grad
                out["grad." + k] = g.numpy().copy()
                # python/singa/opt.py:269-310 with dampening 0, no weight decay, no nesterov
                if self.mu != 0:
                    if k not in self.moments:
                        self.moments[k] = torch.zeros_like(p)
                    buf = self.moments[k]
                    buf.mul_(self.mu).add_(g)
                    g = buf
                p.add_(g, alpha=-self.lr)
                out["param." + k] = p.detach().numpy().copy()
        return out
