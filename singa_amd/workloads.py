"""Whole-step drivers for the benchmark configurations: forward once (to create the activations),
then the backward pass + SGD-momentum update in the order SINGA's tape would run it.

The drivers are written against a small "ops" interface so that the very same driver replays a
configuration on the GPU (``HipOps`` below, the product path) or on any other implementation of
the interface that a caller passes in (the test-suite passes its CPU oracle).  This module
itself never imports a CPU implementation.

Backward order follows ``autograd.backward`` (python/singa/autograd.py:128-224): the ready list
is a stack, so in a residual block the downsample branch is back-propagated before the main
branch, gradients that fan in are accumulated with ``+=`` (:204), and a parameter is updated as
soon as its gradient is complete (``Optimizer.call``, python/singa/opt.py:107-111).

Model graphs: ``examples/mlp/model.py`` (MLP), ``examples/cnn/model/resnet.py`` (ResNet,
BasicBlock :46-78, stem/_make_layer/forward :121-185), and the small CNN of the benchmark
description (conv5x5-32 p2, ReLU, maxpool2, conv5x5-64 p2, ReLU, maxpool2, Linear 4096->10).
"""
import numpy as np

from . import opt as hip_opt
from . import rng
from . import singa_wrap as singa


# ------------------------------------------------------------------------------------ ops (GPU)

class HipOps(object):
    """The ops interface bound to the gfx950 library (through singa_wrap's reference names)."""

    name = "hip"

    def __init__(self, dev):
        self.dev = dev

    def from_numpy(self, a):
        return singa.from_numpy(a, self.dev)

    def to_numpy(self, t):
        return t.to_numpy()

    def reshape(self, t, shape):
        return t.Reshape(shape)

    def shape(self, t):
        return tuple(t.shape())

    def sync(self):
        self.dev.Sync()

    # handles
    def conv_handle(self, x, kernel, stride, pad, cin, cout, bias):
        return singa.CudnnConvHandle(x, kernel, stride, pad, cin, cout, bias)

    def bn_handle(self, momentum, x):
        return singa.CudnnBatchNormHandle(momentum, x)

    def pool_handle(self, x, kernel, stride, pad, is_max):
        return singa.CudnnPoolingHandle(x, kernel, stride, pad, is_max)

    # forward
    def conv_fwd(self, x, W, b, h):
        return singa.GpuConvForward(x, W, b, h)

    def bn_fwd_train(self, h, x, g, b, rm, rv):
        return singa.GpuBatchNormForwardTraining(h, x, g, b, rm, rv)

    # cross-op fusion of the forward pass: the ReLU behind a BatchNorm, or behind the sum that ends a residual
    # block, applied by the kernel that produces its input (the same bits, one tensor pass less each)
    fuse_forward = True

    def bn_relu_fwd_train(self, h, x, g, b, rm, rv):
        return singa.GpuBatchNormReLUForwardTraining(h, x, g, b, rm, rv)

    def add_relu(self, a, b):
        return singa.AddReLU(a, b)

    def bn_add_relu_fwd_train(self, h, x, z, g, b, rm, rv):
        return singa.GpuBatchNormAddReLUForwardTraining(h, x, z, g, b, rm, rv)

    def pool_fwd(self, h, x):
        return singa.GpuPoolingForward(h, x)

    def relu(self, x):
        return singa.ReLU(x)

    def matmul(self, x, W):
        return singa.Mult(x, W)

    def add_bias(self, x, b):
        singa.AddRow(b, x)
        return x

    def add(self, a, b):
        return singa.__add__(a, b)

    def softmax(self, x):
        return singa.SoftMax(x)

    def ce_fwd(self, p, t):
        return singa.CrossEntropyFwd(p, t)

    # backward
    def softmax_ce_bwd(self, p, t, batch):
        # SoftmaxCrossEntropyBwd followed by "dx /= N" (python/singa/autograd.py:1319-1322), fused
        return singa.SoftmaxCrossEntropyBwd(p, t, scale=float(np.float32(1.0) / np.float32(batch)))

    def matmul_bwd(self, dy, x, W):
        return (singa.Mult(dy, singa.DefaultTranspose(W)), singa.Mult(singa.DefaultTranspose(x), dy))

    def sum0(self, dy):
        return singa.Sum(dy, 0)

    def relu_bwd(self, dy, x):
        return singa.ReLUBackward(dy, x)

    def pool_bwd(self, h, dy, x, y):
        return singa.GpuPoolingBackward(h, dy, x, y)

    def bn_bwd(self, h, dy, x, g, mean, var):
        return singa.GpuBatchNormBackward(h, dy, x, g, mean, var)

    # cross-op fusion the tape permits: the ReLU behind a BatchNorm folded into its backward
    fuse_bn_relu = True

    def bn_relu_bwd(self, h, dy, x, g, b, mean, var):
        return singa.GpuBatchNormReLUBackward(h, dy, x, g, b, mean, var)

    def conv_bwd_x(self, dy, W, x, h):
        return singa.GpuConvBackwardx(dy, W, x, h)

    # scheduling the tape permits: nothing reads a weight gradient before the update, so the weight
    # gradients of a backward pass run on the device's auxiliary stream beside the chain of data
    # gradients / BatchNorm / ReLU backward ops (matrix-bound work beside bandwidth-bound work)
    overlap_wgrad = True
    graph_overlap = True   # the weight gradients as a branch of a recorded graph as well (see conv_bwd_w)
    _aux = None          # the auxiliary stream while a backward pass is under way

    # While a graph records, a fork per layer makes a recording whose replay is slower than the plain chain (6.04
    # against 5.53 ms for ResNet-18: every fork is a cross-stream edge of the graph); there the weight gradients
    # are held back and go to the auxiliary stream `graph_wgrad_group` layers at a time, behind ONE fork
    # (groups of 6 to 10: 5.44 ms; ResNet-50 in 16 bits 9.70 against 9.89 ms).
    graph_wgrad_group = 8
    _deferred = ()

    def conv_bwd_w(self, dy, x, W, h):
        if self._aux is not None:
            if self.dev.graph_enabled() and self.graph_wgrad_group > 1:
                dW = singa.Tensor(W.shape(), W.device(), W.data_type())
                self._deferred = list(self._deferred) + [(dy, x, W, h, dW)]
                if len(self._deferred) >= self.graph_wgrad_group:
                    self._flush_deferred()
                return dW
            self._aux = self.dev.Fork()    # (everything enqueued so far, i.e. the producer of dy, comes first)
            # (the tensors it touches are announced to the pool there: nothing is kept alive here)
            return singa.GpuConvBackwardW(dy, x, W, h, stream=self._aux)
        return singa.GpuConvBackwardW(dy, x, W, h)

    def _flush_deferred(self):
        if self._deferred:
            self._aux = self.dev.Fork()
            for dy, x, W, h, dW in self._deferred:
                singa.GpuConvBackwardW(dy, x, W, h, stream=self._aux, out=dW)
            self._deferred = ()

    # cross-op fusion the tape permits: the "+=" of a residual fan-in folded into the data gradient
    fuse_dgrad_add = True

    def conv_bwd_x_acc(self, dy, W, x, h, into):
        return singa.GpuConvBackwardxAccumulate(dy, W, x, h, into)

    def conv_bwd_b(self, dy, b, h):
        return singa.GpuConvBackwardb(dy, b, h)

    # cross-op fusion the tape permits: a layer's bias gradient computed with its weight gradient
    fuse_wgrad_bias = True

    def conv_bwd_wb(self, dy, x, W, b, h):
        return singa.GpuConvBackwardWb(dy, x, W, b, h)

    # cross-op fusion the tape permits: a residual block hands its input gradient on as two summands
    # and the ReLU backward of the block before adds them while gating (HalfHipOps turns it on)
    fuse_add_relu = False

    def relu_bwd_add(self, dy0, dy1, x):
        return singa.ReLUBackwardSum(dy0, dy1, x)

    # batching the tape permits: the weights do not change during a backward pass, so the re-layouts
    # that the data gradients need are done by one launch before the first backward op
    batch_relayout = True

    def prepare_backward(self, convs, update_at_end=False):
        """`update_at_end`: no parameter is updated (no weight gradient read) before finish_backward."""
        # (while a graph is being recorded only if `graph_overlap` says so: the weight gradients become a branch of
        # the recording)
        if self.overlap_wgrad and update_at_end and (self.graph_overlap or not self.dev.graph_enabled()):
            self._aux = self.dev.AuxStream()
        if self.batch_relayout:
            by_type = {}
            for c in convs:
                if c.h is not None:
                    by_type.setdefault(c.W.data_type(), []).append((c.W, c.h))
            for pairs in by_type.values():
                singa.GpuConvPrepareBackward(pairs)

    def finish_backward(self, convs):
        if self._aux is not None:
            self._flush_deferred()
            self.dev.Join()    # the update (and any reader of a weight gradient) comes after the last of them
            self._aux = None

    fusions = ("fuse_bn_relu", "fuse_dgrad_add", "fuse_wgrad_bias", "batch_relayout", "overlap_wgrad", "fuse_forward")   # what set_fusion(True) turns on

    def set_fusion(self, on):
        """All of this implementation's cross-op fusions on, or the reference's op-per-op tape."""
        for f in ("fuse_bn_relu", "fuse_dgrad_add", "fuse_add_relu", "fuse_wgrad_bias", "batch_relayout", "overlap_wgrad",
                  "fuse_forward"):
            setattr(self, f, bool(on) and f in self.fusions)

    def accumulate(self, a, b):
        a += b
        return a

    def make_sgd(self, lr, momentum):
        return hip_opt.SGD(lr=lr, momentum=momentum)

    # precision boundary of a mixed-precision graph (identity here)
    def to_compute(self, x):
        return x

    def to_storage(self, x):
        return x


class _MixedSGD(hip_opt.SGD):
    """16-bit parameters are updated through an fp32 master copy and fp32 momentum
    (``SGD.apply_master``); fp32 parameters as usual."""

    def apply(self, name, p, g):
        if p.data_type() != singa.kFloat32:
            return self.apply_master(name, p, g)
        return super(_MixedSGD, self).apply(name, p, g)

    def apply_all(self, named_params_grads):
        return self.apply_all_mixed(named_params_grads)


class HalfHipOps(HipOps):
    """Mixed precision as the reference trains in half (``layer.py:684-696`` casts the conv / linear
    parameters to the input's type; cuDNN keeps BatchNorm parameters and statistics in fp32):
    4-D tensors -- activations, their gradients and convolution weights -- are stored in `dtype`
    (binary16 or bfloat16), BatchNorm parameters / statistics and the classifier head stay fp32,
    16-bit weights are updated through fp32 master copies."""

    # the residual "+=": folded into the next ReLU backward (the 16-bit data-gradient kernel's
    # scattered 2-byte stores make a read-modify-write epilogue slower than the separate add)
    fuse_dgrad_add = False
    fuse_add_relu = True
    fusions = ("fuse_bn_relu", "fuse_add_relu", "fuse_wgrad_bias", "batch_relayout", "overlap_wgrad", "fuse_forward")

    def __init__(self, dev, dtype):
        HipOps.__init__(self, dev)
        self.dtype = dtype
        self.name = "hip-" + singa._SUFFIX[dtype]

    def from_numpy(self, a):
        t = singa.from_numpy(a, self.dev)
        return t.AsType(self.dtype) if np.ndim(a) == 4 else t

    def relu(self, x):
        if x.data_type() == singa.kFloat32:
            return singa.ReLU(x)
        return singa.ReLUBackward(x, x)   # y = x > 0 ? x : 0, the same selection

    def to_compute(self, x):
        return x.AsType(singa.kFloat32)

    def to_storage(self, x):
        return x.AsType(self.dtype)

    def make_sgd(self, lr, momentum):
        return _MixedSGD(lr=lr, momentum=momentum)


# ------------------------------------------------------------------------------------ layers

class _Layer(object):
    params = ()

    def param_items(self):
        return [(self.name + "." + k, getattr(self, k)) for k in self.params]


class Conv(_Layer):
    def __init__(self, ops, name, W, b, stride, pad):
        self.ops, self.name, self.W, self.b = ops, name, ops.from_numpy(W), (ops.from_numpy(b) if b is not None else None)
        self.k = W.shape
        self.stride, self.pad = stride, pad
        self.params = ("W", "b") if b is not None else ("W",)
        self.h = None

    def fwd(self, x):
        if self.h is None:
            K, C, R, S = self.k
            self.h = self.ops.conv_handle(x, (R, S), self.stride, self.pad, C, K, self.b is not None)
        self.x = x
        return self.ops.conv_fwd(x, self.W, self.b, self.h)

    def bwd(self, dy, grads, add_into=None):
        """`add_into`: a gradient of this convolution's input that arrived earlier over another
        branch; the data gradient is added into that tensor (ops implementations with
        ``fuse_dgrad_add``), which is returned."""
        # A weight gradient that goes to the auxiliary stream is enqueued first, so that it starts beside
        # this layer's data gradient instead of behind it (it has a workspace of its own there).
        early = getattr(self.ops, "_aux", None) is not None
        db = None
        if early:
            dW = self.ops.conv_bwd_w(dy, self.x, self.W, self.h)
        # _Conv2d.backward: dx is always computed, even for the network input (autograd.py:1695-1697)
        if add_into is not None:
            dx = self.ops.conv_bwd_x_acc(dy, self.W, self.x, self.h, add_into)
        else:
            dx = self.ops.conv_bwd_x(dy, self.W, self.x, self.h)
        if not early:
            if self.b is not None and getattr(self.ops, "fuse_wgrad_bias", False):
                dW, db = self.ops.conv_bwd_wb(dy, self.x, self.W, self.b, self.h)
            else:
                dW = self.ops.conv_bwd_w(dy, self.x, self.W, self.h)
        grads(self.name + ".W", self.W, dW)
        if self.b is not None:
            grads(self.name + ".b", self.b, db if db is not None else self.ops.conv_bwd_b(dy, self.b, self.h))
        return dx


class BatchNorm(_Layer):
    params = ("scale", "bias")

    def __init__(self, ops, name, C, momentum=0.9):
        self.ops, self.name, self.momentum = ops, name, momentum
        self.scale = ops.from_numpy(np.ones(C, np.float32))
        self.bias = ops.from_numpy(np.zeros(C, np.float32))
        self.running_mean = ops.from_numpy(np.zeros(C, np.float32))
        self.running_var = ops.from_numpy(np.ones(C, np.float32))
        self.h = None

    def fwd(self, x):
        if self.h is None:
            self.h = self.ops.bn_handle(self.momentum, x)
        y, self.mean, self.var = self.ops.bn_fwd_train(self.h, x, self.scale, self.bias, self.running_mean,
                                                       self.running_var)
        self.x = x
        return y

    def fwd_through_relu(self, relu, x):
        """Forward of ``relu(self(x))``, as one fused call where the ops implementation offers it.  The ReLU then
        keeps its output for its backward: positive exactly where its input was."""
        if not getattr(self.ops, "fuse_forward", False):
            return relu.fwd(self.fwd(x))
        if self.h is None:
            self.h = self.ops.bn_handle(self.momentum, x)
        y, self.mean, self.var = self.ops.bn_relu_fwd_train(self.h, x, self.scale, self.bias, self.running_mean,
                                                            self.running_var)
        self.x = x
        relu.x = y
        return y

    def fwd_add_relu(self, relu, x, residual):
        """Forward of ``relu(self(x) + residual)``, the end of a residual block, as one fused call where the ops
        implementation offers it (this layer's own output is then never stored: its backward needs x only)."""
        if not getattr(self.ops, "fuse_forward", False):
            return relu.fwd_of_sum(self.fwd(x), residual)
        if self.h is None:
            self.h = self.ops.bn_handle(self.momentum, x)
        y, self.mean, self.var = self.ops.bn_add_relu_fwd_train(self.h, x, residual, self.scale, self.bias,
                                                                self.running_mean, self.running_var)
        self.x = x
        relu.x = y
        return y

    def bwd(self, dy, grads):
        dx, ds, db = self.ops.bn_bwd(self.h, dy, self.x, self.scale, self.mean, self.var)
        grads(self.name + ".scale", self.scale, ds)
        grads(self.name + ".bias", self.bias, db)
        return dx

    def bwd_through_relu(self, relu, dy, grads):
        """Backward of ``relu(self(x))``: ReLU.backward then BatchNorm.backward, as one fused call
        where the ops implementation offers it."""
        if not getattr(self.ops, "fuse_bn_relu", False):
            return self.bwd(relu.bwd(dy, grads), grads)
        dx, ds, db = self.ops.bn_relu_bwd(self.h, dy, self.x, self.scale, self.bias, self.mean, self.var)
        grads(self.name + ".scale", self.scale, ds)
        grads(self.name + ".bias", self.bias, db)
        return dx


class _Sum:
    """A gradient still in two summands (``a`` freshly computed and owned by the tape, ``b`` possibly
    shared): what a residual block returns under ``fuse_add_relu``; consumed by the ReLU backward of
    the block before, or summed by ``_summed`` for any other reader."""

    def __init__(self, a, b):
        self.a, self.b = a, b


def _summed(ops, dy):
    return ops.accumulate(dy.a, dy.b) if isinstance(dy, _Sum) else dy


class ReLU(_Layer):
    def __init__(self, ops, name):
        self.ops, self.name = ops, name

    def fwd(self, x):
        self.x = x
        return self.ops.relu(x)

    def fwd_of_sum(self, a, b):
        """Forward of ``relu(a + b)`` (the end of a residual block), in one pass where the ops implementation
        offers it; the output is kept for the backward as in BatchNorm.fwd_through_relu."""
        if not getattr(self.ops, "fuse_forward", False):
            return self.fwd(self.ops.add(a, b))
        self.x = self.ops.add_relu(a, b)
        return self.x

    def bwd(self, dy, grads):
        if isinstance(dy, _Sum):
            return self.ops.relu_bwd_add(dy.a, dy.b, self.x)
        return self.ops.relu_bwd(dy, self.x)


class Pool(_Layer):
    def __init__(self, ops, name, kernel, stride, pad, is_max):
        self.ops, self.name, self.cfg, self.h = ops, name, (kernel, stride, pad, is_max), None

    def fwd(self, x):
        if self.h is None:
            self.h = self.ops.pool_handle(x, *self.cfg)
        self.x = x
        self.y = self.ops.pool_fwd(self.h, x)
        return self.y

    def bwd(self, dy, grads):
        return self.ops.pool_bwd(self.h, dy, self.x, self.y)


class Flatten(_Layer):
    def __init__(self, ops, name):
        self.ops, self.name = ops, name

    def fwd(self, x):
        self.shape = self.ops.shape(x)
        n = self.shape[0]
        return self.ops.reshape(x, (n, int(np.prod(self.shape[1:]))))

    def bwd(self, dy, grads):
        return self.ops.reshape(dy, self.shape)


class Cast(_Layer):
    """Precision boundary in front of the classifier head: storage type -> fp32 and back for the
    gradient (``Tensor::AsType``); the identity for an all-fp32 graph."""

    def __init__(self, ops, name):
        self.ops, self.name = ops, name

    def fwd(self, x):
        return self.ops.to_compute(x) if hasattr(self.ops, "to_compute") else x

    def bwd(self, dy, grads):
        return self.ops.to_storage(dy) if hasattr(self.ops, "to_storage") else dy


class Linear(_Layer):
    params = ("W", "b")

    def __init__(self, ops, name, W, b):
        self.ops, self.name, self.W, self.b = ops, name, ops.from_numpy(W), ops.from_numpy(b)

    def fwd(self, x):
        self.x = x
        return self.ops.add_bias(self.ops.matmul(x, self.W), self.b)

    def bwd(self, dy, grads):
        # tape order: AddBias.backward (db) first, then Matmul.backward (autograd.py:613-623, :696-709)
        grads(self.name + ".b", self.b, self.ops.sum0(dy))
        dx, dW = self.ops.matmul_bwd(dy, self.x, self.W)
        grads(self.name + ".W", self.W, dW)
        return dx


class BasicBlock(_Layer):
    """examples/cnn/model/resnet.py:46-78."""

    def __init__(self, ops, name, rng, inplanes, planes, stride, downsample):
        self.ops, self.name = ops, name
        self.conv1 = Conv(ops, name + ".conv1", he_normal(rng, planes, inplanes, 3, 3), None, (stride, stride), (1, 1))
        self.bn1 = BatchNorm(ops, name + ".bn1", planes)
        self.relu1 = ReLU(ops, name + ".relu1")
        self.conv2 = Conv(ops, name + ".conv2", he_normal(rng, planes, planes, 3, 3), None, (1, 1), (1, 1))
        self.bn2 = BatchNorm(ops, name + ".bn2", planes)
        self.relu2 = ReLU(ops, name + ".relu2")
        self.ds_conv = self.ds_bn = None
        if downsample:
            self.ds_conv = Conv(ops, name + ".downsample.conv", he_normal(rng, planes, inplanes, 1, 1), None,
                                (stride, stride), (0, 0))
            self.ds_bn = BatchNorm(ops, name + ".downsample.bn", planes)

    def sublayers(self):
        ls = [self.conv1, self.bn1, self.relu1, self.conv2, self.bn2, self.relu2]
        if self.ds_conv is not None:
            ls += [self.ds_conv, self.ds_bn]
        return ls

    def fwd(self, x):
        out = self.conv2.fwd(self.bn1.fwd_through_relu(self.relu1, self.conv1.fwd(x)))
        residual = x
        if self.ds_conv is not None:
            residual = self.ds_bn.fwd(self.ds_conv.fwd(x))
        return self.bn2.fwd_add_relu(self.relu2, out, residual)

    def bwd(self, dy, grads):
        d_add = self.relu2.bwd(dy, grads)
        # Add.backward hands the same gradient to both inputs; the stack pops the residual branch first
        if self.ds_conv is not None:
            d_res = self.ds_conv.bwd(self.ds_bn.bwd(d_add, grads), grads)
        else:
            d_res = d_add
        d = self.bn1.bwd_through_relu(self.relu1, self.conv2.bwd(self.bn2.bwd(d_add, grads), grads), grads)
        if getattr(self.ops, "fuse_dgrad_add", False):
            return self.conv1.bwd(d, grads, add_into=d_res)   # every other reader of d_res is done by now
        d_main = self.conv1.bwd(d, grads)
        if getattr(self.ops, "fuse_add_relu", False):
            return _Sum(d_main, d_res)
        if d_res is d_add:
            # the first-arrived buffer is another op's input gradient: accumulate into the fresh one
            return self.ops.accumulate(d_main, d_res)
        return self.ops.accumulate(d_res, d_main)


class Bottleneck(_Layer):
    """examples/cnn/model/resnet.py:68-120: 1x1 reduce, 3x3 (carries the stride), 1x1 expand (x4)."""

    expansion = 4

    def __init__(self, ops, name, rng, inplanes, planes, stride, downsample):
        self.ops, self.name = ops, name
        out = planes * self.expansion
        self.conv1 = Conv(ops, name + ".conv1", he_normal(rng, planes, inplanes, 1, 1), None, (1, 1), (0, 0))
        self.bn1 = BatchNorm(ops, name + ".bn1", planes)
        self.relu1 = ReLU(ops, name + ".relu1")
        self.conv2 = Conv(ops, name + ".conv2", he_normal(rng, planes, planes, 3, 3), None, (stride, stride), (1, 1))
        self.bn2 = BatchNorm(ops, name + ".bn2", planes)
        self.relu2 = ReLU(ops, name + ".relu2")
        self.conv3 = Conv(ops, name + ".conv3", he_normal(rng, out, planes, 1, 1), None, (1, 1), (0, 0))
        self.bn3 = BatchNorm(ops, name + ".bn3", out)
        self.relu3 = ReLU(ops, name + ".relu3")
        self.ds_conv = self.ds_bn = None
        if downsample:
            self.ds_conv = Conv(ops, name + ".downsample.conv", he_normal(rng, out, inplanes, 1, 1), None,
                                (stride, stride), (0, 0))
            self.ds_bn = BatchNorm(ops, name + ".downsample.bn", out)

    def sublayers(self):
        ls = [self.conv1, self.bn1, self.relu1, self.conv2, self.bn2, self.relu2, self.conv3, self.bn3, self.relu3]
        if self.ds_conv is not None:
            ls += [self.ds_conv, self.ds_bn]
        return ls

    def fwd(self, x):
        out = self.bn1.fwd_through_relu(self.relu1, self.conv1.fwd(x))
        out = self.bn2.fwd_through_relu(self.relu2, self.conv2.fwd(out))
        out = self.conv3.fwd(out)
        residual = x
        if self.ds_conv is not None:
            residual = self.ds_bn.fwd(self.ds_conv.fwd(x))
        return self.bn3.fwd_add_relu(self.relu3, out, residual)

    def bwd(self, dy, grads):
        d_add = self.relu3.bwd(dy, grads)
        if self.ds_conv is not None:   # the stack pops the residual branch first, as in BasicBlock
            d_res = self.ds_conv.bwd(self.ds_bn.bwd(d_add, grads), grads)
        else:
            d_res = d_add
        d = self.conv3.bwd(self.bn3.bwd(d_add, grads), grads)
        d = self.conv2.bwd(self.bn2.bwd_through_relu(self.relu2, d, grads), grads)
        d = self.bn1.bwd_through_relu(self.relu1, d, grads)
        if getattr(self.ops, "fuse_dgrad_add", False):
            return self.conv1.bwd(d, grads, add_into=d_res)
        d_main = self.conv1.bwd(d, grads)
        if getattr(self.ops, "fuse_add_relu", False):
            return _Sum(d_main, d_res)
        if d_res is d_add:
            return self.ops.accumulate(d_main, d_res)
        return self.ops.accumulate(d_res, d_main)


def he_normal(rng, *shape):
    fan_in = int(np.prod(shape[1:])) if len(shape) > 2 else shape[0]
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)


# ------------------------------------------------------------------------------------ networks

class Net(object):
    """A sequential stack (blocks may branch internally) + softmax cross-entropy + SGD-momentum."""

    def __init__(self, ops, layers, lr, momentum):
        self.ops, self.layers = ops, layers
        self.sgd = ops.make_sgd(lr, momentum)
        self.grad_log = None  # name -> gradient tensor, filled when keep_grads is set

    def leaf_layers(self):
        out = []
        for l in self.layers:
            out += l.sublayers() if hasattr(l, "sublayers") else [l]
        return out

    def params(self):
        items = []
        for l in self.leaf_layers():
            items += l.param_items()
        return items

    def convs(self):
        return [l for l in self.leaf_layers() if isinstance(l, Conv)]

    SAVED = ("x", "y", "mean", "var")

    def adopt_saved_tensors(self, other):
        """Replace everything this net's forward saved for its backward (layer inputs/outputs, BN
        statistics, softmax output) by copies of `other`'s, converting between the two ops
        implementations.  Lets a backward pass be compared on exactly the same activations."""
        for mine, theirs in zip(self.leaf_layers(), other.leaf_layers()):
            for k in self.SAVED:
                if hasattr(theirs, k):
                    setattr(mine, k, self.ops.from_numpy(other.ops.to_numpy(getattr(theirs, k))))
        self.p = self.ops.from_numpy(other.ops.to_numpy(other.p))

    def forward(self, x, labels):
        """Runs the forward pass, keeps what the backward needs, returns the mean loss tensor data."""
        self.batch = self.ops.shape(x)[0]
        i = 0
        while i < len(self.layers):
            l = self.layers[i]
            if isinstance(l, BatchNorm) and i + 1 < len(self.layers) and isinstance(self.layers[i + 1], ReLU):
                x = l.fwd_through_relu(self.layers[i + 1], x)   # the stem's conv -> BatchNorm -> ReLU
                i += 2
            else:
                x = l.fwd(x)
                i += 1
        self.logits = x
        self.p = self.ops.softmax(x)
        self.t = labels
        return self.ops.ce_fwd(self.p, labels)

    def backward_and_update(self, keep_grads=False, fused_update=False):
        """The timed region: loss-gradient seed -> last parameter updated."""
        ops = self.ops
        self.grad_log = {} if keep_grads else None
        pending = []

        def grads(name, p, g):
            if keep_grads:
                self.grad_log[name] = g
            if fused_update:
                pending.append((name, p, g))
            else:
                self.sgd.apply(name, p, g)

        convs = self.convs() if hasattr(ops, "prepare_backward") else []
        if convs:
            ops.prepare_backward(convs, update_at_end=fused_update)   # (a layer's data gradient runs before its weights change)
        try:
            dy = ops.softmax_ce_bwd(self.p, self.t, self.batch)
            if keep_grads:
                self.grad_log["logits"] = dy
            rev = list(reversed(self.layers))
            i = 0
            while i < len(rev):
                if isinstance(rev[i], ReLU) and i + 1 < len(rev) and isinstance(rev[i + 1], BatchNorm):
                    dy = rev[i + 1].bwd_through_relu(rev[i], _summed(ops, dy), grads)   # the stem's conv -> BatchNorm -> ReLU
                    i += 2
                else:
                    if not isinstance(rev[i], (BasicBlock, Bottleneck)):
                        dy = _summed(ops, dy)
                    dy = rev[i].bwd(dy, grads)
                    i += 1
            dy = _summed(ops, dy)
        finally:
            if convs:
                ops.finish_backward(convs)
        if keep_grads:
            self.grad_log["input"] = dy
        if fused_update:
            self.sgd.apply_all(pending)
        self.sgd.step()
        return dy


def build_mlp(ops, rng, lr=0.05, momentum=0.9, in_dim=784, hidden=1000, classes=10):
    return Net(ops, [
        Linear(ops, "linear1", he_normal(rng, in_dim, hidden), np.zeros(hidden, np.float32)),
        ReLU(ops, "relu"),
        Linear(ops, "linear2", he_normal(rng, hidden, classes), np.zeros(classes, np.float32)),
    ], lr, momentum)


def build_cnn(ops, rng, lr=0.05, momentum=0.9, in_ch=3, image=32, classes=10, c1=32, c2=64):
    feat = c2 * (image // 4) * (image // 4)
    return Net(ops, [
        Conv(ops, "conv1", he_normal(rng, c1, in_ch, 5, 5), np.zeros(c1, np.float32), (1, 1), (2, 2)),
        ReLU(ops, "relu1"),
        Pool(ops, "pool1", (2, 2), (2, 2), (0, 0), True),
        Conv(ops, "conv2", he_normal(rng, c2, c1, 5, 5), np.zeros(c2, np.float32), (1, 1), (2, 2)),
        ReLU(ops, "relu2"),
        Pool(ops, "pool2", (2, 2), (2, 2), (0, 0), True),
        Flatten(ops, "flatten"),
        Linear(ops, "linear", he_normal(rng, feat, classes), np.zeros(classes, np.float32)),
    ], lr, momentum)


def build_resnet18(ops, rng, lr=0.05, momentum=0.9, classes=1000, in_ch=3, widths=(64, 128, 256, 512),
                   blocks=(2, 2, 2, 2), final_pool=7):
    layers = [
        Conv(ops, "conv1", he_normal(rng, widths[0], in_ch, 7, 7), None, (2, 2), (3, 3)),
        BatchNorm(ops, "bn1", widths[0]),
        ReLU(ops, "relu"),
        Pool(ops, "maxpool", (3, 3), (2, 2), (1, 1), True),
    ]
    inplanes = widths[0]
    for si, (planes, nb) in enumerate(zip(widths, blocks)):
        stride = 1 if si == 0 else 2
        for bi in range(nb):
            s = stride if bi == 0 else 1
            ds = bi == 0 and (s != 1 or inplanes != planes)
            layers.append(BasicBlock(ops, "layer%d.%d" % (si + 1, bi), rng, inplanes, planes, s, ds))
            inplanes = planes
    layers += [
        Pool(ops, "avgpool", (final_pool, final_pool), (1, 1), (0, 0), False),
        Flatten(ops, "flatten"),
        Linear(ops, "fc", he_normal(rng, inplanes, classes), np.zeros(classes, np.float32)),
    ]
    return Net(ops, layers, lr, momentum)


def build_resnet50(ops, rng, lr=0.05, momentum=0.9, classes=1000, in_ch=3, widths=(64, 128, 256, 512),
                   blocks=(3, 4, 6, 3), final_pool=7):
    """examples/cnn/model/resnet.py:121-185 with Bottleneck blocks (resnet50: stages [3, 4, 6, 3])."""
    layers = [
        Conv(ops, "conv1", he_normal(rng, widths[0], in_ch, 7, 7), None, (2, 2), (3, 3)),
        BatchNorm(ops, "bn1", widths[0]),
        ReLU(ops, "relu"),
        Pool(ops, "maxpool", (3, 3), (2, 2), (1, 1), True),
    ]
    inplanes = widths[0]
    for si, (planes, nb) in enumerate(zip(widths, blocks)):
        stride = 1 if si == 0 else 2
        for bi in range(nb):
            s = stride if bi == 0 else 1
            ds = bi == 0 and (s != 1 or inplanes != planes * Bottleneck.expansion)
            layers.append(Bottleneck(ops, "layer%d.%d" % (si + 1, bi), rng, inplanes, planes, s, ds))
            inplanes = planes * Bottleneck.expansion
    layers += [
        Pool(ops, "avgpool", (final_pool, final_pool), (1, 1), (0, 0), False),
        Flatten(ops, "flatten"),
        Cast(ops, "head_precision"),
        Linear(ops, "fc", he_normal(rng, inplanes, classes), np.zeros(classes, np.float32)),
    ]
    return Net(ops, layers, lr, momentum)


# ------------------------------------------------------------------------------------ configurations

CONFIGS = {
    # name: (builder, kwargs, input shape without batch, classes, default batch)
    "mlp": (build_mlp, {}, (784,), 10, 128),
    "cnn": (build_cnn, {}, (3, 32, 32), 10, 128),
    "resnet18": (build_resnet18, {}, (3, 224, 224), 1000, 64),
    # reduced variants used where a CPU implementation has to keep up
    "smoke_cnn": (build_cnn, {"image": 16, "c1": 8, "c2": 16}, (3, 16, 16), 10, 4),
    "resnet18_small": (build_resnet18, {"classes": 100, "final_pool": 2}, (3, 64, 64), 100, 2),
    # bottleneck network of the half-precision configuration (run with HalfHipOps), and a narrow one
    "resnet50": (build_resnet50, {}, (3, 224, 224), 1000, 128),
    "resnet50_small": (build_resnet50, {"classes": 100, "final_pool": 2, "widths": (16, 32, 64, 128)},
                       (3, 64, 64), 100, 4),
}

SEED_BASE = 0x5167A000
# Seeds: SEED_BASE + 256 * configuration + tensor index; tensor 0 is the input batch, 1 the labels, 2.. the
# weight tensors in the order the builder creates them.  The generator is counter-based (singa_amd/rng.py:
# splitmix64 -> Box-Muller), so the bytes do not depend on a library's random stream and a smaller batch is
# a prefix of a larger one.  (Fixed numbers: adding a configuration leaves the inputs of the others unchanged.)
_CONFIG_INDEX = {"mlp": 1, "conv": 2, "cnn": 3, "resnet18": 4, "resnet50": 5, "resnet18_small": 6, "smoke_cnn": 7,
                 "resnet50_small": 8}


def make_inputs(name, batch=None):
    builder, kw, xshape, classes, default_batch = CONFIGS[name]
    batch = batch or default_batch
    base = SEED_BASE + 256 * _CONFIG_INDEX[name]
    x = rng.normal(base + 0, (batch,) + xshape)
    labels = rng.integers(base + 1, (batch,), classes)
    return x, labels


def build(name, ops, lr=0.05, momentum=0.9):
    builder, kw, _, _, _ = CONFIGS[name]
    stream = rng.Stream(SEED_BASE + 256 * _CONFIG_INDEX[name])
    stream.index = 2
    return builder(ops, stream, lr=lr, momentum=momentum, **kw)


def resnet18_flops(batch=64):
    """Algorithmic conv FLOPs of one ResNet-18 backward: 2*N*K*P*Q*C*R*S per gradient, for dgrad
    and wgrad of all 20 convolutions (the stem's dgrad included, SINGA computes it)."""
    convs = [(3, 64, 7, 112)]
    inpl, size = 64, 56
    for si, planes in enumerate((64, 128, 256, 512)):
        for bi in range(2):
            s = 2 if (si > 0 and bi == 0) else 1
            size = size // s
            convs.append((inpl, planes, 3, size))
            convs.append((planes, planes, 3, size))
            if bi == 0 and (s != 1 or inpl != planes):
                convs.append((inpl, planes, 1, size))
            inpl = planes
    per_grad = sum(2.0 * batch * k * p * p * c * r * r for c, k, r, p in convs)
    return {"wgrad": per_grad, "dgrad": per_grad, "convs": len(convs)}


# ------------------------------------------------------------------------------------ parity driver

def _nl2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    d = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / (d if d > 0 else 1.0))


def run_parity_case(name, dev, checker_ops, batch=None, steps=1, share_activations=True, hip_ops=None):
    """Replays configuration `name` on the GPU and on `checker_ops` (an ops implementation handed
    in by the caller, e.g. the test-suite's CPU oracle) from identical inputs.  Both run their own
    forward (loss and logits are compared); with share_activations the GPU backward then consumes
    the checker's saved activations, so the reported errors are those of the backward kernels
    alone.  Returns per-tensor normalised L2 errors of every gradient and updated parameter."""
    hip = hip_ops if hip_ops is not None else HipOps(dev)
    if not hasattr(checker_ops, "from_numpy"):
        raise TypeError("checker_ops must implement the ops interface")
    x, labels = make_inputs(name, batch)
    nets = []
    for ops in (hip, checker_ops):
        net = build(name, ops)
        nets.append(net)
    errors = {}
    for step in range(steps):
        losses = []
        for net in nets:
            loss = net.forward(net.ops.from_numpy(x), net.ops.from_numpy(labels))
            losses.append(net.ops.to_numpy(loss))
        errors["step%d.loss" % step] = _nl2(losses[0], losses[1])
        errors["step%d.logits" % step] = _nl2(hip.to_numpy(nets[0].logits), checker_ops.to_numpy(nets[1].logits))
        if share_activations:
            nets[0].adopt_saved_tensors(nets[1])
        for net in nets:
            net.backward_and_update(keep_grads=True)
        for k in nets[1].grad_log:
            errors["step%d.grad.%s" % (step, k)] = _nl2(hip.to_numpy(nets[0].grad_log[k]),
                                                       checker_ops.to_numpy(nets[1].grad_log[k]))
        for (k, p0), (_, p1) in zip(nets[0].params(), nets[1].params()):
            errors["step%d.param.%s" % (step, k)] = _nl2(hip.to_numpy(p0), checker_ops.to_numpy(p1))
    return {"errors": errors}
