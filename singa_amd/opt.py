"""SGD with momentum as ``python/singa/opt.py`` defines it (class SGD :168-333), with the four
tensor ops of ``SGD.apply`` (:269-310) replaced by one fused kernel launch per parameter, or by a
single launch over all parameters (``apply_all``, the loop of ``Optimizer.call`` :107-111).

    [g += weight_decay * p]
    v  = momentum * v + (1 - dampening) * g
    g' = g + momentum * v   (nesterov)   |   v   (otherwise)
    p -= lr * g'
"""
import ctypes as C

import numpy as np

from . import _lib
from . import singa_wrap as singa
from ._lib import check


class SGD(object):

    def __init__(self, lr=0.1, momentum=0, dampening=0, weight_decay=0, nesterov=False, op_by_op=False):
        if momentum < 0.0:
            raise ValueError("Invalid momentum value: {}".format(momentum))
        if weight_decay < 0.0:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError("Nesterov momentum requires a momentum and zero dampening")
        self.lr = float(lr)
        self.momentum = float(momentum)
        self.dampening = float(dampening)
        self.weight_decay = float(weight_decay)
        self.nesterov = bool(nesterov)
        # op_by_op: ``apply`` issues the reference's own tensor ops (Axpy with 1-element device tensors, the
        # in-place product with the momentum tensor) instead of the fused kernel -- what unchanged
        # python/singa/opt.py does through the Axpy / EltwiseMult entry points; bit-identical results
        self.op_by_op = bool(op_by_op)
        self._hyper = None
        self.moments = dict()
        self.masters = dict()
        self.step_counter = 0
        self._table = None
        self._table_key = None
        self._tables = {}

    def _moment(self, name, p):
        if name not in self.moments:
            if p.data_type() == singa.kFloat32:
                v = singa.Tensor(p.shape(), p.device(), singa.kFloat32)
                v.SetFloatValue(0.0)
            else:  # zeros in a 16-bit type: cast fp32 zeros
                z = singa.Tensor(p.shape(), p.device(), singa.kFloat32)
                z.SetFloatValue(0.0)
                v = z.AsType(p.data_type())
            self.moments[name] = v
        return self.moments[name]

    def apply(self, param_name, param_value, param_grad):
        """One fused update of ``param_value`` (in place).  Unlike the reference the gradient
        tensor is left untouched."""
        assert param_value.shape() == param_grad.shape(), ("shape mismatch", param_value.shape(),
                                                             param_grad.shape())
        if param_value.data_type() != param_grad.data_type():
            raise singa.SingaHipError("parameter and gradient differ in data type")
        if self.op_by_op and param_value.data_type() == singa.kFloat32:
            return self._apply_op_by_op(param_name, param_value, param_grad)
        v = self._moment(param_name, param_value) if self.momentum != 0 else None
        name = "sgh_sgd_momentum_" + singa._SUFFIX[param_value.data_type()]   # f32 / f16 / bf16
        check(getattr(_lib.lib(), name)(param_value.ptr, param_grad.ptr, v.ptr if v is not None else None,
                                        param_value.Size(), self.lr, self.momentum, self.dampening,
                                        self.weight_decay, int(self.nesterov), param_value.device().stream), name)

    def _apply_op_by_op(self, param_name, param_value, param_grad):
        """``SGD.apply`` as the reference writes it (python/singa/opt.py:269-310), op by op on 1-element device
        tensors: 3 launches per parameter with momentum and no weight decay.  Unlike the fused kernel it may
        overwrite the gradient tensor, as the reference does."""
        dev = param_value.device()
        if self._hyper is None:
            mk = lambda v: singa.from_numpy(np.array([v], dtype=np.float32), dev)
            self._hyper = {"decay": mk(self.weight_decay), "mom": mk(self.momentum), "alpha": mk(1.0 - self.dampening),
                           "minus_lr": mk(0.0 - self.lr)}
        h = self._hyper
        if self.weight_decay != 0:
            singa.Axpy(h["decay"], param_value, param_grad)            # g += wd * p
        if self.momentum != 0:
            buf = self._moment(param_name, param_value)
            buf *= h["mom"]                                            # v *= mu      (EltwiseMult, scalar tensor)
            singa.Axpy(h["alpha"], param_grad, buf)                    # v += (1 - damp) * g
            if self.nesterov:
                singa.Axpy(h["mom"], buf, param_grad)                  # g += mu * v
            else:
                param_grad = buf
        singa.Axpy(h["minus_lr"], param_grad, param_value)             # p += (-lr) * g

    def apply_master(self, param_name, param_value, param_grad):
        """Mixed precision: ``param_value`` / ``param_grad`` are 16-bit; an fp32 master copy of the
        parameter (created from it on first use) and an fp32 momentum buffer are updated, and
        ``param_value`` is refreshed from the master."""
        if param_value.data_type() not in (singa.kFloat16, singa.kBFloat16):
            raise singa.SingaHipError("apply_master expects 16-bit parameters")
        if param_value.data_type() != param_grad.data_type() or param_value.shape() != param_grad.shape():
            raise singa.SingaHipError("parameter and gradient differ in shape or data type")
        if param_name not in self.masters:
            self.masters[param_name] = param_value.AsType(singa.kFloat32)
        master = self.masters[param_name]
        v = self._moment(param_name, master) if self.momentum != 0 else None
        name = "sgh_sgd_momentum_master_" + singa._SUFFIX[param_value.data_type()]
        check(getattr(_lib.lib(), name)(master.ptr, param_grad.ptr, v.ptr if v is not None else None, param_value.ptr,
                                        param_value.Size(), self.lr, self.momentum, self.dampening,
                                        self.weight_decay, int(self.nesterov), param_value.device().stream), name)

    def apply_all(self, named_params_grads):
        """Update every (name, p, g) triple with ONE kernel launch.  The pointer table is built
        once per distinct set of buffers and kept on the device; the memory pool hands the
        gradient buffers out in a short cycle of address sets, so a few tables are cached and a
        steady-state step usually uploads nothing; when the set is new (with weight gradients on
        the auxiliary stream the cycle of address sets is long) the table goes up through
        ``sgh_upload_async``, which does not drain the stream."""
        items = list(named_params_grads)
        if not items:
            return
        dev = items[0][1].device()
        key = tuple((n, p.ptr, g.ptr) for n, p, g in items)
        cached = self._tables.get(key)
        if cached is not None:
            self._table, self._table_total = cached
            self._table_key = key
        if key != self._table_key:
            arr = (_lib.SgdItem * len(items))()
            total = 0
            for i, (n, p, g) in enumerate(items):
                assert p.shape() == g.shape(), ("shape mismatch", n)
                v = self._moment(n, p) if self.momentum != 0 else None
                arr[i].p, arr[i].g, arr[i].v, arr[i].n = p.ptr, g.ptr, (v.ptr if v is not None else None), p.Size()
                total += p.Size()
            nbytes = C.sizeof(arr)
            table = singa.Tensor(((nbytes + 3) // 4,), dev, singa.kInt)
            check(_lib.lib().sgh_upload_async(dev._h, table.ptr, C.addressof(arr), nbytes), "sgh_upload_async")
            self._table, self._table_key, self._table_total = table, key, total
            if len(self._tables) >= 16:
                self._tables.pop(next(iter(self._tables)))
            self._tables[key] = (table, total)
        check(_lib.lib().sgh_sgd_momentum_multi_f32(self._table.ptr, len(items), self._table_total, self.lr,
                                                    self.momentum, self.dampening, self.weight_decay,
                                                    int(self.nesterov), dev.stream), "sgh_sgd_momentum_multi_f32")

    def apply_all_mixed(self, named_params_grads):
        """``apply_all`` for a mixed-precision network: fp32 parameters and 16-bit parameters (updated
        through fp32 master copies as in ``apply_master``) in ONE launch.  The 16-bit tensors must
        all have the same type."""
        items = list(named_params_grads)
        if not items:
            return
        dev = items[0][1].device()
        key = ("mixed",) + tuple((n, p.ptr, g.ptr) for n, p, g in items)
        cached = self._tables.get(key)
        if cached is None:
            arr = (_lib.SgdMixedItem * len(items))()
            total, half_type = 0, None
            for i, (n, p, g) in enumerate(items):
                assert p.shape() == g.shape(), ("shape mismatch", n)
                if p.data_type() != g.data_type():
                    raise singa.SingaHipError("parameter and gradient differ in data type")
                if p.data_type() == singa.kFloat32:
                    tgt, p16 = p, None
                else:
                    if half_type not in (None, p.data_type()):
                        raise singa.SingaHipError("one 16-bit type per update")
                    half_type = p.data_type()
                    if n not in self.masters:
                        self.masters[n] = p.AsType(singa.kFloat32)
                    tgt, p16 = self.masters[n], p.ptr
                v = self._moment(n, tgt) if self.momentum != 0 else None
                arr[i].p, arr[i].g, arr[i].v, arr[i].p16, arr[i].n = tgt.ptr, g.ptr, (v.ptr if v is not None else None), p16, p.Size()
                total += p.Size()
            nbytes = C.sizeof(arr)
            table = singa.Tensor(((nbytes + 3) // 4,), dev, singa.kInt)
            check(_lib.lib().sgh_upload_async(dev._h, table.ptr, C.addressof(arr), nbytes), "sgh_upload_async")
            if len(self._tables) >= 16:
                self._tables.pop(next(iter(self._tables)))
            cached = self._tables[key] = (table, total, int(half_type == singa.kBFloat16))
        table, total, bf16 = cached
        check(_lib.lib().sgh_sgd_momentum_multi_mixed(table.ptr, len(items), total, bf16, self.lr, self.momentum,
                                                      self.dampening, self.weight_decay, int(self.nesterov),
                                                      dev.stream), "sgh_sgd_momentum_multi_mixed")

    def through_half(self, g, clipping=False, clip_value=100, dtype=None):
        """What ``DistOpt.backward_and_update_half`` (python/singa/opt.py:867-920) does to a gradient on
        one GPU: optional clipping to [-clip_value, clip_value] (``autograd.clip``), then the trip through
        half precision that the gradient takes on its way through the communicator
        (``cuda::float2half`` / ``half2float``, src/io/communicator.cc:369-466).  The exchange between
        GPUs itself is not part of this library."""
        if g.data_type() != singa.kFloat32:
            raise singa.SingaHipError("backward_and_update_half is defined for float32 gradients")
        if clipping:
            g = singa.Clamp(-clip_value, clip_value, g)
        return g.AsType(dtype if dtype is not None else singa.kFloat16).AsType(singa.kFloat32)

    def step(self):
        self.step_counter += 1

    def get_states(self):
        return {k: v.to_numpy() for k, v in self.moments.items()}
