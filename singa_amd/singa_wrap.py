"""Host-side mirror of the slice of SINGA's ``singa_wrap`` (SWIG) module that the backward pass
uses, bound to the gfx950 library through its C ABI.

Names, argument order and meaning follow the reference so that code written against
``singa_wrap`` for a non-CPU device reads the same here:

* tensor functions: ``src/api/core_tensor.i`` (``ReLUBackward`` :344-355, ``Axpy`` :387-388,
  ``Mult``, ``SoftmaxCrossEntropyBwd``, ``CrossEntropyFwd``, ``SoftMax``, ``Sum``, ``SumAll``,
  ``__iadd__`` / ``__imul__``)
* operation handles and functions: ``src/api/model_operation.i:121-191``
  (``CudnnConvHandle``, ``GpuConvForward/Backwardx/BackwardW/Backwardb``,
  ``CudnnBatchNormHandle``, ``GpuBatchNormForwardTraining/Backward``,
  ``CudnnPoolingHandle``, ``GpuPoolingForward/Backward``)
* device factory: ``python/singa/device.py:103-114`` (``create_cuda_gpu_on``)

Every function only enqueues work on the device's stream; ``Device.Sync()`` or a copy to the
host waits for it.  Errors raise ``SingaHipError`` (the reference aborts through CHECK).
There is no CPU path in this module: without the built library and a GPU it cannot run.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import SingaHipError, check  # noqa: F401  (re-exported)

# core.proto DataType values (src/proto/core.proto:26-34)
kFloat32, kFloat16, kInt = 0, 1, 2
# bfloat16 storage is not a SINGA data type; the value lies outside core.proto's range
kBFloat16 = 100
# core.proto LangType (src/proto/core.proto:36-41); 3 is the value a HIP backend takes
kCpp, kCuda, kOpencl, kHip = 0, 1, 2, 3

_NP_OF = {kFloat32: np.float32, kInt: np.int32, kFloat16: np.float16, kBFloat16: np.uint16}
_SIZE_OF = {kFloat32: 4, kInt: 4, kFloat16: 2, kBFloat16: 2}
_SUFFIX = {kFloat32: "f32", kFloat16: "f16", kBFloat16: "bf16"}


def _fn(name, t):
    """The entry point of `name` for t's data type: sgh_<name>_<f32|f16|bf16>."""
    sfx = _SUFFIX.get(t.data_type())
    if sfx is None:
        raise SingaHipError("%s: unsupported data type %r" % (name, t.data_type()))
    full = "sgh_%s_%s" % (name, sfx)
    return getattr(_L(), full), full


def bf16_bits_to_float(bits):
    """uint16 bfloat16 payloads -> float32 values (exact)."""
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def float_to_bf16_bits(a):
    """float32 -> bfloat16 payloads, round to nearest even (NaN stays NaN)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7fffffff) > 0x7f800000
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r

USE_HIP = True


def _L():
    return _lib.lib()


# ------------------------------------------------------------------------------------ device

class HipGPU(object):
    """Counterpart of ``CudaGPU`` (include/singa/core/device.h:57-174): one stream, one pool (and an
    auxiliary stream for work the caller orders itself, see ``Fork``)."""

    def __init__(self, gpu_id=0):
        h = C.c_void_p()
        check(_L().sgh_device_open(int(gpu_id), C.byref(h)), "sgh_device_open")
        self._h = h
        self._id = int(gpu_id)
        self.stream = _L().sgh_device_stream(h)

    def id(self):
        return self._id

    def lang(self):
        return kHip

    def Sync(self):
        check(_L().sgh_device_sync(self._h), "sgh_device_sync")

    # Device::SetRandSeed (include/singa/core/device.h:64): the state behind Uniform / Gaussian is a seed
    # and a count of outputs consumed; a fill of n elements takes the next n (Gaussian: 2n) outputs
    _rand_seed, _rand_offset = 0, 0

    def SetRandSeed(self, seed):
        self._rand_seed, self._rand_offset = int(seed) & 0xFFFFFFFFFFFFFFFF, 0

    def _take_random(self, count):
        off = self._rand_offset
        self._rand_offset += int(count)
        return self._rand_seed, off

    _reduce_ws = None

    def reduce_workspace(self):
        if self._reduce_ws is None:
            self._reduce_ws = Tensor((_L().sgh_reduce_workspace_bytes() // 4,), self, kFloat32)
        return self._reduce_ws

    # A second compute stream for work that the main stream's next ops do not depend on.  Fork():
    # what is enqueued on the auxiliary stream afterwards starts when everything enqueued on the main
    # stream so far has finished; Join(): the main stream waits for the auxiliary one.  Tensors handed
    # to work on the auxiliary stream are announced with UsedOn(): they may then be dropped at any
    # time, the pool hands their memory out again only after the Join().
    _aux = None

    def AuxStream(self):
        if self._aux is None:
            s = _L().sgh_device_aux_stream(self._h)
            if not s:
                raise SingaHipError("no auxiliary stream")
            self._aux = s
        return self._aux

    def Fork(self):
        aux = C.c_void_p()
        check(_L().sgh_device_fork(self._h, C.byref(aux)), "sgh_device_fork")
        self._aux = aux.value
        return self._aux

    def Join(self):
        check(_L().sgh_device_join(self._h), "sgh_device_join")

    def UsedOn(self, stream, *tensors):
        for t in tensors:
            if t._block.owned:    # (memory the pool does not own is the caller's to keep alive)
                check(_L().sgh_block_used_on(self._h, t.ptr, stream), "sgh_block_used_on")

    def GetAllocatedMem(self):
        a, c, d = C.c_size_t(), C.c_size_t(), C.c_size_t()
        check(_L().sgh_pool_stats(self._h, C.byref(a), C.byref(c), C.byref(d)))
        return a.value

    def PoolStats(self):
        a, c, d = C.c_size_t(), C.c_size_t(), C.c_size_t()
        check(_L().sgh_pool_stats(self._h, C.byref(a), C.byref(c), C.byref(d)))
        return {"in_use": a.value, "cached": c.value, "driver_allocs": d.value}

    # Graph mode (include/singa/core/device.h:69-98): EnableGraph(True) .. EnableGraph(False)
    # records what is enqueued on the stream instead of running it (the reference buffers the
    # operations in its scheduler), RunGraph() replays the recording, ResetGraph() drops it.
    _graph = None
    _recording = False

    def graph_enabled(self):
        return self._recording

    def EnableGraph(self, flag):
        if flag and not self._recording:
            self.ResetGraph()
            check(_L().sgh_graph_begin(self._h), "sgh_graph_begin")
            self._recording = True
        elif not flag and self._recording:
            g = C.c_void_p()
            self._recording = False
            check(_L().sgh_graph_end(self._h, C.byref(g)), "sgh_graph_end")
            self._graph = g

    def RunGraph(self, serial=False):
        if self._graph is None:
            raise SingaHipError("RunGraph without a recorded graph")
        check(_L().sgh_graph_launch(self._graph), "sgh_graph_launch")

    def ResetGraph(self):
        if self._graph is not None:
            check(_L().sgh_graph_destroy(self._graph), "sgh_graph_destroy")
            self._graph = None

    def _malloc(self, nbytes):
        p = C.c_void_p()
        check(_L().sgh_malloc(self._h, C.byref(p), nbytes), "sgh_malloc")
        return p.value

    def _free(self, ptr):
        if self._h is not None and _lib._lib is not None:
            _lib._lib.sgh_free(self._h, C.c_void_p(ptr))


_devices = {}


def create_hip_gpu_on(device_id=0):
    """``device.create_cuda_gpu_on`` analogue; devices are cached per id like
    Platform::UsedDevice (src/core/device/platform.cc:137-160)."""
    if device_id not in _devices:
        _devices[device_id] = HipGPU(device_id)
    return _devices[device_id]


create_cuda_gpu_on = create_hip_gpu_on
create_cuda_gpu = create_hip_gpu_on


# ------------------------------------------------------------------------------------ tensor

class _Block(object):
    """Counterpart of ``Block`` (include/singa/core/common.h:64-97): a pool allocation freed
    when the last Tensor referring to it goes away."""

    def __init__(self, dev, nbytes, ptr=None, keepalive=None):
        self.dev = dev
        self.nbytes = nbytes
        self.owned = ptr is None
        self.ptr = dev._malloc(max(nbytes, 1)) if ptr is None else ptr
        self.keepalive = keepalive

    def __del__(self):
        try:
            if self.owned and self.ptr:
                self.dev._free(self.ptr)
                self.ptr = None
        except Exception:
            pass


class Tensor(object):
    """Counterpart of ``singa::Tensor`` as Python sees it (src/api/core_tensor.i:95-232):
    dense row-major data on a HipGPU, plus a transpose flag for 2-D views."""

    def __init__(self, shape=(), device=None, dtype=kFloat32, _block=None, _transposed=False):
        if device is None:
            raise SingaHipError("a HipGPU device is required (this module has no CPU path)")
        if dtype not in _SIZE_OF:
            raise SingaHipError("unsupported data type %r" % (dtype,))
        self._shape = tuple(int(s) for s in shape)
        self._dev = device
        self._dtype = dtype
        self._transposed = _transposed
        self._block = _block if _block is not None else _Block(device, self.Size() * _SIZE_OF[dtype])

    # --- reference accessors
    def shape(self, axis=None):
        return list(self._shape) if axis is None else self._shape[axis]

    def nDim(self):
        return len(self._shape)

    def Size(self):
        n = 1
        for s in self._shape:
            n *= s
        return n

    def MemSize(self):
        return self.Size() * _SIZE_OF[self._dtype]

    def data_type(self):
        return self._dtype

    def device(self):
        return self._dev

    def transpose(self):
        return self._transposed

    @property
    def ptr(self):
        return self._block.ptr

    # --- views
    def Reshape(self, shape):
        shape = tuple(int(s) for s in shape)
        t = Tensor(shape, self._dev, self._dtype, _block=self._block)
        if t.Size() != self.Size():
            raise SingaHipError("Reshape changes the element count")
        if self._transposed:
            raise SingaHipError("Reshape of a transposed view is not supported")
        return t

    def T(self):
        if len(self._shape) != 2:
            raise SingaHipError("T() needs a 2-D tensor")
        return Tensor((self._shape[1], self._shape[0]), self._dev, self._dtype, _block=self._block,
                      _transposed=not self._transposed)

    def Clone(self):
        t = Tensor(self._shape, self._dev, self._dtype, _transposed=self._transposed)
        check(_L().sgh_memcpy(self._dev._h, t.ptr, self.ptr, self.MemSize(), 3), "sgh_memcpy D2D")
        return t

    # --- host transfers
    def CopyFloatDataFromHostPtr(self, arr):
        a = np.ascontiguousarray(arr, dtype=np.float32).ravel()
        if a.size != self.Size() or self._dtype != kFloat32:
            raise SingaHipError("size or type mismatch in CopyFloatDataFromHostPtr")
        check(_L().sgh_memcpy(self._dev._h, self.ptr, a.ctypes.data, a.nbytes, 1), "sgh_memcpy H2D")

    def CopyIntDataFromHostPtr(self, arr):
        a = np.ascontiguousarray(arr, dtype=np.int32).ravel()
        if a.size != self.Size() or self._dtype != kInt:
            raise SingaHipError("size or type mismatch in CopyIntDataFromHostPtr")
        check(_L().sgh_memcpy(self._dev._h, self.ptr, a.ctypes.data, a.nbytes, 1), "sgh_memcpy H2D")

    def CopyHalfDataFromHostPtr(self, arr):
        """float16 values (kFloat16) or raw uint16 bfloat16 payloads (kBFloat16)."""
        a = np.ascontiguousarray(arr, dtype=_NP_OF[self._dtype]).ravel()
        if a.size != self.Size() or self._dtype not in (kFloat16, kBFloat16):
            raise SingaHipError("size or type mismatch in CopyHalfDataFromHostPtr")
        check(_L().sgh_memcpy(self._dev._h, self.ptr, a.ctypes.data, a.nbytes, 1), "sgh_memcpy H2D")

    def AsType(self, dtype):
        """``Tensor::AsType`` (src/core/tensor/tensor.cc:197-214) between fp32 and a 16-bit type or int32."""
        if dtype == self._dtype:
            return self
        if self._transposed:
            raise SingaHipError("AsType of a transposed view is not supported")
        out = Tensor(self._shape, self._dev, dtype)
        if self._dtype == kFloat32 and dtype in (kFloat16, kBFloat16):
            name = "sgh_cast_f32_to_%s" % _SUFFIX[dtype]
        elif dtype == kFloat32 and self._dtype in (kFloat16, kBFloat16):
            name = "sgh_cast_%s_to_f32" % _SUFFIX[self._dtype]
        elif self._dtype == kFloat32 and dtype == kInt:      # (int)x: truncation toward zero
            name = "sgh_cast_f32_to_i32"
        elif self._dtype == kInt and dtype == kFloat32:
            name = "sgh_cast_i32_to_f32"
        else:
            raise SingaHipError("AsType %r -> %r is not on the backward path" % (self._dtype, dtype))
        check(getattr(_L(), name)(self.ptr, out.ptr, self.Size(), self._dev.stream), name)
        return out

    def to_numpy(self):
        """fp32 / int32 / float16 arrays; bfloat16 tensors come back as float32 values."""
        out = np.empty(self.Size(), dtype=_NP_OF[self._dtype])
        if out.size:
            check(_L().sgh_memcpy(self._dev._h, out.ctypes.data, self.ptr, out.nbytes, 2), "sgh_memcpy D2H")
        if self._dtype == kBFloat16:
            out = bf16_bits_to_float(out)
        if self._transposed:
            return out.reshape(self._shape[1], self._shape[0]).T.copy()
        return out.reshape(self._shape)

    def SetFloatValue(self, v):
        fn, name = _fn("memset", self)   # the fill of this tensor's element size (int tensors are not filled with floats)
        check(fn(self.ptr, float(v), self.Size(), self._dev.stream), name)

    # --- arithmetic used by autograd / opt  (Tensor::operator+=, *=: src/core/tensor/tensor.cc:579-589)
    def __iadd__(self, other):
        _same(self, other)
        fn, name = _fn("add", self)
        check(fn(self.ptr, other.ptr, self.ptr, self.Size(), self._dev.stream), name)
        return self

    def __imul__(self, other):
        if isinstance(other, Tensor):
            scalar = other.Size() == 1 and self.Size() != 1
            if not scalar:
                _same(self, other)
            if self._dtype != kFloat32 and not scalar:
                fn, name = _fn("eltwise_mult", self)
                check(fn(self.ptr, other.ptr, self.ptr, self.Size(), self._dev.stream), name)
                return self
            _need_f32("Tensor *=", self, other)
            check(_L().sgh_eltwise_mult_f32(self.ptr, other.ptr, int(scalar), self.ptr, self.Size(),
                                            self._dev.stream), "sgh_eltwise_mult_f32")
        else:
            _need_f32("Tensor *= scalar", self)
            s = from_numpy(np.array([other], dtype=np.float32), self._dev)
            check(_L().sgh_eltwise_mult_f32(self.ptr, s.ptr, 1, self.ptr, self.Size(), self._dev.stream),
                  "sgh_eltwise_mult_f32")
        return self

    def __itruediv__(self, d):
        # Div(tensor, scalar) multiplies by the fp32 reciprocal (src/core/tensor/tensor_math.h:149-153)
        return self.__imul__(float(np.float32(1.0) / np.float32(d)))


def _need_f32(what, *tensors):
    """The fp32-only entry points read their operands as floats: refuse anything else, as the
    reference's TYPE_LANG_SWITCH does for a type it has no kernel for (tensor.cc:760-812)."""
    for t in tensors:
        if t is not None and t.data_type() != kFloat32:
            raise SingaHipError("%s: float32 tensors only, got data type %r" % (what, t.data_type()))


def Transform(t):
    """``singa.Transform``: the dense copy of a view (here: a transposed 2-D view; dense tensors are
    returned as they are)."""
    if not t.transpose():
        return t
    _need_f32("Transform", t)
    rows, cols = t.shape()
    out = Tensor((rows, cols), t.device(), kFloat32)
    shape = (C.c_size_t * 2)(rows, cols)
    strides = (C.c_int64 * 2)(1, rows)       # element (i, j) of the view is element (j, i) of the stored matrix
    check(_L().sgh_transform_f32(t.ptr, out.ptr, 2, shape, strides, t.device().stream), "sgh_transform_f32")
    return out


def Broadcast(t, shape):
    """``Tensor::Broadcast`` (src/core/tensor/tensor.cc:481-503) made dense: NumPy's broadcasting
    rules, trailing dimensions aligned, stride 0 along every broadcast dimension."""
    _need_f32("Broadcast", t)
    t = Transform(t)
    shape = tuple(int(v) for v in shape)
    src = (1,) * (len(shape) - t.nDim()) + tuple(t.shape())
    if len(src) != len(shape) or any(a != b and a != 1 for a, b in zip(src, shape)):
        raise SingaHipError("cannot broadcast %s to %s" % (t.shape(), list(shape)))
    if len(shape) > 8:
        raise SingaHipError("at most 8 dimensions")
    strides, acc = [], 1
    for a in reversed(src):
        strides.append(acc)
        acc *= a
    strides = [0 if a == 1 and b != 1 else st for a, b, st in zip(src, shape, reversed(strides))]
    out = Tensor(shape, t.device(), kFloat32)
    check(_L().sgh_transform_f32(t.ptr, out.ptr, len(shape), (C.c_size_t * len(shape))(*shape),
                                 (C.c_int64 * len(shape))(*strides), t.device().stream), "sgh_transform_f32")
    return out


def _dense_pair(a, b):
    """Operands of an elementwise function as two dense tensors of one shape: what the reference's GPU
    path does with views that are not dense (Transform first, tensor_math_cuda.h:300-362)."""
    a, b = Transform(a), Transform(b)
    if a.shape() == b.shape():
        return a, b
    sa, sb = a.shape(), b.shape()
    n = max(len(sa), len(sb))
    pa, pb = [1] * (n - len(sa)) + sa, [1] * (n - len(sb)) + sb
    if any(x != y and x != 1 and y != 1 for x, y in zip(pa, pb)):
        raise SingaHipError("shapes %s and %s do not broadcast" % (sa, sb))
    shape = [max(x, y) for x, y in zip(pa, pb)]
    return (a if sa == shape else Broadcast(a, shape)), (b if sb == shape else Broadcast(b, shape))


def Clamp(low, high, t):
    """``singa.Clamp`` (autograd.clip): a new tensor with min(max(t, low), high)."""
    _need_f32("Clamp", t)
    out = _like(t)
    check(_L().sgh_clamp_f32(float(low), float(high), t.ptr, out.ptr, t.Size(), t.device().stream), "sgh_clamp_f32")
    return out


def RowMax(t, cpu_rule=False):
    """``singa.RowMax``: the maximum of every row, as the reference's accelerator kernel computes it
    (src/core/tensor/math_kernel.cu:488-499).  ``cpu_rule=True`` (not in the reference signature) gives
    max(0, row maximum), what the reference's CPU function returns (tensor_math_cpp.h:1122-1140)."""
    _need_f32("RowMax", t)
    t = Transform(t)
    if t.nDim() != 2:
        raise SingaHipError("RowMax expects a matrix")
    out = Tensor((t.shape(0),), t.device(), kFloat32)
    name = "sgh_row_max_zero_seeded_f32" if cpu_rule else "sgh_row_max_f32"
    check(getattr(_L(), name)(t.ptr, out.ptr, t.shape(0), t.shape(1), t.device().stream), name)
    return out


def Dot(a, b):
    """``singa.Dot(a, b)`` with a Tensor result: a 1-element tensor on the device."""
    _need_f32("Dot", a, b)
    if a.Size() != b.Size() or a.transpose() or b.transpose():
        raise SingaHipError("Dot expects two dense tensors of one size")
    out, ws = Tensor((1,), a.device(), kFloat32), a.device().reduce_workspace()
    check(_L().sgh_dot_f32(a.ptr, b.ptr, a.Size(), out.ptr, ws.ptr, ws.MemSize(), a.device().stream), "sgh_dot_f32")
    return out


def SumAll(t):
    """``singa.SumAll(t)``: the sum of all elements as a Python float (blocks until it is there)."""
    _need_f32("SumAll", t)
    out, ws = Tensor((1,), t.device(), kFloat32), t.device().reduce_workspace()
    check(_L().sgh_sum_all_f32(t.ptr, t.Size(), out.ptr, ws.ptr, ws.MemSize(), t.device().stream), "sgh_sum_all_f32")
    return float(out.to_numpy()[0])


def Uniform(low, high, t):
    """``singa.Uniform(low, high, t)``: fills `t` from the device's generator state (``SetRandSeed``)."""
    _need_f32("Uniform", t)
    seed, off = t.device()._take_random(t.Size())
    check(_L().sgh_uniform_f32(float(low), float(high), t.ptr, t.Size(), seed, off, t.device().stream), "sgh_uniform_f32")


def Gaussian(mean, std, t):
    """``singa.Gaussian(mean, std, t)``."""
    _need_f32("Gaussian", t)
    seed, off = t.device()._take_random(2 * t.Size())
    check(_L().sgh_gaussian_f32(float(mean), float(std), t.ptr, t.Size(), seed, off, t.device().stream),
          "sgh_gaussian_f32")


def _same(a, b):
    if a.Size() != b.Size() or a.data_type() != b.data_type():
        raise SingaHipError("shape/type mismatch: %s vs %s" % (a.shape(), b.shape()))
    if a.transpose() or b.transpose():
        raise SingaHipError("elementwise ops need contiguous (non-transposed) tensors")


def from_numpy(arr, device):
    arr = np.asarray(arr)
    if arr.dtype == np.float16:
        t = Tensor(arr.shape, device, kFloat16)
        t.CopyHalfDataFromHostPtr(arr)
        return t
    if arr.dtype in (np.int32, np.int64):
        t = Tensor(arr.shape, device, kInt)
        t.CopyIntDataFromHostPtr(arr)
    else:
        t = Tensor(arr.shape, device, kFloat32)
        t.CopyFloatDataFromHostPtr(arr)
    return t


def from_device_pointer(ptr, shape, device, dtype=kFloat32, keepalive=None):
    """Wrap device memory owned by someone else (e.g. a torch tensor; pass it as keepalive)."""
    t = Tensor.__new__(Tensor)
    t._shape = tuple(int(s) for s in shape)
    t._dev = device
    t._dtype = dtype
    t._transposed = False
    t._block = _Block(device, t.Size() * _SIZE_OF[dtype], ptr=int(ptr), keepalive=keepalive)
    return t


def DefaultTranspose(t):
    return t.T()


def Reshape(t, shape):
    return t.Reshape(shape)


# ------------------------------------------------------------------------------------ tensor math

def _like(t):
    return Tensor(t.shape(), t.device(), t.data_type())


def ReLU(x):
    fn, name = _fn("relu_fwd", x)   # (refuses other data types before anything is allocated)
    y = _like(x)
    check(fn(x.ptr, y.ptr, x.Size(), x.device().stream), name)
    return y


def ReLUBackward(dy, x):
    """``singa.ReLUBackward(dy, x)`` (python/singa/autograd.py:432-439)."""
    _same(dy, x)
    fn, name = _fn("relu_bwd", dy)
    dx = _like(dy)
    check(fn(dy.ptr, x.ptr, dx.ptr, dy.Size(), dy.device().stream), name)
    return dx


def ReLUBackwardSum(dy0, dy1, x):
    """``ReLUBackward(dy0 + dy1, x)`` without storing the sum: the fan-in ``+=`` of a residual
    connection (python/singa/autograd.py:204) folded into the ReLU backward that reads it
    (python/singa/autograd.py:432-439); bit-identical to the two steps."""
    _same(dy0, x)
    _same(dy1, x)
    dx = _like(dy0)
    fn, name = _fn("relu_bwd_add", dy0)
    check(fn(dy0.ptr, dy1.ptr, x.ptr, dx.ptr, dy0.Size(), dy0.device().stream), name)
    return dx


def SoftMax(x):
    _need_f32("SoftMax", x)
    batch = x.shape(0) if x.nDim() == 2 else 1
    p = _like(x)
    check(_L().sgh_softmax_fwd_f32(x.ptr, p.ptr, batch, x.Size() // batch, x.device().stream),
          "sgh_softmax_fwd_f32")
    return p


def _ce_dims(p, t, half_ok=False):
    if p.nDim() > 2 or t.nDim() > 2:
        raise SingaHipError("cross entropy expects at most 2-D tensors")
    if not (half_ok and p.data_type() in (kFloat16, kBFloat16)):
        _need_f32("cross entropy", p)
    if t.data_type() != kInt:
        raise SingaHipError("the target tensor must hold int32 (the reference reads it as int)")
    batch = p.shape(0) if p.nDim() == 2 else 1
    dim = p.Size() // batch
    int_target = t.Size() == batch
    if not int_target and t.Size() != p.Size():
        raise SingaHipError("target size matches neither [batch] nor [batch, dim]")
    return batch, dim, int_target


def CrossEntropyFwd(p, t):
    batch, dim, int_target = _ce_dims(p, t)
    loss = Tensor((batch,), p.device(), kFloat32)
    check(_L().sgh_cross_entropy_fwd_f32(p.ptr, t.ptr, loss.ptr, batch, dim, int(int_target),
                                         p.device().stream), "sgh_cross_entropy_fwd_f32")
    return loss


def SoftmaxCrossEntropyBwd(p, t, scale=1.0):
    """``singa.SoftmaxCrossEntropyBwd(p, t)`` (src/core/tensor/tensor.cc:1717-1721): returns a new
    tensor.  ``scale`` (not in the reference signature) fuses the ``dx /= N`` that follows it."""
    batch, dim, int_target = _ce_dims(p, t, half_ok=True)
    g = _like(p)
    fn, name = _fn("softmax_ce_bwd", p)   # 16-bit p: fp32 arithmetic on the stored values, one rounding
    check(fn(p.ptr, t.ptr, g.ptr, batch, dim, int(int_target), float(scale), p.device().stream), name)
    return g


def LabelErrors(device):
    n = C.c_int()
    check(_L().sgh_softmax_ce_label_errors(device.stream, C.byref(n)))
    return n.value


def Axpy(alpha, x, y):
    """``singa.Axpy(alpha, x, y)``: y += alpha * x; alpha is a float or a 1-element device Tensor."""
    _same(x, y)
    if isinstance(alpha, Tensor):
        if alpha.Size() != 1:
            raise SingaHipError("Tensor alpha must have one element")
        _need_f32("Axpy with a Tensor alpha", alpha, x, y)
        check(_L().sgh_axpy_devalpha_f32(alpha.ptr, x.ptr, y.ptr, x.Size(), x.device().stream),
              "sgh_axpy_devalpha_f32")
    else:
        fn, name = _fn("axpy", x)
        check(fn(float(alpha), x.ptr, y.ptr, x.Size(), x.device().stream), name)


def EltwiseMult(a, b, out=None):
    scalar = b.Size() == 1 and a.Size() != 1
    if not scalar and a.data_type() == kFloat32 and (a.shape() != b.shape() or a.transpose() or b.transpose()):
        a, b = _dense_pair(a, b)     # broadcast / transposed operands
    out = _like(a) if out is None else out
    if not scalar:
        _same(a, b)
    if a.data_type() != kFloat32:
        if scalar:
            raise SingaHipError("scalar EltwiseMult is fp32 only")
        fn, name = _fn("eltwise_mult", a)
        check(fn(a.ptr, b.ptr, out.ptr, a.Size(), a.device().stream), name)
        return out
    check(_L().sgh_eltwise_mult_f32(a.ptr, b.ptr, int(scalar), out.ptr, a.Size(), a.device().stream),
          "sgh_eltwise_mult_f32")
    return out


def __add__(a, b):
    if a.data_type() == kFloat32 and (a.shape() != b.shape() or a.transpose() or b.transpose()):
        a, b = _dense_pair(a, b)     # broadcast / transposed operands
    _same(a, b)
    out = _like(a)
    fn, name = _fn("add", a)
    check(fn(a.ptr, b.ptr, out.ptr, a.Size(), a.device().stream), name)
    return out


def AddReLU(a, b):
    """``relu(a + b)`` in one pass, the end of a residual block's forward (examples/cnn/model/resnet.py:74-77):
    the bits ``ReLU(a + b)`` stores."""
    _same(a, b)
    out = _like(a)
    fn, name = _fn("add_relu", a)
    check(fn(a.ptr, b.ptr, out.ptr, a.Size(), a.device().stream), name)
    return out


def _binary_f32(name, a, b):
    _same(a, b)
    if a.data_type() != kFloat32:
        raise SingaHipError(name + " is an fp32 function")
    out = _like(a)
    check(getattr(_L(), name)(a.ptr, b.ptr, out.ptr, a.Size(), a.device().stream), name)
    return out


def _scalar_f32(name, a, x):
    if a.data_type() != kFloat32:
        raise SingaHipError(name + " is an fp32 function")
    out = _like(a)
    check(getattr(_L(), name)(a.ptr, float(x), out.ptr, a.Size(), a.device().stream), name)
    return out


def __sub__(a, b):
    """``singa.__sub__`` (Sub, src/core/tensor/tensor_math_cpp.h:645-650)."""
    return _binary_f32("sgh_sub_f32", a, b)


def __div__(a, b):
    """``singa.__div__`` (tensor / tensor, src/core/tensor/tensor_math_cpp.h:423-430)."""
    return _binary_f32("sgh_div_f32", a, b)


def AddFloat(t, x):
    """``singa.AddFloat`` (tensor + scalar, src/core/tensor/tensor_math_cpp.h:383-388)."""
    return _scalar_f32("sgh_add_scalar_f32", t, x)


def MultFloat(t, x):
    """``singa.MultFloat`` (tensor * scalar, src/core/tensor/tensor_math_cpp.h:432-437)."""
    return _scalar_f32("sgh_mult_scalar_f32", t, x)


def DivFloat(t, x):
    """``singa.DivFloat``: the reference multiplies by the fp32 reciprocal
    (include/singa/core/tensor.h Div -> src/core/tensor/tensor_math.h:149-153)."""
    return _scalar_f32("sgh_mult_scalar_f32", t, np.float32(1.0) / np.float32(x))


def Mult(A, B):
    """``singa.Mult(A, B)`` for 2-D tensors (src/core/tensor/tensor.cc:1633-1706): the transpose
    flags of the views select the GEMM variant, no data is moved."""
    if A.nDim() != 2 or B.nDim() != 2 or A.shape(1) != B.shape(0):
        raise SingaHipError("Mult shape mismatch %s x %s" % (A.shape(), B.shape()))
    if A.data_type() != B.data_type():
        raise SingaHipError("Mult: operands differ in data type")
    fn, name = _fn("gemm", A)   # 16-bit operands: the 16-bit matrix instructions, fp32 accumulation, one rounding
    M, K, N = A.shape(0), A.shape(1), B.shape(1)
    out = Tensor((M, N), A.device(), A.data_type())
    tA, tB = A.transpose(), B.transpose()
    lda = M if tA else K
    ldb = K if tB else N
    check(fn(int(tA), int(tB), M, N, K, 1.0, A.ptr, lda, B.ptr, ldb, 0.0, out.ptr, N, A.device().stream), name)
    return out


def Sum(t, axis):
    """``singa.Sum(t, 0)`` of a 2-D tensor: column sums (bias gradient of AddBias)."""
    if t.nDim() != 2 or axis != 0 or t.transpose():
        raise SingaHipError("only Sum(2-D tensor, 0) is on the backward path")
    _need_f32("Sum", t)
    out = Tensor((t.shape(1),), t.device(), kFloat32)
    check(_L().sgh_sum_rows_f32(t.ptr, out.ptr, t.shape(0), t.shape(1), t.device().stream), "sgh_sum_rows_f32")
    return out


def AddRow(v, m):
    _need_f32("AddRow", v, m)
    check(_L().sgh_add_row_f32(v.ptr, m.ptr, m.shape(0), m.shape(1), m.device().stream), "sgh_add_row_f32")


# ------------------------------------------------------------------------------------ operations

class CudnnConvHandle(object):
    """Geometry + workspace of a convolution on the GPU device.  Same constructor arguments and
    public fields as the reference's handle (src/model/operation/convolution.h:43-129; fields read
    from Python: src/api/model_operation.i:37-54)."""

    def __init__(self, x, kernel_size, stride, padding, in_channels, out_channels, bias, groups=1,
                 workspace_byte_limit=1024 * 1024 * 1024, prefer="fastest"):
        groups = int(groups)
        if groups < 1 or in_channels % groups != 0 or out_channels % groups != 0:
            raise SingaHipError("channels and filters must be multiples of the group count")
        if x.nDim() != 4 or x.shape(1) != in_channels:
            raise SingaHipError("the number of input channels mismatched.")
        self.kernel_h, self.kernel_w = int(kernel_size[0]), int(kernel_size[1])
        self.stride_h, self.stride_w = int(stride[0]), int(stride[1])
        self.pad_h, self.pad_w = int(padding[0]), int(padding[1])
        self.channels, self.num_filters = int(in_channels), int(out_channels)
        self.group = groups
        self.bias_term = bool(bias)
        self.batchsize, _, self.height, self.width = x.shape()
        self.geom = _lib.ConvGeom()
        check(_L().sgh_conv_geom_init_grouped(C.byref(self.geom), self.batchsize, self.channels, self.height,
                                              self.width, self.num_filters, self.kernel_h, self.kernel_w,
                                              self.stride_h, self.stride_w, self.pad_h, self.pad_w, groups),
              "sgh_conv_geom_init_grouped")
        self.channels_per_filter = self.channels // groups   # (convolution.cc:461)
        self.conv_height, self.conv_width = self.geom.P, self.geom.Q
        self.col_height = self.channels * self.kernel_h * self.kernel_w
        self.col_width = self.conv_height * self.conv_width
        self.imagesize = x.Size() // self.batchsize
        # a handle built from a 16-bit input runs every pass on 16-bit tensors (convolution.cc:444-572)
        self.dtype = x.data_type()
        ws_fn = _L().sgh_conv_workspace_bytes if self.dtype == kFloat32 else _L().sgh_conv_workspace_bytes_h
        need = max(ws_fn(C.byref(self.geom), w) for w in (0, 1, 2))
        if need > workspace_byte_limit:
            raise SingaHipError("workspace of %d bytes exceeds the limit" % need)
        self.workspace_count = need // 4
        self.workspace = Tensor((max(self.workspace_count, 1),), x.device(), kFloat32)
        self.wgrad_workspace = None   # a second one, made when a weight gradient runs on the auxiliary stream

    def _check_x(self, x):
        if x.shape() != [self.batchsize, self.channels, self.height, self.width]:
            raise SingaHipError("input sample shape should not change")

    def _check_dy(self, dy):
        if dy.shape() != [self.batchsize, self.num_filters, self.conv_height, self.conv_width]:
            raise SingaHipError("dy shape does not match the handle")


def GpuConvForward(x, W, b, h):
    h._check_x(x)
    y = Tensor((h.batchsize, h.num_filters, h.conv_height, h.conv_width), x.device(), x.data_type())
    bias = b.ptr if (h.bias_term and b is not None) else None
    fn, name = _fn("conv_fwd", x)
    check(fn(C.byref(h.geom), x.ptr, W.ptr, bias, y.ptr, h.workspace.ptr, h.workspace.MemSize(),
             x.device().stream), name)
    return y


def GpuConvBackwardxAccumulate(dy, W, x, h, dx):
    """``dx += GpuConvBackwardx(dy, W, x, h)`` in place, returning ``dx``: the gradient fan-in of a
    residual connection (``+=``, python/singa/autograd.py:204) folded into the store of the data
    gradient where the kernel supports it, otherwise the two separate steps."""
    h._check_dy(dy)
    _same(dx, x)
    if dy.data_type() == kFloat32:   # (on 16-bit tensors the kernel's read-modify-write loses to the separate add)
        rc = _L().sgh_conv_dgrad_acc_f32(C.byref(h.geom), dy.ptr, W.ptr, dx.ptr, h.workspace.ptr,
                                         h.workspace.MemSize(), dy.device().stream)
        if rc != _lib.SGH_EUNSUPPORTED:
            check(rc, "sgh_conv_dgrad_acc_f32")
            return dx
    dx += GpuConvBackwardx(dy, W, x, h)
    return dx


def GpuConvBackwardx(dy, W, x, h):
    h._check_dy(dy)
    dx = _like(x)
    fn, name = _fn("conv_dgrad", dy)
    check(fn(C.byref(h.geom), dy.ptr, W.ptr, dx.ptr, h.workspace.ptr, h.workspace.MemSize(),
             dy.device().stream), name)
    return dx


def GpuConvBackwardW(dy, x, W, h, stream=None, out=None):
    """`stream`: None = the device's stream.  Another stream (``HipGPU.Fork()``) runs the weight
    gradient beside whatever the main stream does next; it then works in a workspace of its own
    (``h.wgrad_workspace``); dy, x, the result and that workspace are announced to the pool
    (``HipGPU.UsedOn``), so the caller may drop them whenever it likes.  `out`: the tensor that
    receives the result (a caller that handed it out before the kernel was enqueued)."""
    h._check_dy(dy)
    h._check_x(x)
    dW = _like(W) if out is None else out
    fn, name = _fn("conv_wgrad", dy)
    ws = h.workspace
    if stream is not None:
        if h.wgrad_workspace is None:
            which = _lib.SGH_CONV_WGRAD
            need = (_L().sgh_conv_workspace_bytes(C.byref(h.geom), which) if dy.data_type() == kFloat32
                    else _L().sgh_conv_workspace_bytes_h(C.byref(h.geom), which))
            h.wgrad_workspace = Tensor(((max(need, 4) + 3) // 4,), dy.device(), kFloat32)
        ws = h.wgrad_workspace
        dy.device().UsedOn(stream, dy, x, dW, ws)
    check(fn(C.byref(h.geom), dy.ptr, x.ptr, dW.ptr, ws.ptr, ws.MemSize(),
             dy.device().stream if stream is None else stream), name)
    return dW


def GpuConvBackwardWb(dy, x, W, b, h):
    """``GpuConvBackwardW`` and ``GpuConvBackwardb`` of one layer in one call: ``(dW, db)``.  Where the
    generic kernel computes the weight gradient the bias gradient rides along in its matrix
    instructions and dy is read once (fp32 tensors; other types make the two calls)."""
    if dy.data_type() != kFloat32:
        return GpuConvBackwardW(dy, x, W, h), GpuConvBackwardb(dy, b, h)
    h._check_dy(dy)
    h._check_x(x)
    dW, db = _like(W), _like(b)
    ws = h.workspace
    check(_L().sgh_conv_wgrad_bias_f32(C.byref(h.geom), dy.ptr, x.ptr, dW.ptr, db.ptr, ws.ptr, ws.MemSize(),
                                       dy.device().stream), "sgh_conv_wgrad_bias_f32")
    return dW, db


def GpuConvPrepareBackward(weights_and_handles):
    """Re-lays the weights of all listed convolutions for their data gradients in ONE launch (the
    re-layout each ``GpuConvBackwardx`` otherwise launches for itself); `weights_and_handles`: pairs
    ``(W, handle)``.  Each handle's next ``GpuConvBackwardx`` uses the prepared weights if nothing
    that may change a weight tensor (an update, Axpy, a fill, an upload) was called in between and no
    other pass wrote the handle's workspace; otherwise it re-lays them itself.  Results are
    bit-identical with and without."""
    pairs = list(weights_and_handles)
    if not pairs:
        return
    W0 = pairs[0][0]
    arr = (_lib.ConvPrepareItem * len(pairs))()
    for i, (W, h) in enumerate(pairs):
        if W.data_type() != W0.data_type():
            raise SingaHipError("one weight type per GpuConvPrepareBackward call")
        arr[i].g, arr[i].W = C.pointer(h.geom), W.ptr
        arr[i].workspace, arr[i].ws_bytes = h.workspace.ptr, h.workspace.MemSize()
    dtype = {kFloat32: 0, kFloat16: 1, kBFloat16: 2}[W0.data_type()]
    check(_L().sgh_conv_dgrad_prepare_multi(arr, len(pairs), dtype, W0.device().stream), "sgh_conv_dgrad_prepare_multi")


def ConvWeightsChanged():
    """For a caller that writes weight tensors by means this library cannot see: prepared weights
    (``GpuConvPrepareBackward``) are not used after this call."""
    _L().sgh_conv_weights_changed()


def GpuConvBackwardb(dy, b, h):
    h._check_dy(dy)
    db = _like(b)
    fn, name = _fn("conv_bgrad", dy)
    check(fn(C.byref(h.geom), dy.ptr, db.ptr, dy.device().stream), name)
    return db


class CudnnBatchNormHandle(object):
    """``CudnnBatchNormHandle(momentum, x)`` (src/model/operation/batchnorm.h:49-101)."""

    def __init__(self, momentum, x):
        self.factor = float(momentum)
        self.is_2d = x.nDim() == 2
        if self.is_2d:
            self.batchsize, self.channels = x.shape()
            self.height = self.width = 1
        elif x.nDim() == 4:
            self.batchsize, self.channels, self.height, self.width = x.shape()
        else:
            raise SingaHipError("BatchNorm expects a 2-D or 4-D input")
        hw = self.height * self.width
        nbytes = _L().sgh_bn_workspace_bytes(self.batchsize, self.channels, hw)
        self.workspace = Tensor((max(nbytes // 4, 1),), x.device(), kFloat32)


_BN_EPS = 1e-5  # CUDNN_BN_MIN_EPSILON, src/model/operation/batchnorm.cc:313


def GpuBatchNormForwardTraining(h, x, scale, bias, running_mean, running_var):
    """Returns ``[y, mean, var]`` where ``var`` holds the saved inverse standard deviation, and
    updates the running statistics in place (src/model/operation/batchnorm.cc:287-329)."""
    y = _like(x)
    mean = Tensor((h.channels,), x.device(), kFloat32)
    var = Tensor((h.channels,), x.device(), kFloat32)
    fn, name = _fn("bn_fwd_train", x)  # 16-bit activations keep fp32 scale / bias / statistics
    check(fn(x.ptr, scale.ptr, bias.ptr,
             running_mean.ptr if running_mean is not None else None,
             running_var.ptr if running_var is not None else None,
             h.factor, _BN_EPS, y.ptr, mean.ptr, var.ptr, h.batchsize, h.channels,
             h.height * h.width, h.workspace.ptr, h.workspace.MemSize(), x.device().stream), name)
    return [y, mean, var]


def GpuBatchNormReLUForwardTraining(h, x, scale, bias, running_mean, running_var):
    """``GpuBatchNormForwardTraining`` with the ReLU that follows folded in: ``[relu(y), mean, var]``, the bits
    ``ReLU(GpuBatchNormForwardTraining(...)[0])`` stores (conv -> BatchNorm -> ReLU, examples/cnn/model/resnet.py:54-60)."""
    y = _like(x)
    mean = Tensor((h.channels,), x.device(), kFloat32)
    var = Tensor((h.channels,), x.device(), kFloat32)
    fn, name = _fn("bn_relu_fwd_train", x)
    check(fn(x.ptr, scale.ptr, bias.ptr,
             running_mean.ptr if running_mean is not None else None,
             running_var.ptr if running_var is not None else None,
             h.factor, _BN_EPS, y.ptr, mean.ptr, var.ptr, h.batchsize, h.channels,
             h.height * h.width, h.workspace.ptr, h.workspace.MemSize(), x.device().stream), name)
    return [y, mean, var]


def GpuBatchNormAddReLUForwardTraining(h, x, z, scale, bias, running_mean, running_var):
    """``[relu(BatchNorm(x) + z), mean, var]``: the forward of ``relu(bn(..) + identity)`` at the end of a residual block
    (examples/cnn/model/resnet.py:70-77) in one call, the bits the three separate calls store."""
    _same(x, z)
    y = _like(x)
    mean = Tensor((h.channels,), x.device(), kFloat32)
    var = Tensor((h.channels,), x.device(), kFloat32)
    fn, name = _fn("bn_add_relu_fwd_train", x)
    check(fn(x.ptr, z.ptr, scale.ptr, bias.ptr,
             running_mean.ptr if running_mean is not None else None,
             running_var.ptr if running_var is not None else None,
             h.factor, _BN_EPS, y.ptr, mean.ptr, var.ptr, h.batchsize, h.channels,
             h.height * h.width, h.workspace.ptr, h.workspace.MemSize(), x.device().stream), name)
    return [y, mean, var]


def GpuBatchNormForwardInference(h, x, scale, bias, running_mean, running_var):
    """``y`` normalised with the running statistics (src/model/operation/batchnorm.cc:331-366)."""
    y = _like(x)
    fn, name = _fn("bn_fwd_infer", x)
    check(fn(x.ptr, scale.ptr, bias.ptr, running_mean.ptr, running_var.ptr, _BN_EPS, y.ptr, h.batchsize, h.channels,
             h.height * h.width, x.device().stream), name)
    return y


def GpuBatchNormBackward(h, dy, x, scale, mean, var):
    """Returns ``[dx, dscale, dbias]`` (src/model/operation/batchnorm.cc:368-404)."""
    _same(dy, x)
    dx = _like(dy)
    ds = _like(scale)
    db = _like(scale)
    fn, name = _fn("bn_bwd", dy)
    check(fn(dy.ptr, x.ptr, scale.ptr, mean.ptr, var.ptr, dx.ptr, ds.ptr, db.ptr,
             h.batchsize, h.channels, h.height * h.width, h.workspace.ptr,
             h.workspace.MemSize(), dy.device().stream), name)
    return [dx, ds, db]


def GpuBatchNormReLUBackward(h, dy, x, scale, bias, mean, var):
    """``GpuBatchNormBackward(h, ReLUBackward(dy, y), x, scale, mean, var)`` for ``y`` = this
    BatchNorm's output, in one pass: ``y`` is recomputed from ``x`` instead of being read, and the
    ReLU's gradient is never written (the conv -> BatchNorm -> ReLU tape of
    examples/cnn/model/resnet.py:54-60).  Returns ``[dx, dscale, dbias]``."""
    _same(dy, x)
    dx = _like(dy)
    ds = _like(scale)
    db = _like(scale)
    fn, name = _fn("bn_relu_bwd", dy)
    check(fn(dy.ptr, x.ptr, scale.ptr, bias.ptr, mean.ptr, var.ptr, dx.ptr, ds.ptr, db.ptr,
             h.batchsize, h.channels, h.height * h.width, h.workspace.ptr,
             h.workspace.MemSize(), dy.device().stream), name)
    return [dx, ds, db]


class CudnnPoolingHandle(object):
    """``CudnnPoolingHandle(x, kernel, stride, padding, is_max)``
    (src/model/operation/pooling.h:40-91)."""

    def __init__(self, x, kernel_size, stride, padding, is_max=True):
        if x.nDim() != 4:
            raise SingaHipError("pooling expects a 4-D input")
        self.kernel_h, self.kernel_w = int(kernel_size[0]), int(kernel_size[1])
        self.stride_h, self.stride_w = int(stride[0]), int(stride[1])
        self.pad_h, self.pad_w = int(padding[0]), int(padding[1])
        self.batchsize, self.channels, self.height, self.width = x.shape()
        self.is_max_pooling = bool(is_max)
        self.geom = _lib.PoolGeom()
        check(_L().sgh_pool_geom_init(C.byref(self.geom), self.batchsize, self.channels, self.height,
                                      self.width, self.kernel_h, self.kernel_w, self.stride_h, self.stride_w,
                                      self.pad_h, self.pad_w, int(self.is_max_pooling)), "sgh_pool_geom_init")
        self.pooled_height, self.pooled_width = self.geom.P, self.geom.Q


def GpuPoolingForward(h, x):
    y = Tensor((h.batchsize, h.channels, h.pooled_height, h.pooled_width), x.device(), x.data_type())
    fn, name = _fn("pool_fwd", x)
    check(fn(C.byref(h.geom), x.ptr, y.ptr, x.device().stream), name)
    return y


def GpuPoolingBackward(h, dy, x, y):
    if dy.shape() != [h.batchsize, h.channels, h.pooled_height, h.pooled_width]:
        raise SingaHipError("dy shape does not match the handle")
    if dy.data_type() != x.data_type():
        raise SingaHipError("dy and x differ in data type")
    dx = _like(x)
    fn, name = _fn("pool_bwd", x)
    check(fn(C.byref(h.geom), dy.ptr, x.ptr, y.ptr if y is not None else None, dx.ptr, dy.device().stream), name)
    return dx
