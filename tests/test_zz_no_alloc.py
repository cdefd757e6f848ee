"""GPU parity of the entry point that allocates nothing: ``sgh_bn_bwd_noalloc_f32`` against
``sgh_bn_bwd_f32`` (bit for bit: same kernels, the partial sums in the library's own buffer instead
of a workspace) and against the CPU oracle (normalised L2 <= 1e-3), on two calls in a row, the
second on a smaller input, so that what the first call left in the shared buffer is there when the
second runs.  Runs last (file name) and must pass alone in a fresh process as well."""
import numpy as np
import pytest

from oracle import cpu_oracle as O
from util import assert_bit_equal, nl2, randn, rng

pytestmark = pytest.mark.gpu

TOL = 1e-3


def _case(singa, dev, shape, seed):
    from singa_amd._lib import check, lib
    r = rng(seed)
    N, C, H, W = shape
    x = (randn(r, *shape) * 1.5 - 0.3).astype(np.float32)
    dy = randn(r, *shape)
    gamma = (randn(r, C) * 0.2 + 1).astype(np.float32)
    mean = x.mean(axis=(0, 2, 3)).astype(np.float32)
    inv = (1.0 / np.sqrt(x.var(axis=(0, 2, 3)) + 1e-5)).astype(np.float32)
    xd, dyd, gd = singa.from_numpy(x, dev), singa.from_numpy(dy, dev), singa.from_numpy(gamma, dev)
    md, vd = singa.from_numpy(mean, dev), singa.from_numpy(inv, dev)
    # the existing entry point, with its workspace
    h = singa.CudnnBatchNormHandle(0.9, xd)
    dx0, dg0, db0 = singa.GpuBatchNormBackward(h, dyd, xd, gd, md, vd)
    # the non-allocating one: outputs are the caller's, nothing else is passed
    dx1, dg1, db1 = singa.Tensor(shape, dev), singa.Tensor((C,), dev), singa.Tensor((C,), dev)
    for t in (dx1, dg1, db1):
        t.SetFloatValue(-77.0)
    print("sgh_bn_bwd_noalloc_f32 shape", shape, "seed", seed, flush=True)
    check(lib().sgh_bn_bwd_noalloc_f32(dyd.ptr, xd.ptr, gd.ptr, md.ptr, vd.ptr, dx1.ptr, dg1.ptr, db1.ptr,
                                       N, C, H * W, dev.stream), "sgh_bn_bwd_noalloc_f32")
    assert_bit_equal(dx1.to_numpy(), dx0.to_numpy(), "dx")
    assert_bit_equal(dg1.to_numpy(), dg0.to_numpy(), "dgamma")
    assert_bit_equal(db1.to_numpy(), db0.to_numpy(), "dbeta")
    dx_o, dg_o, db_o = O.bn_bwd(dy, x, gamma, mean, inv)
    e = (nl2(dx1.to_numpy(), dx_o), nl2(dg1.to_numpy(), dg_o), nl2(db1.to_numpy(), db_o))
    assert max(e) < TOL, e


def test_no_alloc_bn_bwd_two_calls_in_a_row(dev):
    from singa_amd import singa_wrap as singa
    # channels cut into slices (one-pass kernel, partial sums and tickets through the library's buffer),
    # then a smaller input with fewer channels and slices, then an odd plane (two-pass kernels, scalar path),
    # then the first shape again over what the others left in the buffer
    _case(singa, dev, (8, 48, 28, 28), 1)
    _case(singa, dev, (4, 16, 12, 12), 2)
    _case(singa, dev, (3, 5, 7, 5), 3)
    _case(singa, dev, (8, 48, 28, 28), 4)


def test_no_alloc_bn_bwd_recorded_calls_of_two_shapes(dev):
    """The callers this entry point is for record it into graphs: two recorded calls of different shapes share
    the library's buffer (the second overwrites some of the first one's exchange words and not others); every
    replay stores the bits of the eager calls."""
    from singa_amd import singa_wrap as singa
    from singa_amd._lib import check, lib
    shapes = [(8, 48, 28, 28), (16, 20, 20, 20)]
    cases = []
    for k, shape in enumerate(shapes):
        r = rng(40 + k)
        N, C, H, W = shape
        x = (randn(r, *shape) * 1.5 - 0.3).astype(np.float32)
        host = [randn(r, *shape), x, (randn(r, C) * 0.2 + 1).astype(np.float32), x.mean(axis=(0, 2, 3)).astype(np.float32),
                (1.0 / np.sqrt(x.var(axis=(0, 2, 3)) + 1e-5)).astype(np.float32)]
        ins = [singa.from_numpy(a, dev) for a in host]
        outs = [singa.Tensor(shape, dev), singa.Tensor((C,), dev), singa.Tensor((C,), dev)]
        cases.append((shape, ins, outs))

    def call_all():
        for (N, C, H, W), ins, outs in cases:
            check(lib().sgh_bn_bwd_noalloc_f32(*[t.ptr for t in ins], *[t.ptr for t in outs], N, C, H * W, dev.stream),
                  "sgh_bn_bwd_noalloc_f32")

    print("sgh_bn_bwd_noalloc_f32 recorded, shapes", shapes, flush=True)
    call_all()
    want = [[t.to_numpy() for t in outs] for _, _, outs in cases]
    dev.Sync()
    dev.EnableGraph(True)
    call_all()
    dev.EnableGraph(False)
    try:
        for i in range(4):
            for _, _, outs in cases:
                for t in outs:
                    t.SetFloatValue(-77.0)
            dev.RunGraph()
            if i == 1:
                call_all()   # eager calls between replays
            for (shape, _, outs), w in zip(cases, want):
                for t, a, what in zip(outs, w, ("dx", "dgamma", "dbeta")):
                    assert_bit_equal(t.to_numpy(), a, "%s of %r, replay %d" % (what, shape, i))
    finally:
        dev.ResetGraph()


def test_no_alloc_bn_bwd_rejects_sizes_beyond_its_buffer(dev):
    from singa_amd import singa_wrap as singa
    from singa_amd._lib import SGH_ELIMIT, lib
    C = 40000      # 8 bytes of partial sums per channel: beyond the 256 KiB the library holds
    t = singa.Tensor((1, C, 1, 1), dev)
    t.SetFloatValue(0.0)
    v = singa.Tensor((C,), dev)
    v.SetFloatValue(1.0)
    rc = lib().sgh_bn_bwd_noalloc_f32(t.ptr, t.ptr, v.ptr, v.ptr, v.ptr, t.ptr, v.ptr, v.ptr, 1, C, 1, dev.stream)
    assert rc == SGH_ELIMIT
    assert b"non-allocating" in lib().sgh_error_string(rc)
