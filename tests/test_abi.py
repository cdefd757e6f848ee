"""The C-ABI library loads without a GPU and exports every symbol include/singa_hip.h declares;
host-only entry points (geometry, sizes, error strings) behave as documented."""
import ctypes as C
import os
import re

import pytest

from singa_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "singa_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"SGH_API\s+[\w\s\*]+?\b(sgh_\w+)\s*\(", text)))


def test_header_and_binding_agree():
    decl = declared_symbols()
    assert len(decl) >= 40
    assert sorted(_lib.SIGNATURES) == decl


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(_lib.LIBPATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_error_strings_and_identity():
    lib = _lib.lib()
    assert lib.sgh_arch() == b"gfx950"
    assert lib.sgh_error_string(0) == b"ok"
    assert b"workspace" in lib.sgh_error_string(-2)
    assert b"invalid" in lib.sgh_error_string(-1)


def test_conv_geometry_follows_reference_integer_division():
    lib = _lib.lib()
    g = _lib.ConvGeom()
    # 7x7 stride 2 pad 3 on 224 -> 112 ; 3x3 stride 2 pad 1 on 56 -> 28 ; 1x1 stride 2 on 56 -> 28
    for (H, R, s, p, P) in [(224, 7, 2, 3, 112), (56, 3, 2, 1, 28), (56, 1, 2, 0, 28), (3, 3, 2, 1, 2), (8, 3, 3, 1, 3)]:
        assert lib.sgh_conv_geom_init(C.byref(g), 2, 3, H, H, 4, R, R, s, s, p, p) == 0
        assert (g.P, g.Q) == (P, P)
    assert lib.sgh_conv_geom_init(C.byref(g), 2, 3, 2, 2, 4, 5, 5, 1, 1, 0, 0) == -1  # kernel larger than padded input
    assert lib.sgh_conv_geom_init(C.byref(g), 0, 3, 8, 8, 4, 3, 3, 1, 1, 0, 0) == -1
    assert lib.sgh_conv_geom_init(None, 1, 3, 8, 8, 4, 3, 3, 1, 1, 0, 0) == -1


def test_workspace_sizes():
    lib = _lib.lib()
    g = _lib.ConvGeom()
    assert lib.sgh_conv_geom_init(C.byref(g), 64, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1) == 0
    # re-laid weights (256-byte aligned) + partial tiles of the workgroups that share the last
    # wave of tiles: at most two slots of one 128x128 tile for each of 2 * (CU count) workgroups
    dg = lib.sgh_conv_workspace_bytes(C.byref(g), _lib.SGH_CONV_DGRAD)
    assert 9 * 64 * 64 * 4 <= dg <= 9 * 64 * 64 * 4 + 2 * 1024 * 2 * 128 * 128 * 4 and dg % 256 == 0
    fw = lib.sgh_conv_workspace_bytes(C.byref(g), _lib.SGH_CONV_FWD)   # same kernel, same bound
    assert 9 * 64 * 64 * 4 <= fw <= 9 * 64 * 64 * 4 + 2 * 1024 * 2 * 128 * 128 * 4
    w = lib.sgh_conv_workspace_bytes(C.byref(g), _lib.SGH_CONV_WGRAD)
    assert w % (64 * 64 * 9 * 4) == 0  # whole split-K partial copies of dW
    assert lib.sgh_bn_workspace_bytes(64, 64, 56 * 56) >= 64 * 2 * 4
    assert lib.sgh_bn_workspace_bytes(0, 64, 49) == 0


def test_prepare_multi_argument_checks_and_geometry_flag():
    lib = _lib.lib()
    g = _lib.ConvGeom()
    g.weights_prelaid = 7
    assert lib.sgh_conv_geom_init(C.byref(g), 8, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1) == 0
    assert g.weights_prelaid == 0                       # a fresh geometry never claims prepared weights
    items = (_lib.ConvPrepareItem * 1)()
    assert lib.sgh_conv_dgrad_prepare_multi(items, -1, 0, None) == -1
    assert lib.sgh_conv_dgrad_prepare_multi(None, 1, 0, None) == -1
    assert lib.sgh_conv_dgrad_prepare_multi(items, 1, 3, None) == -1      # unknown data type
    assert lib.sgh_conv_dgrad_prepare_multi(items, 1, 0, None) == -1      # item without geometry / weights
    assert lib.sgh_conv_dgrad_prepare_multi(items, 0, 0, None) == 0       # nothing to do


def test_16bit_conv_workspace_covers_every_pass():
    lib = _lib.lib()
    g = _lib.ConvGeom()
    for (Cc, H, K, R, s, p) in [(64, 56, 64, 3, 1, 1), (256, 56, 512, 1, 2, 0), (128, 56, 128, 3, 2, 1), (3, 224, 64, 7, 2, 3)]:
        assert lib.sgh_conv_geom_init(C.byref(g), 4, Cc, H, H, K, R, R, s, s, p, p) == 0
        for which in (_lib.SGH_CONV_FWD, _lib.SGH_CONV_DGRAD, _lib.SGH_CONV_WGRAD):
            b = lib.sgh_conv_workspace_bytes_h(C.byref(g), which)
            assert b > 0 and b % 256 == 0, (Cc, H, K, R, s, which, b)
    assert lib.sgh_conv_workspace_bytes_h(C.byref(g), 3) == 0


def test_pool_geometry():
    lib = _lib.lib()
    g = _lib.PoolGeom()
    assert lib.sgh_pool_geom_init(C.byref(g), 64, 64, 112, 112, 3, 3, 2, 2, 1, 1, 1) == 0
    assert (g.P, g.Q) == (56, 56)
    assert lib.sgh_pool_geom_init(C.byref(g), 64, 64, 7, 7, 7, 7, 1, 1, 0, 0, 0) == 0
    assert (g.P, g.Q) == (1, 1)
    # a pad as large as the kernel would make windows that see no input
    assert lib.sgh_pool_geom_init(C.byref(g), 1, 1, 4, 4, 2, 2, 1, 1, 2, 2, 1) == -1


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(_lib.SingaHipError):
        _lib.load(str(tmp_path / "nope.so"))


def test_fp32_only_wrappers_check_the_data_type_before_any_call():
    """A 16-bit tensor handed to a function that only exists for float32 is refused on the host
    (the kernel would read twice the tensor's bytes).  Needs no GPU: the check comes first."""
    import pytest
    from singa_amd import singa_wrap as singa

    class _NoDevice(object):
        stream = None

    t = singa.from_device_pointer(0x1000, (4, 8), _NoDevice(), singa.kFloat16)
    for call in (lambda: singa.ReLU(t), lambda: singa.SoftMax(t), lambda: singa.Mult(t, t.T()), lambda: singa.Sum(t, 0),
                 lambda: singa.AddRow(t, t), lambda: t.__imul__(2.0)):
        with pytest.raises(singa.SingaHipError, match="float32"):
            call()
