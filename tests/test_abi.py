"""The C-ABI library loads without a GPU and exports every symbol include/singa_hip.h declares;
host-only entry points (geometry, sizes, error strings) behave as documented."""
import ctypes as C
import os
import re
import subprocess

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


def test_grouped_conv_geometry():
    """sgh_conv_geom_init_grouped: channel and filter counts must be multiples of the group count; the workspace
    of a grouped layer holds one group's slices of x and y next to the sub-geometry's own workspace."""
    lib = _lib.lib()
    g, d = _lib.ConvGeom(), _lib.ConvGeom()
    assert lib.sgh_conv_geom_init(C.byref(d), 4, 16, 14, 14, 32, 3, 3, 1, 1, 1, 1) == 0 and d.groups == 1
    assert lib.sgh_conv_geom_init_grouped(C.byref(g), 4, 64, 14, 14, 128, 3, 3, 1, 1, 1, 1, 4) == 0
    assert (g.groups, g.C, g.K, g.P, g.Q) == (4, 64, 128, 14, 14)
    for bad in (0, -1, 3, 5, 128):
        assert lib.sgh_conv_geom_init_grouped(C.byref(g), 4, 64, 14, 14, 128, 3, 3, 1, 1, 1, 1, bad) == -1
    assert lib.sgh_conv_geom_init_grouped(C.byref(g), 4, 64, 14, 14, 128, 3, 3, 1, 1, 1, 1, 4) == 0
    for which in (_lib.SGH_CONV_FWD, _lib.SGH_CONV_DGRAD, _lib.SGH_CONV_WGRAD):
        slices = 4 * 16 * 14 * 14 + 4 * 32 * 14 * 14
        for fn, es in ((lib.sgh_conv_workspace_bytes, 4), (lib.sgh_conv_workspace_bytes_h, 2)):
            got, sub = fn(C.byref(g), which), fn(C.byref(d), which)
            assert slices * es + sub <= got <= slices * es + sub + 512
    g.groups = 3     # a geometry whose fields were edited by hand is refused
    assert lib.sgh_conv_workspace_bytes(C.byref(g), 0) == 0


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
    g.prelaid_W, g.prelaid_ws, g.prelaid_epoch = 0x1000, 0x2000, 1
    assert lib.sgh_conv_geom_init(C.byref(g), 8, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1) == 0
    assert not g.prelaid_W and not g.prelaid_ws and g.prelaid_epoch == 0   # a fresh geometry never claims prepared weights
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
    for call in (lambda: singa.SoftMax(t), lambda: singa.Sum(t, 0), lambda: singa.AddRow(t, t), lambda: t.__imul__(2.0)):
        with pytest.raises(singa.SingaHipError, match="float32"):
            call()
    # functions that exist for float32 and the 16-bit types refuse an int tensor the same way
    i = singa.from_device_pointer(0x1000, (4, 8), _NoDevice(), singa.kInt)
    for call in (lambda: singa.ReLU(i), lambda: singa.Mult(i, i.T()), lambda: singa.ReLUBackward(i, i)):
        with pytest.raises(singa.SingaHipError, match="unsupported data type"):
            call()


# ---- the header as a C and as a C++ translation unit, and the binding's argument lists against it

def _prototypes():
    """{name: (return type text, [argument type texts])} from the header's SGH_API declarations."""
    text = open(os.path.join(ROOT, "include", "singa_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for ret, name, args in re.findall(r"SGH_API\s+([\w\s\*]+?)\b(sgh_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = " ".join(args.split())
        argl = [] if args in ("", "void") else [a.strip() for a in args.split(",")]
        out[name] = (" ".join(ret.split()), argl)
    return out


def _c_class(decl):
    """pointer / size / float / double / int / u64: the machine class of a C parameter declaration."""
    if "*" in decl:
        return "pointer"
    t = re.sub(r"\b\w+$", "", decl).strip() if len(decl.split()) > 1 else decl   # drop the parameter name
    t = t.replace("const", "").strip()
    # (size_t and uint64_t are one machine type on this ABI, and one ctypes type)
    return {"size_t": "u64", "float": "float", "double": "double", "int": "int", "void": "void",
            "uint64_t": "u64", "unsigned long long": "u64"}[t]


def _ctypes_class(t):
    if t is None:
        return "void"
    if t in (C.c_void_p, C.c_char_p) or hasattr(t, "contents"):
        return "pointer"
    return {C.c_size_t: "u64", C.c_float: "float", C.c_double: "double", C.c_int: "int", C.c_uint64: "u64"}[t]


def test_binding_argument_lists_match_the_header_prototypes():
    protos = _prototypes()
    assert set(protos) == set(_lib.SIGNATURES)
    for name, (res, args) in _lib.SIGNATURES.items():
        ret, decl = protos[name]
        assert len(args) == len(decl), (name, len(args), decl)
        assert [_ctypes_class(a) for a in args] == [_c_class(d) for d in decl], (name, decl)
        assert _ctypes_class(res) == ("pointer" if "*" in ret else _c_class(ret)), (name, ret)


def test_struct_layouts_match_the_header(tmp_path):
    """sizeof / offsetof of every struct that crosses the boundary, as a C compiler lays them out."""
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "singa_hip.h"\n'
                   'int main(void) {\n'
                   '  printf("%zu %zu %zu %zu\\n", sizeof(sgh_conv_geom), offsetof(sgh_conv_geom, Q), '
                   'offsetof(sgh_conv_geom, prelaid_W), offsetof(sgh_conv_geom, prelaid_epoch));\n'
                   '  printf("%zu %zu\\n", sizeof(sgh_pool_geom), offsetof(sgh_pool_geom, is_max));\n'
                   '  printf("%zu %zu\\n", sizeof(sgh_conv_prepare_item), offsetof(sgh_conv_prepare_item, ws_bytes));\n'
                   '  printf("%zu %zu\\n", sizeof(sgh_sgd_item), offsetof(sgh_sgd_item, n));\n'
                   '  printf("%zu %zu\\n", sizeof(sgh_sgd_mixed_item), offsetof(sgh_sgd_mixed_item, n));\n'
                   '  return 0;\n}\n')
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = [[int(v) for v in l.split()] for l in subprocess.check_output([str(exe)]).decode().splitlines()]
    G, P, I, S, M = _lib.ConvGeom, _lib.PoolGeom, _lib.ConvPrepareItem, _lib.SgdItem, _lib.SgdMixedItem
    assert got == [[C.sizeof(G), G.Q.offset, G.prelaid_W.offset, G.prelaid_epoch.offset],
                   [C.sizeof(P), P.is_max.offset], [C.sizeof(I), I.ws_bytes.offset],
                   [C.sizeof(S), S.n.offset], [C.sizeof(M), M.n.offset]]


@pytest.mark.parametrize("compiler,flags", [("gcc", ["-std=c11", "-x", "c"]), ("gcc", ["-std=c99", "-x", "c"]),
                                            ("g++", ["-std=c++17", "-x", "c++"])])
def test_header_compiles_as_c_and_cxx(tmp_path, compiler, flags):
    src = tmp_path / "include_only.c"
    src.write_text('#include "singa_hip.h"\n#include "singa_hip.h"\nint sgh_header_compiles;\n')
    subprocess.check_call([compiler] + flags + ["-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only",
                                                "-I", os.path.join(ROOT, "include"), str(src)])


def test_cxx_host_program_calls_through_the_real_prototypes(tmp_path):
    """A C++ host (what SINGA's glue is) resolves entry points from the built library with the types
    the header declares -- decltype of the prototypes, no casts to guessed signatures -- and calls
    the host-only ones."""
    src = tmp_path / "host.cc"
    src.write_text(r'''
#include <dlfcn.h>
#include <cstdio>
#include <cstring>
#include "singa_hip.h"
#define LOAD(name) auto p_##name = reinterpret_cast<decltype(&name)>(dlsym(h, #name)); if (!p_##name) { std::printf("missing %s\n", #name); return 2; }
int main(int argc, char **argv) {
  if (argc < 2) return 9;
  void *h = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!h) { std::printf("dlopen: %s\n", dlerror()); return 1; }
  LOAD(sgh_conv_geom_init) LOAD(sgh_conv_workspace_bytes) LOAD(sgh_error_string) LOAD(sgh_version)
  LOAD(sgh_bn_workspace_bytes) LOAD(sgh_pool_geom_init) LOAD(sgh_conv_dgrad_f32) LOAD(sgh_conv_weights_changed)
  sgh_conv_geom g;
  std::memset(&g, 0x5a, sizeof g);
  if (p_sgh_conv_geom_init(&g, 64, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1) != SGH_OK) return 3;
  if (g.P != 56 || g.Q != 56 || g.prelaid_W != nullptr) return 4;
  const size_t ws = p_sgh_conv_workspace_bytes(&g, SGH_CONV_DGRAD);
  sgh_pool_geom pg;
  if (p_sgh_pool_geom_init(&pg, 64, 64, 112, 112, 3, 3, 2, 2, 1, 1, 1) != SGH_OK || pg.P != 56) return 5;
  // argument checks happen before any device call: a null tensor is refused on a machine without a GPU too
  if (p_sgh_conv_dgrad_f32(&g, nullptr, nullptr, nullptr, nullptr, 0, nullptr) != SGH_EINVAL) return 6;
  p_sgh_conv_weights_changed();
  std::printf("%s %zu %zu %s|%s\n", p_sgh_version(), ws, p_sgh_bn_workspace_bytes(64, 64, 3136),
              p_sgh_error_string(SGH_EWORKSPACE), p_sgh_error_string(SGH_ELIMIT));
  return 0;
}
''')
    exe = tmp_path / "host"
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
                           str(src), "-o", str(exe), "-ldl"])
    out = subprocess.check_output([str(exe), _lib.LIBPATH]).decode().split(None, 3)
    lib = _lib.lib()
    g = _lib.ConvGeom()
    lib.sgh_conv_geom_init(C.byref(g), 64, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1)
    assert out[0].encode() == lib.sgh_version()
    assert int(out[1]) == lib.sgh_conv_workspace_bytes(C.byref(g), _lib.SGH_CONV_DGRAD)
    assert int(out[2]) == lib.sgh_bn_workspace_bytes(64, 64, 3136)
    assert "workspace" in out[3] and "non-allocating" in out[3]
