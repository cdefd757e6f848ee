"""ctypes binding of the C ABI declared in ``include/singa_hip.h``.

The shared library is looked up in-tree (``singa_amd/lib/libsinga_hip.so``).  There is no
fallback: if the library is missing or a symbol cannot be resolved, importing fails loudly.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIBPATH = os.path.join(HERE, "lib", "libsinga_hip.so")

c_float_p = C.POINTER(C.c_float)
c_int32_p = C.POINTER(C.c_int32)
vp = C.c_void_p
sz = C.c_size_t


class ConvGeom(C.Structure):
    """``sgh_conv_geom``"""
    _fields_ = [(n, C.c_int) for n in
                ("N", "C", "H", "W", "K", "R", "S", "stride_h", "stride_w", "pad_h", "pad_w", "P", "Q", "groups",
                 "prelaid_dtype")] + [("prelaid_W", C.c_void_p), ("prelaid_ws", C.c_void_p),
                                      ("prelaid_ws_bytes", C.c_size_t), ("prelaid_epoch", C.c_ulonglong)]


class ConvPrepareItem(C.Structure):
    """``sgh_conv_prepare_item``"""
    _fields_ = [("g", C.POINTER(ConvGeom)), ("W", vp), ("workspace", vp), ("ws_bytes", C.c_size_t)]


class PoolGeom(C.Structure):
    """``sgh_pool_geom``"""
    _fields_ = [(n, C.c_int) for n in
                ("N", "C", "H", "W", "kernel_h", "kernel_w", "stride_h", "stride_w", "pad_h", "pad_w",
                 "P", "Q", "is_max")]


class SgdItem(C.Structure):
    """``sgh_sgd_item``"""
    _fields_ = [("p", vp), ("g", vp), ("v", vp), ("n", C.c_uint64)]


class SgdMixedItem(C.Structure):
    """``sgh_sgd_mixed_item``"""
    _fields_ = [("p", vp), ("g", vp), ("v", vp), ("p16", vp), ("n", C.c_uint64)]


# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
    "sgh_error_string": (C.c_char_p, [C.c_int]),
    "sgh_version": (C.c_char_p, []),
    "sgh_arch": (C.c_char_p, []),
    "sgh_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "sgh_device_open": (C.c_int, [C.c_int, C.POINTER(vp)]),
    "sgh_device_close": (C.c_int, [vp]),
    "sgh_device_stream": (vp, [vp]),
    "sgh_device_aux_stream": (vp, [vp]),
    "sgh_device_sync": (C.c_int, [vp]),
    "sgh_device_fork": (C.c_int, [vp, C.POINTER(vp)]),
    "sgh_device_join": (C.c_int, [vp]),
    "sgh_block_used_on": (C.c_int, [vp, vp, vp]),
    "sgh_malloc": (C.c_int, [vp, C.POINTER(vp), sz]),
    "sgh_free": (C.c_int, [vp, vp]),
    "sgh_pool_stats": (C.c_int, [vp, C.POINTER(sz), C.POINTER(sz), C.POINTER(sz)]),
    "sgh_pool_trim": (C.c_int, [vp]),
    "sgh_memcpy": (C.c_int, [vp, vp, vp, sz, C.c_int]),
    "sgh_upload_async": (C.c_int, [vp, vp, vp, sz]),
    "sgh_memset_f32": (C.c_int, [vp, C.c_float, sz, vp]),
    "sgh_memset_f16": (C.c_int, [vp, C.c_float, sz, vp]),
    "sgh_memset_bf16": (C.c_int, [vp, C.c_float, sz, vp]),
    "sgh_graph_begin": (C.c_int, [vp]),
    "sgh_graph_end": (C.c_int, [vp, C.POINTER(vp)]),
    "sgh_graph_launch": (C.c_int, [vp]),
    "sgh_graph_destroy": (C.c_int, [vp]),
    "sgh_event_create": (C.c_int, [C.POINTER(vp)]),
    "sgh_event_destroy": (C.c_int, [vp]),
    "sgh_event_record": (C.c_int, [vp, vp]),
    "sgh_stream_wait_event": (C.c_int, [vp, vp]),
    "sgh_event_elapsed_ms": (C.c_int, [vp, vp, C.POINTER(C.c_float)]),
    "sgh_prof_enable": (C.c_int, [C.c_int]),
    "sgh_prof_clear": (C.c_int, []),
    "sgh_prof_count": (C.c_int, [C.POINTER(C.c_int)]),
    "sgh_prof_get": (C.c_int, [C.c_int, C.c_char_p, sz, C.POINTER(C.c_float), C.POINTER(C.c_double)]),
    "sgh_relu_bwd_f32": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_relu_fwd_f32": (C.c_int, [vp, vp, sz, vp]),
    "sgh_relu_fwd_f16": (C.c_int, [vp, vp, sz, vp]),
    "sgh_relu_fwd_bf16": (C.c_int, [vp, vp, sz, vp]),
    "sgh_softmax_ce_bwd_f16": (C.c_int, [vp, vp, vp, sz, sz, C.c_int, C.c_float, vp]),
    "sgh_softmax_ce_bwd_bf16": (C.c_int, [vp, vp, vp, sz, sz, C.c_int, C.c_float, vp]),
    "sgh_row_max_zero_seeded_f32": (C.c_int, [vp, vp, sz, sz, vp]),
    "sgh_cast_f32_to_i32": (C.c_int, [vp, vp, sz, vp]),
    "sgh_cast_i32_to_f32": (C.c_int, [vp, vp, sz, vp]),
    "sgh_gemm_f16": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, vp, C.c_int,
                               vp, C.c_int, C.c_float, vp, C.c_int, vp]),
    "sgh_gemm_bf16": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, vp, C.c_int,
                                vp, C.c_int, C.c_float, vp, C.c_int, vp]),
    "sgh_conv_dgrad_acc_supported": (C.c_int, [C.POINTER(ConvGeom)]),
    "sgh_softmax_ce_bwd_f32": (C.c_int, [vp, vp, vp, sz, sz, C.c_int, C.c_float, vp]),
    "sgh_softmax_ce_label_errors": (C.c_int, [vp, C.POINTER(C.c_int)]),
    "sgh_softmax_fwd_f32": (C.c_int, [vp, vp, sz, sz, vp]),
    "sgh_cross_entropy_fwd_f32": (C.c_int, [vp, vp, vp, sz, sz, C.c_int, vp]),
    "sgh_transform_f32": (C.c_int, [vp, vp, C.c_int, C.POINTER(C.c_size_t), C.POINTER(C.c_int64), vp]),
    "sgh_row_max_f32": (C.c_int, [vp, vp, sz, sz, vp]),
    "sgh_reduce_workspace_bytes": (sz, []),
    "sgh_dot_f32": (C.c_int, [vp, vp, sz, vp, vp, sz, vp]),
    "sgh_sum_all_f32": (C.c_int, [vp, sz, vp, vp, sz, vp]),
    "sgh_uniform_f32": (C.c_int, [C.c_float, C.c_float, vp, sz, C.c_uint64, C.c_uint64, vp]),
    "sgh_gaussian_f32": (C.c_int, [C.c_float, C.c_float, vp, sz, C.c_uint64, C.c_uint64, vp]),
    "sgh_clamp_f32": (C.c_int, [C.c_float, C.c_float, vp, vp, sz, vp]),
    "sgh_axpy_f32": (C.c_int, [C.c_float, vp, vp, sz, vp]),
    "sgh_axpy_devalpha_f32": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_eltwise_mult_f32": (C.c_int, [vp, vp, C.c_int, vp, sz, vp]),
    "sgh_add_f32": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_add_relu_f32": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_add_relu_f16": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_add_relu_bf16": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_sgd_momentum_multi_mixed": (C.c_int, [vp, C.c_int, sz, C.c_int, C.c_float, C.c_float, C.c_float, C.c_float,
                                               C.c_int, vp]),
    "sgh_sub_f32": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_div_f32": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_add_scalar_f32": (C.c_int, [vp, C.c_float, vp, sz, vp]),
    "sgh_mult_scalar_f32": (C.c_int, [vp, C.c_float, vp, sz, vp]),
    "sgh_bn_fwd_infer_f32": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, vp, C.c_int, C.c_int, C.c_int, vp]),
    "sgh_bn_fwd_infer_f16": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, vp, C.c_int, C.c_int, C.c_int, vp]),
    "sgh_bn_fwd_infer_bf16": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, vp, C.c_int, C.c_int, C.c_int, vp]),
    "sgh_cast_f32_to_f16": (C.c_int, [vp, vp, sz, vp]),
    "sgh_cast_f16_to_f32": (C.c_int, [vp, vp, sz, vp]),
    "sgh_cast_f32_to_bf16": (C.c_int, [vp, vp, sz, vp]),
    "sgh_cast_bf16_to_f32": (C.c_int, [vp, vp, sz, vp]),
    "sgh_relu_bwd_f16": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_relu_bwd_add_f32": (C.c_int, [vp, vp, vp, vp, sz, vp]),
    "sgh_relu_bwd_add_f16": (C.c_int, [vp, vp, vp, vp, sz, vp]),
    "sgh_relu_bwd_add_bf16": (C.c_int, [vp, vp, vp, vp, sz, vp]),
    "sgh_relu_bwd_bf16": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_add_f16": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_add_bf16": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_eltwise_mult_f16": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_eltwise_mult_bf16": (C.c_int, [vp, vp, vp, sz, vp]),
    "sgh_axpy_f16": (C.c_int, [C.c_float, vp, vp, sz, vp]),
    "sgh_axpy_bf16": (C.c_int, [C.c_float, vp, vp, sz, vp]),
    "sgh_sgd_momentum_f32": (C.c_int, [vp, vp, vp, sz, C.c_float, C.c_float, C.c_float, C.c_float,
                                       C.c_int, vp]),
    "sgh_sgd_momentum_devhyper_f32": (C.c_int, [vp, vp, vp, sz, vp, C.c_int, vp]),
    "sgh_sgd_momentum_multi_f32": (C.c_int, [vp, C.c_int, sz, C.c_float, C.c_float, C.c_float,
                                             C.c_float, C.c_int, vp]),
    "sgh_sgd_momentum_f16": (C.c_int, [vp, vp, vp, sz, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int, vp]),
    "sgh_sgd_momentum_bf16": (C.c_int, [vp, vp, vp, sz, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int, vp]),
    "sgh_sgd_momentum_master_f16": (C.c_int, [vp, vp, vp, vp, sz, C.c_float, C.c_float, C.c_float, C.c_float,
                                              C.c_int, vp]),
    "sgh_sgd_momentum_master_bf16": (C.c_int, [vp, vp, vp, vp, sz, C.c_float, C.c_float, C.c_float, C.c_float,
                                               C.c_int, vp]),
    "sgh_gemm_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, vp, C.c_int,
                               vp, C.c_int, C.c_float, vp, C.c_int, vp]),
    "sgh_sum_rows_f32": (C.c_int, [vp, vp, C.c_int, C.c_int, vp]),
    "sgh_add_row_f32": (C.c_int, [vp, vp, C.c_int, C.c_int, vp]),
    "sgh_conv_geom_init": (C.c_int, [C.POINTER(ConvGeom)] + [C.c_int] * 11),
    "sgh_conv_geom_init_grouped": (C.c_int, [C.POINTER(ConvGeom)] + [C.c_int] * 12),
    "sgh_conv_workspace_bytes": (sz, [C.POINTER(ConvGeom), C.c_int]),
    "sgh_conv_dgrad_f32": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, sz, vp]),
    "sgh_conv_dgrad_acc_f32": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, sz, vp]),
    "sgh_conv_wgrad_f32": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, sz, vp]),
    "sgh_conv_wgrad_bias_f32": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, vp, sz, vp]),
    "sgh_conv_bgrad_f32": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp]),
    "sgh_conv_fwd_f32": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, vp, sz, vp]),
    "sgh_conv_workspace_bytes_h": (sz, [C.POINTER(ConvGeom), C.c_int]),
    "sgh_conv_dgrad_prepare_multi": (C.c_int, [C.POINTER(ConvPrepareItem), C.c_int, C.c_int, vp]),
    "sgh_conv_weights_changed": (None, []),
    "sgh_conv_dgrad_f16": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, sz, vp]),
    "sgh_conv_dgrad_bf16": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, sz, vp]),
    "sgh_conv_wgrad_f16": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, sz, vp]),
    "sgh_conv_wgrad_bf16": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, sz, vp]),
    "sgh_conv_wgrad16_split_mode": (None, [C.c_int]),
    "sgh_conv_bgrad_f16": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp]),
    "sgh_conv_bgrad_bf16": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp]),
    "sgh_conv_fwd_f16": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, vp, sz, vp]),
    "sgh_conv_fwd_bf16": (C.c_int, [C.POINTER(ConvGeom), vp, vp, vp, vp, vp, sz, vp]),
    "sgh_bn_workspace_bytes": (sz, [C.c_int, C.c_int, C.c_int]),
    "sgh_bn_exchange_failures": (C.c_int, [vp, C.POINTER(C.c_int)]),
    "sgh_bn_exchange_spin_limit": (None, [C.c_int]),
    "sgh_bn_fwd_train_f32": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, vp, C.c_int,
                                       C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_relu_fwd_train_f32": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, vp, C.c_int,
                                       C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_add_relu_fwd_train_f32": (C.c_int, [vp, vp, vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, vp, C.c_int,
                                       C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_add_relu_fwd_train_f16": (C.c_int, [vp, vp, vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, vp, C.c_int,
                                       C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_add_relu_fwd_train_bf16": (C.c_int, [vp, vp, vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, vp, C.c_int,
                                       C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_relu_fwd_train_f16": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, vp, C.c_int,
                                       C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_relu_fwd_train_bf16": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, vp, C.c_int,
                                       C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_bwd_f32": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_bwd_noalloc_f32": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp]),
    "sgh_bn_fwd_train_f16": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, vp, C.c_int,
                                       C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_fwd_train_bf16": (C.c_int, [vp, vp, vp, vp, vp, C.c_float, C.c_float, vp, vp, vp, C.c_int,
                                        C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_bwd_f16": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_relu_bwd_f32": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_relu_bwd_f16": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_relu_bwd_bf16": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp, sz, vp]),
    "sgh_bn_bwd_bf16": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp, sz, vp]),
    "sgh_pool_geom_init": (C.c_int, [C.POINTER(PoolGeom)] + [C.c_int] * 11),
    "sgh_pool_fwd_f32": (C.c_int, [C.POINTER(PoolGeom), vp, vp, vp]),
    "sgh_pool_bwd_f32": (C.c_int, [C.POINTER(PoolGeom), vp, vp, vp, vp, vp]),
    "sgh_pool_fwd_f16": (C.c_int, [C.POINTER(PoolGeom), vp, vp, vp]),
    "sgh_pool_fwd_bf16": (C.c_int, [C.POINTER(PoolGeom), vp, vp, vp]),
    "sgh_pool_bwd_f16": (C.c_int, [C.POINTER(PoolGeom), vp, vp, vp, vp, vp]),
    "sgh_pool_bwd_bf16": (C.c_int, [C.POINTER(PoolGeom), vp, vp, vp, vp, vp]),
}

SGH_CONV_FWD, SGH_CONV_DGRAD, SGH_CONV_WGRAD = 0, 1, 2
SGH_EUNSUPPORTED = -3
SGH_ELIMIT = -6
SGH_EEXCHANGE = -7


class SingaHipError(RuntimeError):
    pass


def load(path=LIBPATH):
    """dlopen the library and attach prototypes to every declared symbol."""
    if not os.path.exists(path):
        raise SingaHipError(
            "%s not found: build it with `python -m singa_amd.build` (no CPU fallback exists)" % path)
    lib = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = load()
    return _lib


def check(rc, what=""):
    """The glue-side CHECK_EQ(rc, 0): raise with the library's message on failure."""
    if rc != 0:
        msg = lib().sgh_error_string(rc).decode()
        raise SingaHipError("%s failed: rc=%d (%s)" % (what or "singa_hip call", rc, msg))
