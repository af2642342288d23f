"""ctypes binding of librembrandt_hip.so (the C ABI declared in include/rembrandt_hip.h).

The library is loaded from the package directory; there is no fallback implementation: if the
shared object is missing, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("RH_LIB") or os.path.join(_HERE, "librembrandt_hip.so")

RH_CONV_FWD, RH_CONV_BWD_FILTER, RH_CONV_BWD_DATA = 0, 1, 2
RH_POOL_MAX, RH_POOL_AVG_INCL_PAD = 0, 1
RH_ROUND_FLOOR, RH_ROUND_CEIL = 0, 1
RH_FUSE_BIAS, RH_FUSE_RELU = 0x10, 0x20
RH_ALGO_GATHER, RH_ALGO_SCALAR_OFFSET, RH_ALGO_WINOGRAD, RH_ALGO_DIRECT = 0x100, 0x200, 0x400, 0x800
RH_ALGO_SHARED_GPU = 0x1000
RH_MATH_BF16_MFMA_FP32ACC = 0x1
RH_E_INVALID, RH_E_WORKSPACE, RH_E_UNSUPPORTED, RH_E_LIMIT = -1, -2, -3, -4


class ConvGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("N", "C", "H", "W", "K", "R", "S", "stride", "pad")]


class LrnGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("N", "C", "H", "W", "size")] + [(n, C.c_float) for n in ("scale", "power", "min_div")]


class SgdTensor(C.Structure):
    _fields_ = [("W", C.c_void_p), ("g", C.c_void_p), ("v", C.c_void_p), ("n", C.c_int64), ("l2", C.c_float),
                ("keep_grad", C.c_int32)]


class PoolGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("N", "C", "H", "W", "size", "stride", "pad", "mode", "round")]


_vp, _f, _i32, _i64, _sz, _int = C.c_void_p, C.c_float, C.c_int32, C.c_int64, C.c_size_t, C.c_int

# name -> (restype, argtypes).  Device pointers are passed as integers (c_void_p).
PROTOTYPES = {
    "rh_version": (C.c_char_p, []),
    "rh_last_error": (_int, []),
    "rh_error_string": (C.c_char_p, [_int]),
    "rh_ctx_create": (_int, [_int, C.POINTER(_vp)]),
    "rh_ctx_destroy": (_int, [_vp]),
    "rh_ctx_stream": (_vp, [_vp]),
    "rh_ctx_sync": (_int, [_vp]),
    "rh_ctx_aux_stream": (_vp, [_vp]),
    "rh_ctx_fork": (_int, [_vp]),
    "rh_ctx_join": (_int, [_vp]),
    "rh_malloc": (_int, [_vp, _sz, C.POINTER(_vp)]),
    "rh_free": (_int, [_vp, _vp]),
    "rh_memset_f32": (_int, [_vp, _f, _sz, _vp]),
    "rh_copy_d2d": (_int, [_vp, _vp, _sz, _vp]),
    "rh_load_sync": (_int, [_vp, _vp, _vp, _sz]),
    "rh_store_sync": (_int, [_vp, _vp, _vp, _sz]),
    "rh_cast_u8_f32": (_int, [_vp, _vp, _sz, _f, _vp]),
    "rh_crop_nchw": (_int, [_vp, _vp, C.c_int64, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "rembrandt_kernel_batch_blockmap256_flip": (None, [_vp, _i32, _i32, _vp, _vp]),
    "rembrandt_kernel_batch_map_preproc_pca3_noise": (None, [_vp, _i32, _i32, _vp, _vp, _vp, _vp, _vp]),
    "rembrandt_kernel_map_dropout": (None, [_vp, _i32, _f, _f, _vp, _vp, _vp, _vp]),
    "rembrandt_kernel_map_dropout_backprop": (None, [_vp, _i32, _f, _f, _vp, _vp, _vp]),
    "rh_rng_fill_uniform01_device": (_int, [C.c_uint64, C.c_uint64, C.c_uint64, _vp, _sz, _vp]),
    "rh_lrn_fwd": (_int, [C.POINTER(LrnGeom), _vp, _vp, _vp, _vp]),
    "rh_lrn_bwd": (_int, [C.POINTER(LrnGeom), _vp, _vp, _vp, _vp, _vp, _vp]),
    "rh_ctx_begin_capture": (_int, [_vp]),
    "rh_ctx_end_capture": (_int, [_vp, C.POINTER(_vp)]),
    "rh_graph_launch": (_int, [_vp, _vp]),
    "rh_graph_destroy": (_int, [_vp]),
    "rh_profile_enabled": (_int, []),
    "rh_bnorm_workspace_bytes": (_sz, [_int, _int, _int]),
    "rh_bnorm_fwd_train": (_int, [_int, _int, _int, _f, _vp, _f, _vp, C.c_double, C.c_double, _vp, _vp, _vp, _vp, _vp, _vp,
                                  _vp, _sz, _int, _vp]),
    "rh_bnorm_fwd_infer": (_int, [_int, _int, _int, _f, _vp, _f, _vp, C.c_double, _vp, _vp, _vp, _vp, _vp, _sz, _int, _vp]),
    "rh_bnorm_bwd": (_int, [_int, _int, _int, _f, _f, _vp, _vp, _vp, _f, _f, C.c_double, _vp, _vp, _vp, _vp, _vp, _vp, _sz,
                            _vp]),
    "rh_load_overlapped": (_int, [_vp, _vp, _vp, _sz]),
    "rh_mark_consumed": (_int, [_vp]),
    "rh_store_begin": (_int, [_vp, _vp, _vp, _sz]),
    "rh_store_wait": (_int, [_vp]),
    "rh_host_malloc": (_int, [_vp, _sz, C.POINTER(_vp)]),
    "rh_host_free": (_int, [_vp, _vp]),
    "rh_bnorm_bwd_relu": (_int, [_int, _int, _int, _f, _f, _vp, _vp, _vp, _f, _f, C.c_double, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                 _sz, _vp]),
    "rh_conv2d_out_dim": (_i32, [_i32, _i32, _i32, _i32]),
    "rh_conv2d_winograd_flops": (C.c_double, [C.POINTER(ConvGeom), _int, _int]),
    "rh_conv2d_workspace_bytes": (_sz, [C.POINTER(ConvGeom), _int]),
    "rh_conv2d_workspace_bytes_upto": (_sz, [C.POINTER(ConvGeom), _int]),
    "rh_conv2d_bwd_bias_workspace_bytes_upto": (_sz, [_i32, _i32, _i32]),
    "rh_sgemm_workspace_bytes_upto": (_sz, [_i32, _i32, _i32, _int]),
    "rh_bnorm_workspace_bytes_upto": (_sz, [_int, _int, _int]),
    "rh_conv2d_fwd": (_int, [C.POINTER(ConvGeom), _f, _vp, _vp, _f, _vp, _vp, _vp, _sz, _int, _vp]),
    "rh_conv2d_bwd_filter": (_int, [C.POINTER(ConvGeom), _f, _vp, _vp, _f, _vp, _vp, _sz, _int, _vp]),
    "rh_conv2d_bwd_filter_bias": (_int, [C.POINTER(ConvGeom), _f, _vp, _vp, _f, _vp, _vp, _vp, _sz, _int, _vp]),
    "rh_conv2d_bwd_bias": (_int, [_i32, _i32, _i32, _f, _vp, _f, _vp, _vp]),
    "rh_conv2d_bwd_bias_workspace_bytes": (_sz, [_i32, _i32, _i32]),
    "rh_conv2d_bwd_bias_ws": (_int, [_i32, _i32, _i32, _f, _vp, _f, _vp, _vp, _sz, _vp]),
    "rh_noalloc_scratch_bytes": (_sz, []),
    "rh_conv2d_bwd_bias_noalloc": (_int, [_i32, _i32, _i32, _f, _vp, _f, _vp, _vp]),
    "rh_conv2d_bwd_data": (_int, [C.POINTER(ConvGeom), _f, _vp, _vp, _f, _vp, _vp, _sz, _int, _vp]),
    "rh_conv2d_bwd_data_relu_supported": (_int, [C.POINTER(ConvGeom)]),
    "rh_conv2d_bwd_data_relu": (_int, [C.POINTER(ConvGeom), _f, _vp, _vp, _f, _vp, _vp, _vp, _sz, _int, _vp]),
    "rh_add_bias_nchw": (_int, [_vp, _vp, _i32, _i32, _i32, _f, _f, _vp]),
    "rembrandt_kernel_batch_map_rect_inplace": (None, [_vp, _i32, _i32, _vp]),
    "rembrandt_kernel_batch_map_rect_backprop_inplace": (None, [_vp, _i32, _i32, _vp, _vp]),
    "rh_sgemm_workspace_bytes": (_sz, [_i32, _i32, _i32]),
    "rh_sgemm": (_int, [_int, _int, _i32, _i32, _i32, _f, _vp, _i32, _vp, _i32, _f, _vp, _i32, _vp, _sz, _int, _vp]),
    "rh_sgemm_bias_act": (_int, [_int, _int, _i32, _i32, _i32, _f, _vp, _i32, _vp, _i32, _f, _vp, _i32, _vp, _vp, _sz, _int, _vp]),
    "rh_saxpy": (_int, [_i64, _f, _vp, _vp, _vp]),
    "rh_sscal": (_int, [_i64, _f, _vp, _vp]),
    "rh_pool2d_out_dim": (_i32, [_i32, _i32, _i32, _i32, _i32]),
    "rh_pool2d_fwd": (_int, [C.POINTER(PoolGeom), _vp, _vp, _vp, _vp]),
    "rh_pool2d_bwd": (_int, [C.POINTER(PoolGeom), _vp, _vp, _vp, _vp, _vp, _vp]),
    "rh_pool2d_bwd_relu_supported": (_int, [C.POINTER(PoolGeom)]),
    "rh_pool2d_bwd_relu": (_int, [C.POINTER(PoolGeom), _vp, _vp, _vp, _vp, _vp]),
    "rh_pool2d_bwd_avg_relu": (_int, [C.POINTER(PoolGeom), _vp, _vp, _vp, _vp]),
    "rh_pool2d_slot_supported": (_int, [C.POINTER(PoolGeom)]),
    "rh_pool2d_fwd_slot": (_int, [C.POINTER(PoolGeom), _vp, _vp, _vp, _vp]),
    "rh_pool2d_bwd_slot": (_int, [C.POINTER(PoolGeom), _vp, _vp, _vp, _vp, _vp]),
    "rh_softmax_fwd": (_int, [_vp, _vp, _i32, _i32, _vp]),
    "rembrandt_kernel_batch_map_softmax_kl_backward": (None, [_vp, _i32, _i32, _vp, _vp, _vp, _vp]),
    "rembrandt_kernel_batch_map_softmax_kl_loss1": (None, [_vp, _i32, _i32, _vp, _vp, _f, _vp, _vp]),
    "rembrandt_kernel_batch_blockreduce_sum": (None, [_vp, _i32, _i32, _vp, _f, _vp]),
    "rembrandt_kernel_batch_blockreduce_argmax": (None, [_vp, _i32, _i32, _vp, _vp, _vp]),
    "rh_softmax_kl_step": (_int, [_vp, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "rh_affine2_softmax_kl_step_supported": (_int, [_i32, _i32, _i32, _i32]),
    "rh_affine2_softmax_kl_step": (_int, [_i32, _i32, _i32, _i32, _i32] + [_vp] * 19),
    "rh_affine2_bwd_params": (_int, [_i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _f, _vp, _vp, _f, _vp, _vp, _vp]),
    "rh_sgd_momentum_step": (_int, [_i64, _vp, _vp, _vp, _f, _f, _f, _f, _int, _vp]),
    "rh_sgd_momentum_step_multi": (_int, [_i32, C.POINTER(SgdTensor), _f, _f, _f, _int, _vp]),
    "rh_descend": (_int, [_i64, _vp, _vp, _f, _f, _vp]),
    "rh_profile_enable": (_int, [_int]),
    "rh_profile_filter": (_int, [C.c_char_p]),
    "rh_profile_count": (_int, []),
    "rh_profile_get": (_int, [_int, C.POINTER(C.c_char_p), C.POINTER(C.c_double), C.POINTER(_f)]),
    "rh_profile_reset": (_int, []),
    "rh_probe_mfma_loop": (_int, [_int, _int, _int, _vp, _vp]),
    "rh_probe_mfma_loop_varied": (_int, [_int, _int, _vp, _vp]),
    "rh_probe_copy": (_int, [_vp, _vp, _sz, _vp]),
    "rh_bf16_act_bytes": (_sz, [_i32, _i32, _i32, _i32, _i32]),
    "rh_bf16_pack_nchw": (_int, [_i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp]),
    "rh_bf16_unpack_nchw": (_int, [_i32, _i32, _i32, _i32, _i32, _vp, _vp, _vp]),
    "rh_conv2d_fwd_bf16_filter_bytes": (_sz, [C.POINTER(ConvGeom)]),
    "rh_conv2d_fwd_bf16_takes_packed": (_int, [C.POINTER(ConvGeom)]),
    "rh_conv2d_fwd_bf16_workspace_bytes": (_sz, [C.POINTER(ConvGeom)]),
    "rh_conv2d_fwd_bf16_prep_filter": (_int, [C.POINTER(ConvGeom), _vp, _vp, _sz, _vp]),
    "rh_conv2d_fwd_bf16_packed": (_int, [C.POINTER(ConvGeom), _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _sz, _int, _vp]),
    "rh_pool2d_fwd_bf16_packed": (_int, [C.POINTER(PoolGeom), _vp, _vp, _i32, _vp]),
    "rh_rng_fill_uniform": (_int, [C.c_uint64, C.c_uint64, _vp, _sz, _f, _f]),
    "rh_rng_fill_normal": (_int, [C.c_uint64, C.c_uint64, _vp, _sz, _f, _f]),
    "rh_rng_fill_int": (_int, [C.c_uint64, C.c_uint64, _vp, _sz, _i32]),
}

_lib = None


class RembrandtHipError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        msg = lib().rh_error_string(code)
        super().__init__("%s failed: %d (%s)" % (where, code, msg.decode() if msg else "?"))


def lib():
    """The loaded shared library, with prototypes set.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: build it with `python -m rembrandt_amd.build` "
                              "(there is no CPU fallback)" % LIB_PATH)
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(code, where):
    """Reproduces the reference's panic-on-error convention (src/operator/mod.rs:1685-1696)."""
    if code != 0:
        raise RembrandtHipError(code, where)
