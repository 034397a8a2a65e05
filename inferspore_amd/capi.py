"""ctypes view of include/inferspore_amd.h.  Loading fails loudly when the library is not built."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libinferspore_amd.so")

OK = 0
ERR_NULL_POINTER = -1
ERR_BAD_SHAPE = -2
ERR_UNSUPPORTED = -3
ERR_LAUNCH = -4
ERR_DEVICE = -5
NORM_RESIDUAL_EXCLUDES_BIAS = 1
(TUNE_NORM_WAVES_PER_ROW, TUNE_NORM_STORE, TUNE_SWIGLU_UNROLL, TUNE_SWIGLU_STORE, TUNE_EMBED_VARIANT,
 TUNE_EMBED_STORE, TUNE_QKV_STORE, TUNE_QKV_WAVES, TUNE_NORM_BLOCK_THREADS, TUNE_NORM_ORDER,
 TUNE_MOVER_BLOCK_THREADS) = range(11)

_vp, _i, _f, _u = C.c_void_p, C.c_int, C.c_float, C.c_uint

# name -> (restype, argtypes); one entry per function declared in the public header
SIGNATURES = {
    "isp_version": (C.c_char_p, []),
    "isp_strerror": (C.c_char_p, [_i]),
    "isp_last_hip_error": (_i, []),
    "isp_init": (_i, []),
    "isp_embedding_f16": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "isp_embedding_f32": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "isp_cal_padding_offset": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "isp_rmsnorm_f32": (_i, [_vp, _vp, _f, _i, _i, _vp]),
    "isp_rmsnorm_f16": (_i, [_vp, _vp, _f, _i, _i, _vp]),
    "isp_fused_add_bias_residual_rmsnorm_f32": (_i, [_vp, _vp, _vp, _vp, _f, _i, _i, _u, _vp]),
    "isp_fused_add_bias_residual_rmsnorm_f16": (_i, [_vp, _vp, _vp, _vp, _f, _i, _i, _u, _vp]),
    "isp_qkv_bias_rope_transpose_f32": (_i, [_vp] * 8 + [_i] * 7 + [_f, _i, _i, _vp]),
    "isp_qkv_bias_rope_transpose_f16": (_i, [_vp] * 8 + [_i] * 7 + [_f, _i, _i, _vp]),
    "isp_qkv_bias_rope_transpose_append_f32": (_i, [_vp] * 5 + [_i, _i] + [_vp] * 5 + [_i] * 7 + [_f, _vp]),
    "isp_qkv_bias_rope_transpose_append_f16": (_i, [_vp] * 5 + [_i, _i] + [_vp] * 5 + [_i] * 7 + [_f, _vp]),
    "isp_swiglu_f32": (_i, [_vp, _vp, _i, _i, _vp]),
    "isp_swiglu_f16": (_i, [_vp, _vp, _i, _i, _vp]),
    "isp_rope_decode_f32": (_i, [_vp, _i, _i, _i, _i, _i, _i, _f, _vp]),
    "isp_rope_decode_f16": (_i, [_vp, _i, _i, _i, _i, _i, _i, _f, _vp]),
    "isp_rope_decode_append_f32": (_i, [_vp] * 4 + [_i, _i, _vp] + [_i] * 6 + [_f, _vp]),
    "isp_rope_decode_append_f16": (_i, [_vp] * 4 + [_i, _i, _vp] + [_i] * 6 + [_f, _vp]),
    "isp_transpose_remove_padding_f32": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "isp_transpose_remove_padding_f16": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "isp_concat_kv_cache_f32": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "isp_concat_kv_cache_f16": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "isp_repeat_kv_cache_f32": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "isp_repeat_kv_cache_f16": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "isp_tuning_set": (_i, [_i, _i]),
    "isp_calibration_copy": (_i, [_vp, _vp, C.c_size_t, _vp]),
    "isp_norm_launch_config": (_i, [_i, _i, _i, _i] + [C.POINTER(C.c_int)] * 4),
    "isp_norm_launch_variant": (_i, [_i, _i, _i, _i, _i, C.c_uint]),
}

_lib = None


class IspError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = lib().isp_strerror(status).decode()
        if status == ERR_LAUNCH:
            msg += " (hipError %d)" % lib().isp_last_hip_error()
        super().__init__("[inferspore_amd] %s failed: %s (status %d)" % (where, msg, status))


def lib():
    """The loaded C-ABI library.  Raises if it has not been built (python -m inferspore_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "inferspore_amd: %s is missing -- build it with `python -m inferspore_amd.build`; "
                "there is no fallback implementation" % LIB_PATH)
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(status, where):
    if status != OK:
        raise IspError(status, where)
