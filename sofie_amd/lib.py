"""ctypes binding of libsofie_hip.so, the C-ABI kernel library (include/sofie_hip.h).

There is no CPU fallback: if the library has not been built, loading raises.
"""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsofie_hip.so")

OK, EINVAL, EHIP, ENOMEM, EUNSUPPORTED = 0, -1, -2, -3, -4
ACT_NONE, ACT_RELU = 0, 1
BIAS_NONE, BIAS_ROW, BIAS_FULL, BIAS_COL = 0, 1, 2, 3
OUT_S8, OUT_F32, OUT_S32, OUT_BF16 = 0, 1, 2, 3
LAYOUT_NCHW, LAYOUT_NHWC = 0, 1

_p, _i, _f, _z = C.c_void_p, C.c_int, C.c_float, C.c_size_t

# name -> argument types (after the leading context pointer, where there is one)
SIGNATURES = {
    "sofie_hip_create": [C.POINTER(_p), _i, _p],
    "sofie_hip_destroy": [_p],
    "sofie_hip_last_error": [_p],
    "sofie_hip_version": [],
    "sofie_hip_malloc": [_p, C.POINTER(_p), _z],
    "sofie_hip_free": [_p, _p],
    "sofie_hip_host_malloc": [_p, C.POINTER(_p), _z],
    "sofie_hip_host_free": [_p, _p],
    "sofie_hip_upload": [_p, _p, _p, _z],
    "sofie_hip_download": [_p, _p, _p, _z],
    "sofie_hip_copy": [_p, _p, _p, _z],
    "sofie_hip_memset": [_p, _p, _i, _z],
    "sofie_hip_sync": [_p],
    "sofie_hip_timer_start": [_p],
    "sofie_hip_timer_stop": [_p, C.POINTER(_f)],
    "sofie_hip_trace_begin": [_p],
    "sofie_hip_trace_end": [_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_int)],
    "sofie_hip_gemm_f32": [_p, _i, _i, _i, _i, _i, _f, _p, _i, _p, _i, _f, _p, _i, _p, _i, _i],
    "sofie_hip_mlp_f32": [_p, _i, C.POINTER(_i), C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.POINTER(_i), _p, _i, _p, _i, _i],
    "sofie_hip_gemm_f32_stacked": [_p, _i, _i, _i, _i, _i, _f, _p, _i, _p, _i, _p, _i, _i, C.POINTER(_i),
                                   C.POINTER(C.c_longlong), C.POINTER(C.c_longlong), _i],
    "sofie_hip_conv2d_f32": [_p, _p, _p, _p, _p] + [_i] * 17,
    "sofie_hip_conv3d_f32": [_p, _p, _p, _p, _p] + [_i] * 20,
    "sofie_hip_conv_transpose2d_f32": [_p, _p, _p, _p, _p] + [_i] * 17,
    "sofie_hip_capture_begin": [_p],
    "sofie_hip_capture_end": [_p, _p],
    "sofie_hip_graph_launch": [_p, _p],
    "sofie_hip_graph_destroy": [_p, _p],
    "sofie_hip_batchnorm_f32": [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i],
    "sofie_hip_einsum_f32": [_p, _i, C.POINTER(_p), _i, _i, C.POINTER(_i), C.POINTER(C.c_longlong), _p],
    "sofie_hip_relu_f32": [_p, _p, _p, _z],
    "sofie_hip_maxpool2d_f32": [_p, _p, _p] + [_i] * 11,
    "sofie_hip_avgpool2d_f32": [_p, _p, _p] + [_i] * 12,
    "sofie_hip_constant_weights": [_p, _i],
    "sofie_hip_maxpool3d_f32": [_p, _p, _p, _i, _p, _p, _p, _p],
    "sofie_hip_avgpool3d_f32": [_p, _p, _p, _i, _p, _p, _p, _p, _i],
    "sofie_hip_quantize_f32_s8": [_p, _p, _p, _z, _f, _i],
    "sofie_hip_dequantize_s8_f32": [_p, _p, _p, _z, _f, _i],
    "sofie_hip_qgemm_s8": [_p, _i, _i, _i, _i, _p, _i, _p, _i, _p, _p, _i, _i, _p, _i, _i],
    "sofie_hip_qgemm_s8_pair": [_p, _i, _i, _p, _i, _i, _p, _i, _p, _p, _i, _i, _p, _i, _i, _p, _i, _p, _p, _i, _i, _p, _i, _i],
    "sofie_hip_qgemm_s8_noalloc": [_p, _i, _i, _i, _i, _p, _i, _p, _i, _p, _p, _i, _i, _p, _i, _i],
    "sofie_hip_qconv2d_s8": [_p, _p, _i, _p, _i, _p, _p, _p, _i] + [_i] * 18,
    "sofie_hip_qconv2d_pool_s8": [_p, _p, _i, _p, _i, _p, _p, _p, _i] + [_i] * 21,
    "sofie_hip_quantize_qconv2d_s8": [_p, _p, C.c_float, _i, _p, _i, _p, _p, _p, _i] + [_i] * 20,
    "sofie_hip_maxpool2d_s8": [_p, _p, _p] + [_i] * 13,
    "sofie_hip_relayout_s8": [_p, _p, _p] + [_i] * 6,
    "sofie_hip_transpose_bytes": [_p, _p, _p, _i, _i, _i, _i],
    "sofie_hip_gemm_fp8": [_p, _i, _i, _i, _i, _p, _i, _p, _i, _f, _f, _p, _p, _i, _i],
    "sofie_hip_quantize_f32_e4m3": [_p, _p, _p, _z, _f],
}


class QConvLayer(C.Structure):
    """sofie_hip_qconv_layer of include/sofie_hip.h."""
    _fields_ = [("w", _p), ("w_layout", _i), ("bias", _p), ("scale", _p), ("y", _p), ("y_layout", _i)] + \
               [(n, _i) for n in ("C", "H", "W", "OC", "KH", "KW", "pad_top", "pad_left", "pad_bottom", "pad_right", "stride_h",
                                  "stride_w", "groups", "zp_x", "zp_y", "act", "pool_kh", "pool_kw", "pool_stride_h",
                                  "pool_stride_w")]


SIGNATURES["sofie_hip_qconv2d_s8_chain"] = [_p, _p, _i, _i, _i, C.POINTER(QConvLayer)]


def build(verbose=False):
    """Compile every HIP source for gfx950 into libsofie_hip.so (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), "-j8"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode:
        print(res.stdout)
    if res.returncode:
        raise RuntimeError("building libsofie_hip.so failed")
    return LIB_PATH


_lib = None


def load():
    """dlopen the library and attach signatures. Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("libsofie_hip.so is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                           "(there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.argtypes = args
        fn.restype = C.c_char_p if name == "sofie_hip_last_error" else C.c_int
    _lib = lib
    return lib
