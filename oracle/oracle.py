"""ctypes/numpy front end of the CPU oracle (test infrastructure, not product code).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this module. Every function forwards to ``liboracle.so`` built from
``sofie_oracle.c``; see that file for the reference lines each routine follows.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# SOFIE_ORACLE_LIB: another build of the same source (the sanitizer build the test suite runs in a child process)
_LIB_PATH = os.environ.get("SOFIE_ORACLE_LIB") or os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile liboracle.so with gcc (a few seconds)."""
    args = ["make", "-C", _HERE]
    if force:
        args.insert(1, "-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_i8p = np.ctypeslib.ndpointer(np.int8, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")


def _opt(arr, dtype):
    if arr is None:
        return None
    a = np.ascontiguousarray(arr, dtype=dtype)
    return a.ctypes.data_as(C.c_void_p)


def _sig(name, restype, argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = argtypes
    return fn


_sgemm = _sig("or_sgemm", None, [C.c_char, C.c_char, C.c_int, C.c_int, C.c_int, C.c_float,
                                 _f32p, C.c_int, _f32p, C.c_int, C.c_float, _f32p, C.c_int])
_gemm_f32 = _sig("or_gemm_f32", C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float,
                                          _f32p, _f32p, C.c_float, C.c_void_p, _f32p, C.c_int])
_relu = _sig("or_relu_f32", None, [_f32p, _f32p, C.c_size_t])
_im2col = _sig("or_im2col", None, [_f32p] + [C.c_int] * 11 + [_f32p])
_conv2d = _sig("or_conv2d_f32", C.c_int, [_f32p, _f32p, C.c_void_p, _f32p] + [C.c_int] * 15)
_conv3d = _sig("or_conv3d_f32", C.c_int, [_f32p, _f32p, C.c_void_p, _f32p] + [C.c_int] * 20)
_convt = _sig("or_conv_transpose2d_f32", C.c_int, [_f32p, _f32p, C.c_void_p, _f32p] + [C.c_int] * 17)
_einsum = _sig("or_einsum_f32", None, [C.c_int, C.POINTER(C.c_void_p), C.c_int, C.c_int, C.POINTER(C.c_int),
                                     C.POINTER(C.c_longlong), _f32p])
_bn = _sig("or_batchnorm_f32", None, [_f32p] * 5 + [C.c_float, _f32p] + [C.c_int] * 4)
_maxpool = _sig("or_maxpool2d_f32", None, [_f32p, _f32p] + [C.c_int] * 11)
_avgpool = _sig("or_avgpool2d_f32", None, [_f32p, _f32p] + [C.c_int] * 12)
_maxpool_s8 = _sig("or_maxpool2d_s8", None, [_i8p, _i8p] + [C.c_int] * 11)
_pool3d = _sig("or_pool3d_f32", None, [_f32p, _f32p, C.c_int] + [C.POINTER(C.c_int)] * 4 + [C.c_int] * 2)
_requant_one = _sig("or_requant_one", C.c_int8, [C.c_int32, C.c_float, C.c_int, C.c_int])
_quant = _sig("or_quantize_f32_s8", None, [_f32p, _i8p, C.c_size_t, C.c_float, C.c_int])
_dequant = _sig("or_dequantize_s8_f32", None, [_i8p, _f32p, C.c_size_t, C.c_float, C.c_int])
_igemm = _sig("or_igemm_s8", None, [C.c_int] * 4 + [_i8p, _i8p, C.c_int, C.c_int, _i32p])
_qgemm = _sig("or_qgemm_s8", None, [C.c_int] * 4 + [_i8p, _i8p, C.c_int, _f32p, C.c_void_p,
                                                     C.c_int, C.c_int, _i8p])
_qgemm_f = _sig("or_qgemm_s8_f32out", None, [C.c_int] * 4 + [_i8p, _i8p, C.c_int, _f32p,
                                                              C.c_void_p, C.c_int, _f32p])
_iconv = _sig("or_iconv2d_s8", C.c_int, [_i8p, _i8p, _i32p] + [C.c_int] * 13)
_qconv = _sig("or_qconv2d_s8", C.c_int, [_i8p, _i8p, C.c_void_p, _f32p, _i8p] + [C.c_int] * 15)
_e4m3_dec = _sig("or_e4m3_to_f32", C.c_float, [C.c_uint8])
_e4m3_enc = _sig("or_f32_to_e4m3_sat", C.c_uint8, [C.c_float])
_bf16_enc = _sig("or_f32_to_bf16", C.c_uint16, [C.c_float])
_bf16_dec = _sig("or_bf16_to_f32", C.c_float, [C.c_uint16])
_gemm_fp8 = _sig("or_gemm_fp8", None, [C.c_int] * 4 + [_u8p, _u8p, C.c_float, C.c_float,
                                                        C.c_void_p, C.c_void_p, C.c_void_p, C.c_int])


def sgemm(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, Cmat, ldc):
    """Column-major SGEMM on flat float32 arrays; Cmat is updated in place."""
    _sgemm(transa.encode(), transb.encode(), m, n, k, alpha, A, lda, B, ldb, beta, Cmat, ldc)
    return Cmat


def gemm_f32(A, B, bias=None, alpha=1.0, beta=1.0, transA=False, transB=False, relu=False):
    """Y = alpha*op(A)*op(B) + beta*broadcast(bias) [ReLU], as SOFIE's Gemm emits it.

    ``bias`` may be rank-1 [N] or full [M,N]; rank-1 is broadcast to [M,N] first,
    as the generated Session constructor does.
    """
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    N = B.shape[0] if transB else B.shape[1]
    Y = np.empty((M, N), np.float32)
    bb = None
    if bias is not None:
        bias = np.asarray(bias, np.float32)
        bb = np.ascontiguousarray(np.broadcast_to(bias, (M, N)))
    rc = _gemm_f32(int(transA), int(transB), M, N, K, alpha, A, B, beta, _opt(bb, np.float32), Y,
                   int(relu))
    if rc:
        raise RuntimeError("TMVA SOFIE Gemm Op Bias tensor is not present but beta value in Gemm is not zero")
    return Y


def relu_f32(x):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    _relu(x.reshape(-1), y.reshape(-1), x.size)
    return y


def _pads_hw(x, pads, fill=0):
    """The C restatement follows the reference's Im2col, which knows one pad per axis (SOFIE_common.hxx:485-518).
    pads = (h, w) is handed over as it is; pads = (top, left, bottom, right) with begin != end pads, which the
    reference cannot express (it averages them, ROperator_Conv.hxx:387-401), is ONNX's definition taken literally:
    the padded tensor is written out (cells hold `fill`) and convolved without pads."""
    pads = tuple(int(p) for p in pads)
    if len(pads) == 2:
        return x, pads
    pt, pl, pb, pr = pads
    if pt == pb and pl == pr:
        return x, (pt, pl)
    return np.pad(x, ((0, 0), (0, 0), (pt, pb), (pl, pr)), constant_values=fill), (0, 0)


def conv_out_hw(H, W, kh, kw, ph, pw, sh, sw, dh=1, dw=1):
    return ((H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1,
            (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1)


def im2col(im, kh, kw, ph, pw, sh, sw, dh=1, dw=1):
    im = np.ascontiguousarray(im, np.float32)
    Cc, H, W = im.shape
    OH, OW = conv_out_hw(H, W, kh, kw, ph, pw, sh, sw, dh, dw)
    col = np.empty((Cc * kh * kw, OH * OW), np.float32)
    _im2col(im, Cc, H, W, kh, kw, ph, pw, sh, sw, dh, dw, col)
    return col


def conv2d_f32(x, w, bias=None, pads=(0, 0), strides=(1, 1), dilations=(1, 1), groups=1,
               relu=False):
    x, pads = _pads_hw(np.asarray(x, np.float32), pads)
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    N, Cc, H, W = x.shape
    OC, _, kh, kw = w.shape
    OH, OW = conv_out_hw(H, W, kh, kw, pads[0], pads[1], strides[0], strides[1], *dilations)
    y = np.empty((N, OC, OH, OW), np.float32)
    rc = _conv2d(x, w, _opt(bias, np.float32), y, N, Cc, H, W, OC, kh, kw, pads[0], pads[1],
                 strides[0], strides[1], dilations[0], dilations[1], groups, int(relu))
    if rc:
        raise RuntimeError("or_conv2d_f32 failed: %d" % rc)
    return y


def conv3d_f32(x, w, bias=None, pads=(0, 0, 0), strides=(1, 1, 1), dilations=(1, 1, 1), groups=1, relu=False):
    """3-D convolution, NCDHW (ROperator_Conv.hxx:432-451 with Im2col_3d); pads are the begin pads (d, h, w)."""
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    N, Cc, D, H, W = x.shape
    OC, _, kd, kh, kw = w.shape
    out = [(i + 2 * p - (d * (k - 1) + 1)) // s + 1 for i, p, d, k, s in zip((D, H, W), pads, dilations, (kd, kh, kw), strides)]
    y = np.empty((N, OC, out[0], out[1], out[2]), np.float32)
    rc = _conv3d(x, w, _opt(bias, np.float32), y, N, Cc, D, H, W, OC, kd, kh, kw, *pads, *strides, *dilations, groups, int(relu))
    if rc:
        raise RuntimeError("or_conv3d_f32 failed: %d" % rc)
    return y


def conv_transpose2d_f32(x, w, bias=None, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), groups=1,
                         output_padding=(0, 0), relu=False):
    """ONNX ConvTranspose (ROperator_ConvTranspose.icc:232-474): x [N,C,H,W], w [C, OC/groups, kh, kw],
    pads = (top, left, bottom, right); begin pads position the result, end pads only shorten it."""
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    N, Cc, H, W = x.shape
    _, ocg, kh, kw = w.shape
    OC = ocg * groups
    OH = strides[0] * (H - 1) + dilations[0] * (kh - 1) + 1 + output_padding[0] - pads[0] - pads[2]
    OW = strides[1] * (W - 1) + dilations[1] * (kw - 1) + 1 + output_padding[1] - pads[1] - pads[3]
    y = np.empty((N, OC, OH, OW), np.float32)
    rc = _convt(x, w, _opt(bias, np.float32), y, N, Cc, H, W, OC, kh, kw, pads[0], pads[1], strides[0], strides[1],
                dilations[0], dilations[1], groups, OH, OW, int(relu))
    if rc:
        raise RuntimeError("or_conv_transpose2d_f32 failed: %d" % rc)
    return y


def batchnorm_f32(x, scale, bias, mean, var, epsilon=1e-5, relu=False):
    """Inference BatchNormalization over axis 1 (ROperator_BatchNormalization.hxx:127-226)."""
    x = np.ascontiguousarray(x, np.float32)
    N, Cc = x.shape[0], x.shape[1]
    plane = int(np.prod(x.shape[2:])) if x.ndim > 2 else 1
    y = np.empty_like(x)
    f = lambda a: np.ascontiguousarray(a, np.float32)
    _bn(x.reshape(-1), f(scale), f(bias), f(mean), f(var), float(epsilon), y.reshape(-1), N, Cc, plane, int(relu))
    return y


def einsum_plan(equation, shapes):
    """Labels (output labels first, then the summed ones sorted by character, the order of the reference's
    std::map, ROperator_Einsum.hxx:125-165), their extents, per-operand strides, the output shape."""
    eq = equation.replace(" ", "")
    lhs, out = eq.split("->")
    ins = lhs.split(",")
    assert len(ins) == len(shapes)
    extent = {}
    for labels, shape in zip(ins, shapes):
        assert len(labels) == len(shape)
        for l, d in zip(labels, shape):
            assert extent.setdefault(l, d) == d
    summed = "".join(sorted(l for l in extent if l not in out))
    labels = out + summed
    strides = []
    for lab, shape in zip(ins, shapes):
        st = [int(np.prod(shape[j + 1:], dtype=np.int64)) for j in range(len(shape))]
        row = [0] * len(labels)
        for j, l in enumerate(lab):
            row[labels.index(l)] += st[j]
        strides.append(row)
    return labels, len(out), [extent[l] for l in labels], strides, [extent[l] for l in out]


def einsum_f32(equation, operands):
    """Einsum as the reference's emitted loop nest computes it (ROperator_Einsum.hxx:236-278)."""
    xs = [np.ascontiguousarray(x, np.float32) for x in operands]
    labels, n_out, extent, strides, oshape = einsum_plan(equation, [x.shape for x in xs])
    y = np.empty(oshape, np.float32)
    ptrs = (C.c_void_p * len(xs))(*[x.ctypes.data for x in xs])
    ext = (C.c_int * max(1, len(labels)))(*extent)
    flat = [v for row in strides for v in row]
    st = (C.c_longlong * max(1, len(flat)))(*flat)
    _einsum(len(xs), ptrs, len(labels), n_out, ext, st, y.reshape(-1))
    return y


def _pool_out(H, W, k, pads, s):
    return ((H + pads[0] + pads[2] - k[0]) // s[0] + 1, (W + pads[1] + pads[3] - k[1]) // s[1] + 1)


def maxpool2d(x, kernel, strides, pads=(0, 0, 0, 0)):
    """pads = (top, left, bottom, right), the ONNX order."""
    x = np.ascontiguousarray(x)
    N, Cc, H, W = x.shape
    OH, OW = _pool_out(H, W, kernel, pads, strides)
    y = np.empty((N, Cc, OH, OW), x.dtype)
    fn = _maxpool if x.dtype == np.float32 else _maxpool_s8
    fn(x, y, N * Cc, H, W, kernel[0], kernel[1], pads[0], pads[1], pads[2], pads[3],
       strides[0], strides[1])
    return y


def avgpool2d(x, kernel, strides, pads=(0, 0, 0, 0), count_include_pad=False):
    """fp32 NCHW average pooling (ROperator_Pool.hxx:371-416); pads = (top, left, bottom, right)."""
    x = np.ascontiguousarray(x, np.float32)
    N, Cc, H, W = x.shape
    OH, OW = _pool_out(H, W, kernel, pads, strides)
    y = np.empty((N, Cc, OH, OW), np.float32)
    _avgpool(x, y, N * Cc, H, W, kernel[0], kernel[1], pads[0], pads[1], pads[2], pads[3], strides[0], strides[1],
             int(count_include_pad))
    return y


def pool3d(x, kernel, strides, pads=(0, 0, 0, 0, 0, 0), average=False, count_include_pad=False):
    """fp32 [N, C, D0, D1, D2] pooling (ROperator_Pool.hxx:417-470); pads = three begin pads, then three end pads."""
    x = np.ascontiguousarray(x, np.float32)
    N, Cc = x.shape[:2]
    D = x.shape[2:]
    out = tuple((D[i] + pads[i] + pads[3 + i] - kernel[i]) // strides[i] + 1 for i in range(3))
    y = np.empty((N, Cc) + out, np.float32)
    arr = lambda v: (C.c_int * len(v))(*[int(e) for e in v])
    _pool3d(x, y, N * Cc, arr(D), arr(kernel), arr(pads), arr(strides), int(average), int(count_include_pad))
    return y


def requant_one(acc, scale, zp=0, relu=False):
    return int(_requant_one(int(acc), float(scale), int(zp), int(relu)))


def quantize_f32_s8(x, scale, zp=0):
    x = np.ascontiguousarray(x, np.float32)
    q = np.empty(x.shape, np.int8)
    _quant(x.reshape(-1), q.reshape(-1), x.size, scale, zp)
    return q


def dequantize_s8_f32(q, scale, zp=0):
    q = np.ascontiguousarray(q, np.int8)
    x = np.empty(q.shape, np.float32)
    _dequant(q.reshape(-1), x.reshape(-1), q.size, scale, zp)
    return x


def _mnk(A, B, transB):
    M, K = A.shape
    N = B.shape[0] if transB else B.shape[1]
    assert (B.shape[1] if transB else B.shape[0]) == K
    return M, N, K


def igemm_s8(A, B, transB=False, zpa=0, zpb=0):
    A = np.ascontiguousarray(A, np.int8)
    B = np.ascontiguousarray(B, np.int8)
    M, N, K = _mnk(A, B, transB)
    acc = np.empty((M, N), np.int32)
    _igemm(int(transB), M, N, K, A, B, zpa, zpb, acc)
    return acc


def qgemm_s8(A, B, scale, bias=None, transB=False, zpa=0, zpy=0, relu=False):
    A = np.ascontiguousarray(A, np.int8)
    B = np.ascontiguousarray(B, np.int8)
    M, N, K = _mnk(A, B, transB)
    scale = np.ascontiguousarray(scale, np.float32)
    Y = np.empty((M, N), np.int8)
    _qgemm(int(transB), M, N, K, A, B, zpa, scale, _opt(bias, np.int32), zpy, int(relu), Y)
    return Y


def qgemm_s8_f32out(A, B, scale, bias=None, transB=False, zpa=0, relu=False):
    A = np.ascontiguousarray(A, np.int8)
    B = np.ascontiguousarray(B, np.int8)
    M, N, K = _mnk(A, B, transB)
    scale = np.ascontiguousarray(scale, np.float32)
    Y = np.empty((M, N), np.float32)
    _qgemm_f(int(transB), M, N, K, A, B, zpa, scale, _opt(bias, np.int32), int(relu), Y)
    return Y


def iconv2d_s8(x, w, pads=(0, 0), strides=(1, 1), groups=1, zpx=0):
    x, pads = _pads_hw(np.asarray(x, np.int8), pads, zpx)
    x = np.ascontiguousarray(x, np.int8)
    w = np.ascontiguousarray(w, np.int8)
    N, Cc, H, W = x.shape
    OC, _, kh, kw = w.shape
    OH, OW = conv_out_hw(H, W, kh, kw, pads[0], pads[1], strides[0], strides[1])
    acc = np.empty((N, OC, OH, OW), np.int32)
    rc = _iconv(x, w, acc, N, Cc, H, W, OC, kh, kw, pads[0], pads[1], strides[0], strides[1],
                groups, zpx)
    if rc:
        raise RuntimeError("or_iconv2d_s8 failed: %d" % rc)
    return acc


def qconv2d_s8(x, w, scale, bias=None, pads=(0, 0), strides=(1, 1), groups=1, zpx=0, zpy=0,
               relu=False):
    x, pads = _pads_hw(np.asarray(x, np.int8), pads, zpx)
    x = np.ascontiguousarray(x, np.int8)
    w = np.ascontiguousarray(w, np.int8)
    N, Cc, H, W = x.shape
    OC, _, kh, kw = w.shape
    OH, OW = conv_out_hw(H, W, kh, kw, pads[0], pads[1], strides[0], strides[1])
    scale = np.ascontiguousarray(scale, np.float32)
    y = np.empty((N, OC, OH, OW), np.int8)
    rc = _qconv(x, w, _opt(bias, np.int32), scale, y, N, Cc, H, W, OC, kh, kw, pads[0], pads[1],
                strides[0], strides[1], groups, zpx, zpy, int(relu))
    if rc:
        raise RuntimeError("or_qconv2d_s8 failed: %d" % rc)
    return y


def e4m3_table():
    """All 256 e4m3 code points decoded to float32."""
    return np.array([_e4m3_dec(i) for i in range(256)], np.float32)


def e4m3_decode(codes):
    return e4m3_table()[np.asarray(codes, np.uint8)]


def e4m3_encode(x):
    """fp32 -> e4m3 codes, RNE, saturating at +-448."""
    x = np.asarray(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    flat_in, flat_out = x.reshape(-1), out.reshape(-1)
    for i in range(flat_in.size):
        flat_out[i] = _e4m3_enc(float(flat_in[i]))
    return out


def bf16_encode(x):
    x = np.asarray(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    fi, fo = x.reshape(-1), out.reshape(-1)
    for i in range(fi.size):
        fo[i] = _bf16_enc(float(fi[i]))
    return out


def bf16_decode(b):
    b = np.asarray(b, np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def gemm_fp8(A, B, sa, sb, bias=None, transB=False, acc64=False):
    """Returns (bf16 bit patterns [M,N] uint16, fp32 values [M,N])."""
    A = np.ascontiguousarray(A, np.uint8)
    B = np.ascontiguousarray(B, np.uint8)
    M, N, K = _mnk(A, B, transB)
    yb = np.empty((M, N), np.uint16)
    yf = np.empty((M, N), np.float32)
    _gemm_fp8(int(transB), M, N, K, A, B, sa, sb, _opt(bias, np.float32),
              yb.ctypes.data_as(C.c_void_p), yf.ctypes.data_as(C.c_void_p), int(acc64))
    return yb, yf
