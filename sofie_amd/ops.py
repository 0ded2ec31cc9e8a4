"""Operator front end over the C ABI: numpy or torch arrays in, same kind out.

torch is used only to own device memory and the stream; every computation is a call into
libsofie_hip.so. The function names and argument meanings mirror what the reference's
operators compute (ROperator_Gemm, ROperator_Conv, ROperator_Relu, ROperator_Pool) plus the
quantized / FP8 operators this library adds.
"""
import ctypes as C

import numpy as np
import torch

from . import lib as L


class SofieHipError(RuntimeError):
    pass


GUARD_BYTES = 512          # sentinel band on either side of every output buffer (a multiple of 256: keeps alignment)
GUARD_VALUE = 0xA5


class Context:
    """One sofie_hip_ctx on `device`. The library launches on torch's current stream when that is a stream of
    its own; with torch's default (null) stream the handle is NULL and sofie_hip_create opens a blocking stream,
    which the null stream's implicit synchronisation orders against torch's own work (copies, fills).

    Every output buffer that `empty` hands out lies between two sentinel bands that `ret` checks after the
    call: a store outside the tensor (a ragged tile written past its edge) raises instead of going unseen."""

    def __init__(self, device=0, guard=True, stream=None):
        if not torch.cuda.is_available():
            raise SofieHipError("no GPU visible: the HIP library has no CPU fallback")
        self.lib = L.load()
        self.device = torch.device("cuda", device)
        torch.cuda.set_device(self.device)
        self.stream = stream if stream is not None else torch.cuda.current_stream(self.device)
        h = C.c_void_p()
        rc = self.lib.sofie_hip_create(C.byref(h), device, C.c_void_p(self.stream.cuda_stream))
        if rc:
            raise SofieHipError("sofie_hip_create failed: %d" % rc)
        self.h = h
        self.guard = guard
        self._guarded = []

    def close(self):
        if self.h:
            self.lib.sofie_hip_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def check(self, rc):
        if rc:
            msg = self.lib.sofie_hip_last_error(self.h).decode()
            raise SofieHipError("%s (status %d)" % (msg, rc))

    def sync(self):
        """Waits for the stream, then checks the sentinel bands of the buffers handed out since the last wait."""
        self.check(self.lib.sofie_hip_sync(self.h))
        self._check_guards()

    def timer_start(self):
        self.check(self.lib.sofie_hip_timer_start(self.h))

    def timer_stop(self):
        ms = C.c_float()
        self.check(self.lib.sofie_hip_timer_stop(self.h, C.byref(ms)))
        return ms.value

    # -- helpers ---------------------------------------------------------------------
    def dev(self, a, dtype=None):
        """numpy/torch -> contiguous device tensor (no copy if already there)."""
        if a is None:
            return None
        if isinstance(a, np.ndarray):
            a = torch.from_numpy(np.ascontiguousarray(a))
        if dtype is not None and a.dtype != dtype:
            a = a.to(dtype)
        return a.to(self.device).contiguous()

    @staticmethod
    def ptr(t):
        return C.c_void_p(t.data_ptr()) if t is not None else None

    def empty(self, shape, dtype):
        if not self.guard:
            return torch.empty(shape, dtype=dtype, device=self.device)
        shape = tuple(int(d) for d in shape)
        n = int(np.prod(shape, dtype=np.int64)) * torch.empty((), dtype=dtype).element_size()
        raw = torch.empty(2 * GUARD_BYTES + n, dtype=torch.uint8, device=self.device)
        raw[:GUARD_BYTES] = GUARD_VALUE
        raw[GUARD_BYTES + n:] = GUARD_VALUE
        self._guarded.append((raw, n))
        return raw[GUARD_BYTES:GUARD_BYTES + n].view(dtype).view(shape)

    def verify_guards(self):
        if self._guarded:
            self.sync()

    def _check_guards(self):
        pending, self._guarded = self._guarded, []
        for raw, n in pending:
            lo, hi = raw[:GUARD_BYTES], raw[GUARD_BYTES + n:]
            if not (bool((lo == GUARD_VALUE).all()) and bool((hi == GUARD_VALUE).all())):
                bad_lo = int((lo != GUARD_VALUE).sum())
                bad_hi = int((hi != GUARD_VALUE).sum())
                raise SofieHipError("a kernel wrote outside its output buffer of %d bytes: %d bytes changed in front of it, "
                                    "%d behind it" % (n, bad_lo, bad_hi))

    def ret(self, t, like):
        self.verify_guards()
        return t.cpu().numpy() if isinstance(like, np.ndarray) else t


_default = None


def default_context():
    global _default
    if _default is None:
        _default = Context(0)
    return _default


# ------------------------------------------------------------------------------- fp32
def gemm_f32(A, B, bias=None, alpha=1.0, beta=1.0, transA=False, transB=False, relu=False, ctx=None):
    """Y = alpha*op(A)*op(B) + beta*bias [ReLU]; bias rank-1 [N] or full [M,N]."""
    ctx = ctx or default_context()
    a, b = ctx.dev(A, torch.float32), ctx.dev(B, torch.float32)
    M, K = (a.shape[1], a.shape[0]) if transA else a.shape
    N = b.shape[0] if transB else b.shape[1]
    y = ctx.empty((M, N), torch.float32)
    kind, bt = L.BIAS_NONE, None
    if bias is not None:
        bt = ctx.dev(bias, torch.float32)
        if bt.numel() == N and bt.dim() <= 2 and bt.shape[-1] == N:
            kind = L.BIAS_ROW
        elif tuple(bt.shape) == (M, N):
            kind = L.BIAS_FULL
        else:
            raise SofieHipError("bias shape %s cannot be broadcast to (%d, %d)" % (tuple(bt.shape), M, N))
    ctx.check(ctx.lib.sofie_hip_gemm_f32(ctx.h, int(transA), int(transB), M, N, K, alpha, ctx.ptr(a), a.shape[1],
                                         ctx.ptr(b), b.shape[1], beta, ctx.ptr(bt), kind, ctx.ptr(y), N,
                                         L.ACT_RELU if relu else L.ACT_NONE))
    return ctx.ret(y, A)


def mlp_f32(x, weights, biases=None, relus=None, ctx=None):
    """y = act_L(... act_1(x W_1 + b_1) ... W_L + b_L) in one launch; W_l [K_l, N_l], b_l [N_l] or None."""
    ctx = ctx or default_context()
    xd = ctx.dev(x, torch.float32)
    n = len(weights)
    wd = [ctx.dev(w, torch.float32) for w in weights]
    bd = [ctx.dev(b, torch.float32) if biases is not None and b is not None else None for b in (biases or [None] * n)]
    dims = [xd.shape[1]] + [w.shape[1] for w in wd]
    y = ctx.empty((xd.shape[0], dims[-1]), torch.float32)
    c_dims = (C.c_int * (n + 1))(*dims)
    c_w = (C.c_void_p * n)(*[w.data_ptr() for w in wd])
    c_b = (C.c_void_p * n)(*[b.data_ptr() if b is not None else None for b in bd])
    c_a = (C.c_int * n)(*[L.ACT_RELU if (relus and relus[i]) else L.ACT_NONE for i in range(n)])
    ctx.check(ctx.lib.sofie_hip_mlp_f32(ctx.h, n, c_dims, c_w, c_b, c_a, ctx.ptr(xd), xd.shape[1], ctx.ptr(y), dims[-1],
                                        xd.shape[0]))
    return ctx.ret(y, x)


def relu_f32(x, ctx=None):
    ctx = ctx or default_context()
    xd = ctx.dev(x, torch.float32)
    y = ctx.empty(tuple(xd.shape), torch.float32)
    ctx.check(ctx.lib.sofie_hip_relu_f32(ctx.h, ctx.ptr(xd), ctx.ptr(y), xd.numel()))
    return ctx.ret(y, x)


def pads4(pads):
    """(h, w) -> (top, left, bottom, right) with equal begin and end pads; a 4-tuple is ONNX order already."""
    pads = tuple(int(p) for p in pads)
    return pads if len(pads) == 4 else (pads[0], pads[1], pads[0], pads[1])


def conv_out_hw(H, W, kh, kw, pads, sh, sw, dh=1, dw=1):
    pt, pl, pb, pr = pads4(pads)
    return ((H + pt + pb - (dh * (kh - 1) + 1)) // sh + 1, (W + pl + pr - (dw * (kw - 1) + 1)) // sw + 1)


def conv2d_f32(x, w, bias=None, pads=(0, 0), strides=(1, 1), dilations=(1, 1), groups=1, relu=False, ctx=None):
    ctx = ctx or default_context()
    xd, wd, bd = ctx.dev(x, torch.float32), ctx.dev(w, torch.float32), ctx.dev(bias, torch.float32)
    N, Cc, H, W = xd.shape
    OC, _, kh, kw = wd.shape
    OH, OW = conv_out_hw(H, W, kh, kw, pads, strides[0], strides[1], *dilations)
    y = ctx.empty((N, OC, OH, OW), torch.float32)
    ctx.check(ctx.lib.sofie_hip_conv2d_f32(ctx.h, ctx.ptr(xd), ctx.ptr(wd), ctx.ptr(bd), ctx.ptr(y), N, Cc, H, W,
                                           OC, kh, kw, *pads4(pads), strides[0], strides[1], dilations[0],
                                           dilations[1], groups, L.ACT_RELU if relu else L.ACT_NONE))
    return ctx.ret(y, x)


def conv3d_f32(x, w, bias=None, pads=(0, 0, 0), strides=(1, 1, 1), dilations=(1, 1, 1), groups=1, relu=False, ctx=None):
    """NCDHW 3-D convolution; pads are the begin pads (d, h, w), applied on both sides."""
    ctx = ctx or default_context()
    xd, wd, bd = ctx.dev(x, torch.float32), ctx.dev(w, torch.float32), ctx.dev(bias, torch.float32)
    N, Cc, D, H, W = xd.shape
    OC, _, kd, kh, kw = wd.shape
    out = [(i + 2 * p - (d * (k - 1) + 1)) // s + 1 for i, p, d, k, s in zip((D, H, W), pads, dilations, (kd, kh, kw), strides)]
    y = ctx.empty((N, OC, out[0], out[1], out[2]), torch.float32)
    ctx.check(ctx.lib.sofie_hip_conv3d_f32(ctx.h, ctx.ptr(xd), ctx.ptr(wd), ctx.ptr(bd), ctx.ptr(y), N, Cc, D, H, W, OC, kd, kh, kw,
                                           *pads, *strides, *dilations, groups, L.ACT_RELU if relu else L.ACT_NONE))
    return ctx.ret(y, x)


def conv_transpose2d_f32(x, w, bias=None, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), groups=1,
                         output_padding=(0, 0), relu=False, ctx=None):
    """ONNX ConvTranspose, NCHW; w [C, OC/groups, KH, KW]; pads = (top, left, bottom, right)."""
    ctx = ctx or default_context()
    xd, wd, bd = ctx.dev(x, torch.float32), ctx.dev(w, torch.float32), ctx.dev(bias, torch.float32)
    N, Cc, H, W = xd.shape
    _, ocg, kh, kw = wd.shape
    OC = ocg * groups
    OH = strides[0] * (H - 1) + dilations[0] * (kh - 1) + 1 + output_padding[0] - pads[0] - pads[2]
    OW = strides[1] * (W - 1) + dilations[1] * (kw - 1) + 1 + output_padding[1] - pads[1] - pads[3]
    y = ctx.empty((N, OC, OH, OW), torch.float32)
    ctx.check(ctx.lib.sofie_hip_conv_transpose2d_f32(ctx.h, ctx.ptr(xd), ctx.ptr(wd), ctx.ptr(bd), ctx.ptr(y), N, Cc, H,
                                                     W, OC, kh, kw, pads[0], pads[1], strides[0], strides[1],
                                                     dilations[0], dilations[1], groups, OH, OW,
                                                     L.ACT_RELU if relu else L.ACT_NONE))
    return ctx.ret(y, x)


def batchnorm_f32(x, scale, bias, mean, var, epsilon=1e-5, relu=False, ctx=None):
    """Inference BatchNormalization over axis 1; the variance is folded into the scale on the host the way the
    emitter does it: scale * float(1 / sqrt(double(var + epsilon)))."""
    ctx = ctx or default_context()
    xd = ctx.dev(x, torch.float32)
    folded = (np.asarray(scale, np.float32) *
              (1.0 / np.sqrt((np.asarray(var, np.float32) + np.float32(epsilon)).astype(np.float64))).astype(np.float32))
    sd, md, bd = ctx.dev(folded.astype(np.float32), torch.float32), ctx.dev(mean, torch.float32), ctx.dev(bias, torch.float32)
    N, Cc = xd.shape[0], xd.shape[1]
    plane = int(np.prod(xd.shape[2:])) if xd.dim() > 2 else 1
    y = ctx.empty(tuple(xd.shape), torch.float32)
    ctx.check(ctx.lib.sofie_hip_batchnorm_f32(ctx.h, ctx.ptr(xd), ctx.ptr(sd), ctx.ptr(md), ctx.ptr(bd), ctx.ptr(y), N, Cc,
                                              plane, L.ACT_RELU if relu else L.ACT_NONE))
    return ctx.ret(y, x)


def _matrix_product_type(ins, out, summed):
    """The emitter's test (ROperator_Einsum::MatrixProductType): "nn" / "tn" / "nt" / "tt" or ""."""
    if len(ins) != 2 or len(summed) != 1:
        return ""
    la, lb = ins
    if len(la) < 2 or len(lb) < 2 or len(out) < 2 or len(set(la)) != len(la) or len(set(lb)) != len(lb):
        return ""
    s = summed[0]
    pa, pb = la.find(s), lb.find(s)
    if pa < len(la) - 2 or pb < len(lb) - 2:
        return ""
    ta, tb = pa == len(la) - 2, pb == len(lb) - 1
    m = la[-1] if ta else la[-2]
    n = lb[-2] if tb else lb[-1]
    if m == n or out[-2] != m or out[-1] != n or m in lb or n in la:
        return ""
    if any(l not in out[:-2] for l in la[:-2] + lb[:-2]):
        return ""
    return ("t" if ta else "n") + ("t" if tb else "n")


def einsum_f32(equation, operands, ctx=None):
    """Einsum the way the emitted Session runs it: a (stacked) matrix product as one sofie_hip_gemm_f32 call per
    stacked matrix, anything else as one sofie_hip_einsum_f32 call."""
    ctx = ctx or default_context()
    xs = [ctx.dev(x, torch.float32).contiguous() for x in operands]
    eq = equation.replace(" ", "")
    lhs, out = eq.split("->")
    ins = lhs.split(",")
    extent = {}
    for labels, x in zip(ins, xs):
        if len(labels) != x.dim():
            raise SofieHipError("operand of rank %d with labels %s" % (x.dim(), labels))
        for l, d in zip(labels, x.shape):
            if extent.setdefault(l, int(d)) != int(d):
                raise SofieHipError("label %s has two sizes" % l)
    summed = "".join(sorted(l for l in extent if l not in out))
    oshape = tuple(extent[l] for l in out)
    y = ctx.empty(oshape if oshape else (1,), torch.float32)
    kind = _matrix_product_type(ins, out, summed)
    if kind:
        a, b = xs
        ta, tb = kind[0] == "t", kind[1] == "t"
        M = a.shape[-1] if ta else a.shape[-2]
        K = a.shape[-2] if ta else a.shape[-1]
        N = b.shape[-2] if tb else b.shape[-1]
        lead = out[:-2]
        y3 = y.view(-1, M, N)
        for idx in range(y3.shape[0]):
            pos, rem = {}, idx
            for l in reversed(lead):
                pos[l] = rem % extent[l]
                rem //= extent[l]
            am = a[tuple(pos[l] for l in ins[0][:-2])]
            bm = b[tuple(pos[l] for l in ins[1][:-2])]
            ctx.check(ctx.lib.sofie_hip_gemm_f32(ctx.h, int(ta), int(tb), M, N, K, 1.0, ctx.ptr(am), a.shape[-1], ctx.ptr(bm),
                                                 b.shape[-1], 0.0, None, L.BIAS_NONE, ctx.ptr(y3[idx]), N, L.ACT_NONE))
    else:
        labels = out + summed
        strides = []
        for lab, x in zip(ins, xs):
            row = [0] * len(labels)
            for j, l in enumerate(lab):
                row[labels.index(l)] += int(x.stride(j))
            strides += row
        ptrs = (C.c_void_p * len(xs))(*[x.data_ptr() for x in xs])
        ext = (C.c_int * max(1, len(labels)))(*[extent[l] for l in labels])
        st = (C.c_longlong * max(1, len(strides)))(*strides)
        ctx.check(ctx.lib.sofie_hip_einsum_f32(ctx.h, len(xs), ptrs, len(labels), len(out), ext, st, ctx.ptr(y)))
    y = y.view(oshape)
    return ctx.ret(y, operands[0])


def maxpool2d(x, kernel, strides, pads=(0, 0, 0, 0), layout=L.LAYOUT_NCHW, ctx=None):
    """pads = (top, left, bottom, right). int8 tensors may be NHWC (layout flag); fp32 is NCHW."""
    ctx = ctx or default_context()
    xd = ctx.dev(x)
    if layout == L.LAYOUT_NCHW:
        N, Cc, H, W = xd.shape
    else:
        N, H, W, Cc = xd.shape
    OH = (H + pads[0] + pads[2] - kernel[0]) // strides[0] + 1
    OW = (W + pads[1] + pads[3] - kernel[1]) // strides[1] + 1
    shape = (N, Cc, OH, OW) if layout == L.LAYOUT_NCHW else (N, OH, OW, Cc)
    y = ctx.empty(shape, xd.dtype)
    if xd.dtype == torch.float32:
        ctx.check(ctx.lib.sofie_hip_maxpool2d_f32(ctx.h, ctx.ptr(xd), ctx.ptr(y), N * Cc, H, W, kernel[0],
                                                  kernel[1], pads[0], pads[1], pads[2], pads[3], strides[0],
                                                  strides[1]))
    else:
        ctx.check(ctx.lib.sofie_hip_maxpool2d_s8(ctx.h, ctx.ptr(xd), ctx.ptr(y), layout, N, Cc, H, W, kernel[0],
                                                 kernel[1], pads[0], pads[1], pads[2], pads[3], strides[0],
                                                 strides[1]))
    return ctx.ret(y, x)


def avgpool2d(x, kernel, strides, pads=(0, 0, 0, 0), count_include_pad=False, ctx=None):
    """fp32 NCHW average pooling; pads = (top, left, bottom, right)."""
    ctx = ctx or default_context()
    xd = ctx.dev(x, torch.float32)
    N, Cc, H, W = xd.shape
    OH = (H + pads[0] + pads[2] - kernel[0]) // strides[0] + 1
    OW = (W + pads[1] + pads[3] - kernel[1]) // strides[1] + 1
    y = ctx.empty((N, Cc, OH, OW), torch.float32)
    ctx.check(ctx.lib.sofie_hip_avgpool2d_f32(ctx.h, ctx.ptr(xd), ctx.ptr(y), N * Cc, H, W, kernel[0], kernel[1], pads[0],
                                              pads[1], pads[2], pads[3], strides[0], strides[1], int(count_include_pad)))
    return ctx.ret(y, x)


def pool3d(x, kernel, strides, pads=(0, 0, 0, 0, 0, 0), average=False, count_include_pad=False, ctx=None):
    """fp32 [N, C, D0, D1, D2] max or average pooling; pads = the three begin pads, then the three end pads."""
    import ctypes as C
    ctx = ctx or default_context()
    xd = ctx.dev(x, torch.float32)
    N, Cc = xd.shape[:2]
    dims = tuple(xd.shape[2:])
    out = tuple((dims[i] + pads[i] + pads[3 + i] - kernel[i]) // strides[i] + 1 for i in range(3))
    y = ctx.empty((N, Cc) + out, torch.float32)
    arr = lambda v: (C.c_int * len(v))(*[int(e) for e in v])
    d, k, p, s = arr(dims), arr(kernel), arr(pads), arr(strides)
    if average:
        ctx.check(ctx.lib.sofie_hip_avgpool3d_f32(ctx.h, ctx.ptr(xd), ctx.ptr(y), N * Cc, d, k, p, s, int(count_include_pad)))
    else:
        ctx.check(ctx.lib.sofie_hip_maxpool3d_f32(ctx.h, ctx.ptr(xd), ctx.ptr(y), N * Cc, d, k, p, s))
    return ctx.ret(y, x)


# ------------------------------------------------------------------------------- int8
def quantize_f32_s8(x, scale, zp=0, ctx=None):
    ctx = ctx or default_context()
    xd = ctx.dev(x, torch.float32)
    q = ctx.empty(xd.shape, torch.int8)
    ctx.check(ctx.lib.sofie_hip_quantize_f32_s8(ctx.h, ctx.ptr(xd), ctx.ptr(q), xd.numel(), float(scale), int(zp)))
    return ctx.ret(q, x)


def dequantize_s8_f32(q, scale, zp=0, ctx=None):
    ctx = ctx or default_context()
    qd = ctx.dev(q, torch.int8)
    x = ctx.empty(qd.shape, torch.float32)
    ctx.check(ctx.lib.sofie_hip_dequantize_s8_f32(ctx.h, ctx.ptr(qd), ctx.ptr(x), qd.numel(), float(scale), int(zp)))
    return ctx.ret(x, q)


_OUT_DTYPE = {L.OUT_S8: torch.int8, L.OUT_F32: torch.float32, L.OUT_S32: torch.int32, L.OUT_BF16: torch.bfloat16}


def fold_zero_point_gemm(B, bias, zpa, transB=False):
    """bias[n] - zp_a * sum_k B[k,n]: lets the kernel accumulate raw A values (host side, once)."""
    Bn = np.asarray(B.cpu() if isinstance(B, torch.Tensor) else B).astype(np.int64)
    colsum = Bn.sum(axis=1 if transB else 0)
    base = np.zeros(colsum.shape, np.int64) if bias is None else \
        np.asarray(bias.cpu() if isinstance(bias, torch.Tensor) else bias).astype(np.int64)
    return (base - int(zpa) * colsum).astype(np.int32)


def qgemm_s8(A, B, scale, bias=None, transB=False, zpa=0, zpy=0, relu=False, out=L.OUT_S8, ctx=None):
    """int8 GEMM, int32 accumulate, per-column scale; out: OUT_S8 / OUT_F32 / OUT_S32."""
    ctx = ctx or default_context()
    if zpa != 0:
        bias = fold_zero_point_gemm(B, bias, zpa, transB)
    a, b = ctx.dev(A, torch.int8), ctx.dev(B, torch.int8)
    M, K = a.shape
    N = b.shape[0] if transB else b.shape[1]
    sd, bd = ctx.dev(scale, torch.float32), ctx.dev(bias, torch.int32)
    y = ctx.empty((M, N), _OUT_DTYPE[out])
    ctx.check(ctx.lib.sofie_hip_qgemm_s8(ctx.h, int(transB), M, N, K, ctx.ptr(a), a.shape[1], ctx.ptr(b),
                                         b.shape[1], ctx.ptr(sd), ctx.ptr(bd), int(zpy),
                                         L.ACT_RELU if relu else L.ACT_NONE, ctx.ptr(y), N, out))
    return ctx.ret(y, A)


def qgemm_s8_pair(A, B1, scale1, bias1, zp_mid, relu1, B2, scale2, bias2, zpy=0, relu2=False, out=L.OUT_S8, ctx=None):
    """Two QLinearMatMul layers in one call; B1 [N1, K] and B2 [N2, N1] (K-contiguous), biases with the zero-points
    of their inputs already folded in."""
    ctx = ctx or default_context()
    a, b1, b2 = ctx.dev(A, torch.int8), ctx.dev(B1, torch.int8), ctx.dev(B2, torch.int8)
    M, K = a.shape
    N1, N2 = b1.shape[0], b2.shape[0]
    s1, s2 = ctx.dev(scale1, torch.float32), ctx.dev(scale2, torch.float32)
    q1, q2 = ctx.dev(bias1, torch.int32), ctx.dev(bias2, torch.int32)
    mid = ctx.empty((M, N1), torch.int8)
    y = ctx.empty((M, N2), _OUT_DTYPE[out])
    ctx.check(ctx.lib.sofie_hip_qgemm_s8_pair(ctx.h, M, K, ctx.ptr(a), K, N1, ctx.ptr(b1), K, ctx.ptr(s1), ctx.ptr(q1),
                                              int(zp_mid), L.ACT_RELU if relu1 else L.ACT_NONE, ctx.ptr(mid), N1, N2,
                                              ctx.ptr(b2), N1, ctx.ptr(s2), ctx.ptr(q2), int(zpy),
                                              L.ACT_RELU if relu2 else L.ACT_NONE, ctx.ptr(y), N2, out))
    return ctx.ret(y, A)


def qgemm_s8_f32out(A, B, scale, bias=None, transB=False, zpa=0, relu=False, ctx=None):
    return qgemm_s8(A, B, scale, bias, transB, zpa, 0, relu, L.OUT_F32, ctx)


def igemm_s8(A, B, transB=False, ctx=None):
    return qgemm_s8(A, B, None, None, transB, out=L.OUT_S32, ctx=ctx)


def fold_zero_point_conv(w, bias, zpx):
    wn = np.asarray(w.cpu() if isinstance(w, torch.Tensor) else w).astype(np.int64)
    wsum = wn.reshape(wn.shape[0], -1).sum(axis=1)
    base = np.zeros(wsum.shape, np.int64) if bias is None else \
        np.asarray(bias.cpu() if isinstance(bias, torch.Tensor) else bias).astype(np.int64)
    return (base - int(zpx) * wsum).astype(np.int32)


def qconv2d_s8(x, w, scale, bias=None, pads=(0, 0), strides=(1, 1), groups=1, zpx=0, zpy=0, relu=False,
               x_layout=L.LAYOUT_NCHW, y_layout=L.LAYOUT_NCHW, out=L.OUT_S8, ctx=None, w_layout=L.LAYOUT_NCHW):
    """QLinearConv. x in x_layout, w [OC, C/g, KH, KW] (or [OC, KH, KW, C/g] with w_layout NHWC); bias is
    the ONNX int32 bias (the input zero-point is folded here, host side, as a Session constructor would
    do once)."""
    ctx = ctx or default_context()
    if zpx != 0:
        bias = fold_zero_point_conv(w, bias, zpx)
    xd, wd = ctx.dev(x, torch.int8), ctx.dev(w, torch.int8)
    if x_layout == L.LAYOUT_NCHW:
        N, Cc, H, W = xd.shape
    else:
        N, H, W, Cc = xd.shape
    if w_layout == L.LAYOUT_NCHW:
        OC, _, kh, kw = wd.shape
    else:
        OC, kh, kw, _ = wd.shape
    OH, OW = conv_out_hw(H, W, kh, kw, pads, strides[0], strides[1])
    shape = (N, OC, OH, OW) if y_layout == L.LAYOUT_NCHW else (N, OH, OW, OC)
    y = ctx.empty(shape, _OUT_DTYPE[out])
    sd, bd = ctx.dev(scale, torch.float32), ctx.dev(bias, torch.int32)
    ctx.check(ctx.lib.sofie_hip_qconv2d_s8(ctx.h, ctx.ptr(xd), x_layout, ctx.ptr(wd), w_layout, ctx.ptr(bd), ctx.ptr(sd),
                                           ctx.ptr(y), y_layout, N, Cc, H, W, OC, kh, kw, *pads4(pads),
                                           strides[0], strides[1], groups, int(zpx), int(zpy),
                                           L.ACT_RELU if relu else L.ACT_NONE, out))
    return ctx.ret(y, x)


def qconv2d_pool_s8(x, w, scale, bias=None, pads=(0, 0), strides=(1, 1), groups=1, zpx=0, zpy=0, relu=False,
                    pool=(2, 2), pool_strides=(2, 2), x_layout=L.LAYOUT_NCHW, y_layout=L.LAYOUT_NCHW, ctx=None,
                    w_layout=L.LAYOUT_NCHW):
    """QLinearConv -> (ReLU) -> MaxPool(pool, pool_strides, no pads) in one library call."""
    ctx = ctx or default_context()
    if zpx != 0:
        bias = fold_zero_point_conv(w, bias, zpx)
    xd, wd = ctx.dev(x, torch.int8), ctx.dev(w, torch.int8)
    if x_layout == L.LAYOUT_NCHW:
        N, Cc, H, W = xd.shape
    else:
        N, H, W, Cc = xd.shape
    if w_layout == L.LAYOUT_NCHW:
        OC, _, kh, kw = wd.shape
    else:
        OC, kh, kw, _ = wd.shape
    OH, OW = conv_out_hw(H, W, kh, kw, pads, strides[0], strides[1])
    PH, PW = (OH - pool[0]) // pool_strides[0] + 1, (OW - pool[1]) // pool_strides[1] + 1
    y = ctx.empty((N, OC, PH, PW) if y_layout == L.LAYOUT_NCHW else (N, PH, PW, OC), torch.int8)
    sd, bd = ctx.dev(scale, torch.float32), ctx.dev(bias, torch.int32)
    ctx.check(ctx.lib.sofie_hip_qconv2d_pool_s8(ctx.h, ctx.ptr(xd), x_layout, ctx.ptr(wd), w_layout, ctx.ptr(bd),
                                                ctx.ptr(sd), ctx.ptr(y), y_layout, N, Cc, H, W, OC, kh, kw, *pads4(pads),
                                                strides[0], strides[1], groups, int(zpx), int(zpy),
                                                L.ACT_RELU if relu else L.ACT_NONE, pool[0], pool[1], pool_strides[0],
                                                pool_strides[1]))
    return ctx.ret(y, x)


def quantize_qconv2d_s8(x, x_scale, zpx, w, scale, bias=None, pads=(0, 0), strides=(1, 1), groups=1, zpy=0, relu=False,
                        pool=None, pool_strides=(2, 2), y_layout=L.LAYOUT_NCHW, w_layout=L.LAYOUT_NCHW, ctx=None):
    """QuantizeLinear(x float NCHW) -> QLinearConv -> (ReLU) -> (MaxPool) in one library call."""
    ctx = ctx or default_context()
    if zpx != 0:
        bias = fold_zero_point_conv(w, bias, zpx)
    xd, wd = ctx.dev(x, torch.float32), ctx.dev(w, torch.int8)
    N, Cc, H, W = xd.shape
    if w_layout == L.LAYOUT_NCHW:
        OC, _, kh, kw = wd.shape
    else:
        OC, kh, kw, _ = wd.shape
    OH, OW = conv_out_hw(H, W, kh, kw, pads, strides[0], strides[1])
    if pool:
        OH, OW = (OH - pool[0]) // pool_strides[0] + 1, (OW - pool[1]) // pool_strides[1] + 1
    y = ctx.empty((N, OC, OH, OW) if y_layout == L.LAYOUT_NCHW else (N, OH, OW, OC), torch.int8)
    sd, bd = ctx.dev(scale, torch.float32), ctx.dev(bias, torch.int32)
    pk = pool or (0, 0)
    ctx.check(ctx.lib.sofie_hip_quantize_qconv2d_s8(ctx.h, ctx.ptr(xd), float(x_scale), int(zpx), ctx.ptr(wd), w_layout,
                                                    ctx.ptr(bd), ctx.ptr(sd), ctx.ptr(y), y_layout, N, Cc, H, W, OC, kh, kw,
                                                    *pads4(pads), strides[0], strides[1], groups, int(zpy),
                                                    L.ACT_RELU if relu else L.ACT_NONE, pk[0], pk[1],
                                                    pool_strides[0] if pool else 0, pool_strides[1] if pool else 0))
    return ctx.ret(y, x)


def qconv2d_s8_chain(x, layers, x_layout=L.LAYOUT_NHWC, ctx=None):
    """A chain of QLinearConv layers in one library call (sofie_hip_qconv2d_s8_chain). `layers` is a list of dicts with
    the keyword arguments of qconv2d_s8 / qconv2d_pool_s8: w, scale, bias, pads, strides, groups, zpx, zpy, relu,
    pool (None or (kh, kw)), pool_strides, y_layout, w_layout. Returns the list of every layer's output."""
    ctx = ctx or default_context()
    xd = ctx.dev(x, torch.int8)
    if x_layout == L.LAYOUT_NCHW:
        N, Cc, H, W = xd.shape
    else:
        N, H, W, Cc = xd.shape
    descs = (L.QConvLayer * len(layers))()
    keep, outs = [], []
    for d, q in zip(descs, layers):
        w, pads, strides = q["w"], q.get("pads", (0, 0)), q.get("strides", (1, 1))
        bias = fold_zero_point_conv(w, q.get("bias"), q.get("zpx", 0)) if q.get("zpx", 0) != 0 else q.get("bias")
        w_layout, y_layout = q.get("w_layout", L.LAYOUT_NCHW), q.get("y_layout", L.LAYOUT_NHWC)
        wd = ctx.dev(w, torch.int8)
        if w_layout == L.LAYOUT_NCHW:
            OC, _, kh, kw = wd.shape
        else:
            OC, kh, kw, _ = wd.shape
        OH, OW = conv_out_hw(H, W, kh, kw, pads, strides[0], strides[1])
        pool, ps = q.get("pool"), q.get("pool_strides", (2, 2))
        if pool:
            OH, OW = (OH - pool[0]) // ps[0] + 1, (OW - pool[1]) // ps[1] + 1
        y = ctx.empty((N, OC, OH, OW) if y_layout == L.LAYOUT_NCHW else (N, OH, OW, OC), torch.int8)
        sd, bd = ctx.dev(q["scale"], torch.float32), ctx.dev(bias, torch.int32)
        keep += [wd, sd, bd]
        d.w, d.w_layout, d.bias, d.scale = wd.data_ptr(), w_layout, (bd.data_ptr() if bd is not None else None), sd.data_ptr()
        d.y, d.y_layout = y.data_ptr(), y_layout
        d.C, d.H, d.W, d.OC, d.KH, d.KW = Cc, H, W, OC, kh, kw
        d.pad_top, d.pad_left, d.pad_bottom, d.pad_right = pads4(pads)
        d.stride_h, d.stride_w, d.groups = strides[0], strides[1], q.get("groups", 1)
        d.zp_x, d.zp_y, d.act = int(q.get("zpx", 0)), int(q.get("zpy", 0)), L.ACT_RELU if q.get("relu") else L.ACT_NONE
        d.pool_kh, d.pool_kw = (pool[0], pool[1]) if pool else (0, 0)
        d.pool_stride_h, d.pool_stride_w = (ps[0], ps[1]) if pool else (0, 0)
        outs.append(y)
        Cc, H, W = OC, OH, OW
    ctx.check(ctx.lib.sofie_hip_qconv2d_s8_chain(ctx.h, ctx.ptr(xd), x_layout, N, len(layers), descs))
    ctx.verify_guards()
    return [o.cpu().numpy() if isinstance(x, np.ndarray) else o for o in outs]


def iconv2d_s8(x, w, pads=(0, 0), strides=(1, 1), groups=1, zpx=0, ctx=None):
    return qconv2d_s8(x, w, None, None, pads, strides, groups, zpx, out=L.OUT_S32, ctx=ctx)


def relayout_s8(x, from_layout, to_layout, ctx=None):
    ctx = ctx or default_context()
    xd = ctx.dev(x, torch.int8)
    if from_layout == L.LAYOUT_NCHW:
        N, Cc, H, W = xd.shape
    else:
        N, H, W, Cc = xd.shape
    shape = (N, Cc, H, W) if to_layout == L.LAYOUT_NCHW else (N, H, W, Cc)
    y = ctx.empty(shape, torch.int8)
    ctx.check(ctx.lib.sofie_hip_relayout_s8(ctx.h, ctx.ptr(xd), ctx.ptr(y), N, Cc, H, W, from_layout, to_layout))
    return ctx.ret(y, x)


# ------------------------------------------------------------------------------- fp8
def quantize_f32_e4m3(x, inv_scale, ctx=None):
    ctx = ctx or default_context()
    xd = ctx.dev(x, torch.float32)
    q = ctx.empty(xd.shape, torch.uint8)
    ctx.check(ctx.lib.sofie_hip_quantize_f32_e4m3(ctx.h, ctx.ptr(xd), ctx.ptr(q), xd.numel(), float(inv_scale)))
    return ctx.ret(q, x)


def gemm_fp8(A, B, sa, sb, bias=None, transB=False, out=L.OUT_BF16, ctx=None):
    """e4m3 codes (uint8) in; returns bf16 bit patterns as uint16 (numpy) / bfloat16 tensor, or fp32."""
    ctx = ctx or default_context()
    a, b = ctx.dev(A, torch.uint8), ctx.dev(B, torch.uint8)
    M, K = a.shape
    N = b.shape[0] if transB else b.shape[1]
    bd = ctx.dev(bias, torch.float32)
    y = ctx.empty((M, N), _OUT_DTYPE[out])
    ctx.check(ctx.lib.sofie_hip_gemm_fp8(ctx.h, int(transB), M, N, K, ctx.ptr(a), a.shape[1], ctx.ptr(b),
                                         b.shape[1], float(sa), float(sb), ctx.ptr(bd), ctx.ptr(y), N, out))
    ctx.verify_guards()
    if isinstance(A, np.ndarray):
        if out == L.OUT_BF16:
            return y.view(torch.int16).cpu().numpy().view(np.uint16)
        return y.cpu().numpy()
    return y
