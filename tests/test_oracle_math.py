"""Pins the CPU oracle with facts that do not depend on its own formulas: float64 /
int64 closed forms, torch CPU operators, brute force on tiny inputs, exact rational
rounding, and library fp8 / bf16 casts. The reference has no quantized or FP8 operators,
so for those these checks are the only pin ("parity unpinned" by the reference)."""
from fractions import Fraction

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle


def rng(seed):
    return np.random.default_rng(seed)


# ----------------------------------------------------------------------------- fp32 Gemm
@pytest.mark.parametrize("transA,transB,alpha,beta,relu", [
    (0, 0, 1.0, 1.0, False), (0, 1, 1.0, 1.0, True), (1, 0, 0.5, 2.0, False),
    (1, 1, -1.25, 0.0, True), (0, 0, 1.0, 0.0, False)])
def test_gemm_f32_closed_form(transA, transB, alpha, beta, relu):
    r = rng(1)
    M, N, K = 37, 29, 53
    A = r.standard_normal((K, M) if transA else (M, K)).astype(np.float32)
    B = r.standard_normal((N, K) if transB else (K, N)).astype(np.float32)
    bias = r.standard_normal(N).astype(np.float32) if beta != 0.0 else None
    y = oracle.gemm_f32(A, B, bias, alpha, beta, bool(transA), bool(transB), relu)
    a = (A.T if transA else A).astype(np.float64)
    b = (B.T if transB else B).astype(np.float64)
    t = alpha * (a @ b) + (beta * bias.astype(np.float64) if bias is not None else 0.0)
    if relu:
        t = np.maximum(t, 0)
    assert np.max(np.abs(y - t)) <= 1e-5 * np.max(np.abs(t))


def test_gemm_without_bias_and_nonzero_beta_is_an_error():
    A = np.ones((2, 2), np.float32)
    with pytest.raises(RuntimeError):
        oracle.gemm_f32(A, A, None, 1.0, 1.0)


def test_gemm_full_shape_bias_is_taken_as_is():
    r = rng(2)
    A = r.standard_normal((5, 7)).astype(np.float32)
    B = r.standard_normal((7, 3)).astype(np.float32)
    Cfull = r.standard_normal((5, 3)).astype(np.float32)
    y = oracle.gemm_f32(A, B, Cfull)
    assert np.allclose(y, A.astype(np.float64) @ B + Cfull, rtol=1e-5, atol=1e-5)


# ----------------------------------------------------------------------------- fp32 Conv
def brute_conv(x, w, b, ph, pw, sh, sw, dh, dw, groups):
    N, C, H, W = x.shape
    OC, icg, kh, kw = w.shape
    OH = (H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1
    OW = (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1
    y = np.zeros((N, OC, OH, OW), np.float64)
    ocg = OC // groups
    for n in range(N):
        for oc in range(OC):
            g = oc // ocg
            for oh in range(OH):
                for ow in range(OW):
                    s = 0.0
                    for ic in range(icg):
                        for r in range(kh):
                            for q in range(kw):
                                ih, iw = oh * sh - ph + r * dh, ow * sw - pw + q * dw
                                if 0 <= ih < H and 0 <= iw < W:
                                    s += float(x[n, g * icg + ic, ih, iw]) * float(w[oc, ic, r, q])
                    y[n, oc, oh, ow] = s + (float(b[oc]) if b is not None else 0.0)
    return y


@pytest.mark.parametrize("cfg", [
    dict(N=2, C=3, H=7, W=6, OC=4, k=(3, 3), p=(1, 1), s=(1, 1), d=(1, 1), g=1, bias=True),
    dict(N=1, C=4, H=9, W=8, OC=6, k=(3, 2), p=(0, 1), s=(2, 1), d=(1, 1), g=2, bias=False),
    dict(N=2, C=2, H=8, W=8, OC=2, k=(2, 2), p=(1, 1), s=(2, 2), d=(1, 1), g=1, bias=True),
    dict(N=1, C=2, H=10, W=9, OC=3, k=(3, 3), p=(2, 2), s=(1, 1), d=(2, 2), g=1, bias=True),
])
def test_conv2d_f32_against_brute_force_and_torch(cfg):
    r = rng(3)
    x = r.standard_normal((cfg["N"], cfg["C"], cfg["H"], cfg["W"])).astype(np.float32)
    w = r.standard_normal((cfg["OC"], cfg["C"] // cfg["g"]) + cfg["k"]).astype(np.float32)
    b = r.standard_normal(cfg["OC"]).astype(np.float32) if cfg["bias"] else None
    y = oracle.conv2d_f32(x, w, b, cfg["p"], cfg["s"], cfg["d"], cfg["g"])
    t = brute_conv(x, w, b, *cfg["p"], *cfg["s"], *cfg["d"], cfg["g"])
    assert y.shape == t.shape
    assert np.max(np.abs(y - t)) <= 1e-5 * np.max(np.abs(t))
    tt = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(),
                  torch.from_numpy(b).double() if b is not None else None,
                  stride=cfg["s"], padding=cfg["p"], dilation=cfg["d"], groups=cfg["g"]).numpy()
    assert np.max(np.abs(y - tt)) <= 1e-5 * np.max(np.abs(tt))


def test_conv_1x1_is_a_gemm_and_ones_kernel_is_a_box_sum():
    r = rng(4)
    x = r.integers(-5, 6, (2, 8, 5, 5)).astype(np.float32)
    w = r.integers(-3, 4, (6, 8, 1, 1)).astype(np.float32)
    y = oracle.conv2d_f32(x, w)
    t = np.einsum("oc,nchw->nohw", w[:, :, 0, 0], x)
    assert np.array_equal(y, t)
    ones = np.ones((1, 8, 3, 3), np.float32)
    yb = oracle.conv2d_f32(x, ones, pads=(1, 1))
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    tb = sum(xp[:, :, i:i + 5, j:j + 5] for i in range(3) for j in range(3)).sum(1, keepdims=True)
    assert np.array_equal(yb, tb)


def test_im2col_times_weights_equals_direct_conv():
    r = rng(5)
    x = r.integers(-4, 5, (3, 6, 7)).astype(np.float32)
    w = r.integers(-2, 3, (5, 3, 3, 3)).astype(np.float32)
    col = oracle.im2col(x, 3, 3, 1, 1, 1, 1)
    y = (w.reshape(5, -1) @ col).reshape(1, 5, 6, 7)
    assert np.array_equal(y, oracle.conv2d_f32(x[None], w, pads=(1, 1)))


def test_relu_and_maxpool_against_torch():
    r = rng(6)
    x = r.standard_normal((2, 3, 9, 8)).astype(np.float32)
    assert np.array_equal(oracle.relu_f32(x), np.maximum(x, 0))
    for k, s, p in [((2, 2), (2, 2), (0, 0, 0, 0)), ((3, 2), (1, 1), (0, 0, 0, 0)),
                    ((3, 3), (2, 2), (1, 1, 1, 1))]:
        y = oracle.maxpool2d(x, k, s, p)
        t = F.max_pool2d(torch.from_numpy(x), k, s, (p[0], p[1])).numpy()
        assert np.array_equal(y, t)
    q = r.integers(-128, 128, (2, 3, 8, 8)).astype(np.int8)
    yq = oracle.maxpool2d(q, (2, 2), (2, 2))
    tq = q.reshape(2, 3, 4, 2, 4, 2).max(axis=(3, 5))
    assert np.array_equal(yq, tq)


# ----------------------------------------------------------------------------- int8
def exact_requant(acc, scale32, zp, relu):
    """Independent statement: fp32(acc) and the fp32 product are obtained by exact
    arithmetic followed by one correctly rounded conversion; half-even via Fraction."""
    a32 = np.float32(acc)                                  # correctly rounded int->fp32
    prod = np.float32(np.float64(a32) * np.float64(scale32))  # exact in fp64, one rounding
    r = round(Fraction(float(prod)))                       # Python rounds halves to even
    lo = max(zp, -128) if relu else -128
    return int(min(127, max(lo, r + zp)))


def test_requant_rounding_boundaries_exhaustive():
    r = rng(7)
    scales = [np.float32(0.5), np.float32(0.25), np.float32(1.0), np.float32(0.001953125),
              np.float32(1e-3), np.float32(7.3e-3), np.float32(1.2e-4), np.float32(0.0123)]
    for s in scales:
        inv = int(round(1.0 / float(s)))
        accs = set()
        for q in range(-140, 141):                         # around every .5 boundary
            c = int(round((q + 0.5) / float(s)))
            accs.update(range(c - 3, c + 4))
        accs.update([0, 1, -1, inv, -inv, 2 ** 24 + 1, -(2 ** 24) - 1, 2 ** 31 - 1, -(2 ** 31),
                     16777217, 33554435])
        accs.update(int(v) for v in r.integers(-2 ** 31, 2 ** 31, 200))
        for acc in accs:
            acc = max(-(2 ** 31), min(2 ** 31 - 1, acc))
            for zp, relu in [(0, False), (-128, True), (3, True), (-5, False)]:
                assert oracle.requant_one(acc, s, zp, relu) == exact_requant(acc, s, zp, relu), \
                    (acc, s, zp, relu)


def test_rne_examples():
    assert [oracle.requant_one(a, 0.5) for a in (1, 3, 5, -1, -3, -5)] == [0, 2, 2, 0, -2, -2]
    assert oracle.requant_one(10 ** 6, 1.0) == 127 and oracle.requant_one(-10 ** 6, 1.0) == -128
    assert oracle.requant_one(-10, 1.0, zp=-128, relu=True) == -128


@pytest.mark.parametrize("transB", [False, True])
def test_igemm_and_qgemm_against_int64(transB):
    r = rng(8)
    M, N, K = 33, 47, 300
    A = r.integers(-127, 128, (M, K)).astype(np.int8)
    B = r.integers(-127, 128, (N, K) if transB else (K, N)).astype(np.int8)
    acc = oracle.igemm_s8(A, B, transB)
    b = B.T if transB else B
    t = A.astype(np.int64) @ b.astype(np.int64)
    assert np.array_equal(acc, t)
    ti = torch._int_mm(torch.from_numpy(np.ascontiguousarray(np.pad(A, ((0, 31), (0, 4))))),
                       torch.from_numpy(np.ascontiguousarray(np.pad(b, ((0, 4), (0, 1))))))
    assert np.array_equal(ti.numpy()[:M, :N], t)
    scale = r.uniform(2e-5, 2e-4, N).astype(np.float32)
    bias = r.integers(-5000, 5000, N).astype(np.int32)
    y = oracle.qgemm_s8(A, B, scale, bias, transB, zpy=-3, relu=True)
    want = np.array([[exact_requant(int(t[i, j] + bias[j]), scale[j], -3, True)
                      for j in range(N)] for i in range(M)], np.int8)
    assert np.array_equal(y, want)
    yf = oracle.qgemm_s8_f32out(A, B, scale, bias, transB)
    wf = ((t + bias).astype(np.float32) * scale).astype(np.float32)
    assert np.array_equal(yf, wf)


def test_igemm_zero_points():
    r = rng(9)
    A = r.integers(-128, 128, (5, 40)).astype(np.int8)
    B = r.integers(-128, 128, (40, 6)).astype(np.int8)
    acc = oracle.igemm_s8(A, B, False, zpa=-128, zpb=7)
    assert np.array_equal(acc, (A.astype(np.int64) + 128) @ (B.astype(np.int64) - 7))


def test_quantize_dequantize():
    r = rng(10)
    x = r.uniform(0, 1, 1000).astype(np.float32)
    s = np.float32(1 / 255)
    q = oracle.quantize_f32_s8(x, s, -128)
    want = np.clip(np.rint(x / s) - 128, -128, 127).astype(np.int8)
    assert np.array_equal(q, want)
    halves = (np.arange(-6, 7, dtype=np.float32) + np.float32(0.5))
    assert np.array_equal(oracle.quantize_f32_s8(halves, 1.0, 0),
                          np.array([round(Fraction(float(v))) for v in halves], np.int8))
    assert np.array_equal(oracle.dequantize_s8_f32(q, s, -128),
                          ((q.astype(np.int32) + 128).astype(np.float32) * s))


def test_qconv_against_int64_convolution():
    r = rng(11)
    x = r.integers(-128, 128, (2, 6, 7, 6)).astype(np.int8)
    w = r.integers(-127, 128, (8, 3, 3, 3)).astype(np.int8)
    zpx = -128
    acc = oracle.iconv2d_s8(x, w, (1, 1), (1, 1), groups=2, zpx=zpx)
    xs = x.astype(np.float64) - zpx                       # padding then contributes 0
    t = F.conv2d(torch.from_numpy(xs), torch.from_numpy(w.astype(np.float64)), None,
                 stride=1, padding=1, groups=2).numpy()
    assert np.array_equal(acc, t.astype(np.int64))
    scale = r.uniform(1e-4, 1e-3, 8).astype(np.float32)
    bias = r.integers(-3000, 3000, 8).astype(np.int32)
    y = oracle.qconv2d_s8(x, w, scale, bias, (1, 1), (1, 1), 2, zpx, -128, True)
    tt = t.astype(np.int64) + bias[None, :, None, None]
    want = np.empty_like(y)
    for idx in np.ndindex(*y.shape):
        want[idx] = exact_requant(int(tt[idx]), scale[idx[1]], -128, True)
    assert np.array_equal(y, want)


def test_integer_valued_fp32_conv_pins_int8_accumulators():
    """For integer data with |acc| < 2^24 the fp32 Conv path (pinned by the reference's
    fixtures) is exact, so it fixes the int32 accumulators of the int8 path."""
    r = rng(12)
    x = r.integers(-15, 16, (2, 8, 9, 9)).astype(np.int8)
    w = r.integers(-15, 16, (4, 8, 3, 3)).astype(np.int8)
    acc = oracle.iconv2d_s8(x, w, (1, 1), (1, 1))
    yf = oracle.conv2d_f32(x.astype(np.float32), w.astype(np.float32), None, (1, 1))
    assert np.array_equal(acc, yf.astype(np.int32))
    A = r.integers(-15, 16, (16, 1024)).astype(np.int8)
    B = r.integers(-15, 16, (1024, 24)).astype(np.int8)
    assert np.array_equal(oracle.igemm_s8(A, B),
                          oracle.gemm_f32(A.astype(np.float32), B.astype(np.float32),
                                          beta=0.0).astype(np.int32))


# ----------------------------------------------------------------------------- fp8 / bf16
def test_e4m3_table_against_torch_and_closed_form():
    table = oracle.e4m3_table()
    codes = torch.arange(256, dtype=torch.uint8)
    tt = codes.view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(table), np.isnan(tt))
    ok = ~np.isnan(tt)
    assert np.array_equal(table[ok], tt[ok])
    assert table[0x7e] == 448.0 and table[0x08] == 2.0 ** -6 and table[0x01] == 2.0 ** -9


def test_e4m3_encode_against_torch_cast():
    r = rng(13)
    x = np.concatenate([r.standard_normal(4000).astype(np.float32) * 50,
                        r.uniform(-1e-2, 1e-2, 2000).astype(np.float32),
                        oracle.e4m3_table()[~np.isnan(oracle.e4m3_table())],
                        np.array([0.0, -0.0, 448.0, -448.0, 1000.0, -1e9, 464.0, 463.9, 2 ** -10,
                                  2 ** -10 * 1.01, 2 ** -9 * 1.5, 2 ** -9 * 2.5], np.float32)])
    mine = oracle.e4m3_encode(x)
    clamped = torch.from_numpy(np.clip(x, -448, 448))
    theirs = clamped.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    # -0.0 and +0.0 may differ in sign bit after underflow; compare decoded values
    assert np.array_equal(oracle.e4m3_decode(mine), oracle.e4m3_decode(theirs))


def test_bf16_round_to_nearest_even_against_torch():
    r = rng(14)
    x = np.concatenate([r.standard_normal(5000).astype(np.float32) * 100,
                        np.array([1.0, 1.00390625, 1.01171875, -3.0e38, 1e-40, 0.0], np.float32)])
    mine = oracle.bf16_encode(x)
    theirs = torch.from_numpy(x).bfloat16().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(mine, theirs)
    assert np.array_equal(oracle.bf16_decode(mine),
                          torch.from_numpy(x).bfloat16().float().numpy())


@pytest.mark.parametrize("transB", [False, True])
def test_gemm_fp8_against_float64(transB):
    r = rng(15)
    M, N, K = 24, 40, 512
    a = r.standard_normal((M, K)).astype(np.float32)
    b = r.standard_normal((N, K) if transB else (K, N)).astype(np.float32)
    sa, sb = np.float32(np.abs(a).max() / 448), np.float32(np.abs(b).max() / 448)
    A, B = oracle.e4m3_encode(a / sa), oracle.e4m3_encode(b / sb)
    bias = r.standard_normal(N).astype(np.float32)
    yb, yf = oracle.gemm_fp8(A, B, sa, sb, bias, transB)
    da, db = oracle.e4m3_decode(A).astype(np.float64), oracle.e4m3_decode(B).astype(np.float64)
    if transB:
        db = db.T
    truth = (da @ db) * (np.float64(sa) * np.float64(sb)) + bias
    assert np.max(np.abs(yf - truth)) <= 2e-6 * np.max(np.abs(truth)) * np.sqrt(K)
    assert np.array_equal(yb, oracle.bf16_encode(yf))
    yb64, yf64 = oracle.gemm_fp8(A, B, sa, sb, bias, transB, acc64=True)
    assert np.max(np.abs(yf64 - truth)) <= 1e-6 * np.max(np.abs(truth))


EINSUM_CASES = [
    ("ik,kj->ij", [(4, 5), (5, 6)]), ("bik,bjk->bij", [(3, 4, 5), (3, 6, 5)]), ("ik,kj->ji", [(4, 5), (5, 6)]),
    ("abc,abd->ad", [(2, 4, 3), (2, 4, 5)]), ("i,i->", [(9,), (9,)]), ("ii->i", [(6, 6)]), ("ij->ji", [(3, 7)]),
    ("i,j->ij", [(4,), (3,)]), ("ab,bc,cd->ad", [(3, 4), (4, 5), (5, 2)]), ("abcd,abed->abce", [(2, 1, 2, 3), (2, 1, 3, 3)]),
    ("zy,y->z", [(5, 8), (8,)]), ("ijk->", [(2, 3, 4)]),
]


@pytest.mark.parametrize("eq,shapes", EINSUM_CASES)
def test_einsum_against_numpy_float64(eq, shapes):
    """The oracle's loop nest against numpy.einsum on float64 copies (1e-6 relative), and exactly on small
    integers, where the order of the sums cannot matter."""
    r = np.random.default_rng(sum(map(ord, eq)))
    xs = [r.standard_normal(s).astype(np.float32) for s in shapes]
    y = oracle.einsum_f32(eq, xs)
    truth = np.einsum(eq, *[x.astype(np.float64) for x in xs])
    assert y.shape == truth.shape
    assert np.max(np.abs(y - truth)) <= 1e-6 * max(1.0, float(np.max(np.abs(truth))))
    xi = [r.integers(-4, 5, s).astype(np.float32) for s in shapes]
    assert np.array_equal(oracle.einsum_f32(eq, xi), np.einsum(eq, *[x.astype(np.float64) for x in xi]).astype(np.float32))


def test_einsum_sums_in_label_order():
    """Summed labels run sorted by character, the first outermost (a std::map in the reference): with values that
    cancel in one order only, the result tells the order."""
    big = np.float32(2.0 ** 25)
    x = np.array([[big, 1.0], [-big, 1.0]], np.float32)          # labels (a, b): terms in order (0,0) (0,1) (1,0) (1,1)
    # ((big + 1) - big) + 1 = 1 in float32 (big + 1 rounds to big): a outermost, b inner
    assert float(oracle.einsum_f32("ab->", [x])) == 1.0
    # with the labels renamed so that the second axis sorts first, the loop order turns around: (big - big) + 1 + 1 = 2
    assert float(oracle.einsum_f32("ba->", [x])) == 2.0


@pytest.mark.parametrize("cfg", [
    (2, 3, 5, 6, 7, 4, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1),
    (1, 4, 8, 9, 10, 6, (2, 3, 1), (0, 1, 0), (2, 1, 3), (1, 2, 1), 2),
    (2, 6, 4, 4, 12, 6, (1, 1, 5), (0, 0, 2), (1, 1, 1), (1, 1, 2), 6),
])
def test_conv3d_f32_against_torch_and_depth_one_conv2d(cfg):
    import torch
    N, C, D, H, W, OC, k, pads, strides, dil, groups = cfg
    r = np.random.default_rng(700 + C + W)
    x = r.standard_normal((N, C, D, H, W)).astype(np.float32)
    w = r.standard_normal((OC, C // groups) + k).astype(np.float32)
    b = r.standard_normal(OC).astype(np.float32)
    y = oracle.conv3d_f32(x, w, b, pads, strides, dil, groups)
    t = torch.nn.functional.conv3d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), torch.from_numpy(b).double(),
                                   strides, pads, dil, groups).numpy()
    assert y.shape == t.shape
    assert np.max(np.abs(y - t)) <= 1e-5 * np.max(np.abs(t))
    # a depth of one with a depth-one kernel is the 2-D convolution, term by term
    x2, w2 = x[:, :, :1], w[:, :, :1]
    y3 = oracle.conv3d_f32(x2, w2, b, (0,) + tuple(pads[1:]), (1,) + tuple(strides[1:]), (1,) + tuple(dil[1:]), groups, relu=True)
    y2 = oracle.conv2d_f32(x2[:, :, 0], w2[:, :, 0], b, pads[1:], strides[1:], dil[1:], groups, relu=True)
    assert np.array_equal(y3[:, :, 0], y2)


# ----------------------------------------------------------------------------- fp32 BatchNormalization
@pytest.mark.parametrize("shape", [(3, 5, 4, 7), (6, 9), (2, 4, 11)])
@pytest.mark.parametrize("eps", [1e-5, 1e-3])
@pytest.mark.parametrize("relu", [False, True])
def test_batchnorm_f32_against_torch_and_float64(shape, eps, relu):
    """Inference BatchNormalization (the reference holds no fixture for it): torch's batch_norm in
    evaluation mode on CPU and the float64 closed form gamma * (x - mean) / sqrt(var + eps) + beta.
    The operands are drawn apart (mean far from 0, variance near eps in one channel, a negative gamma)
    so that a swapped operand, a missing eps or a ReLU applied before the shift fails."""
    r = rng(70 + len(shape))
    C = shape[1]
    x = (r.standard_normal(shape) * 3 + 1.5).astype(np.float32)
    gamma = r.uniform(0.5, 2.0, C).astype(np.float32)
    gamma[1] = -gamma[1]
    beta = r.standard_normal(C).astype(np.float32)
    mean = (r.standard_normal(C) * 2 + 0.7).astype(np.float32)
    var = r.uniform(0.2, 3.0, C).astype(np.float32)
    var[0] = 2e-4                                             # eps matters here
    y = oracle.batchnorm_f32(x, gamma, beta, mean, var, eps, relu)
    bshape = (1, C) + (1,) * (len(shape) - 2)
    x64 = x.astype(np.float64)
    t = (gamma.astype(np.float64).reshape(bshape) * (x64 - mean.astype(np.float64).reshape(bshape))
         / np.sqrt(var.astype(np.float64).reshape(bshape) + eps) + beta.astype(np.float64).reshape(bshape))
    tt = F.batch_norm(torch.from_numpy(x), torch.from_numpy(mean), torch.from_numpy(var), torch.from_numpy(gamma),
                      torch.from_numpy(beta), training=False, eps=eps).numpy()
    if relu:
        t = np.maximum(t, 0)
        tt = np.maximum(tt, 0)
    assert y.shape == x.shape
    assert np.max(np.abs(y - t)) <= 1e-5 * np.max(np.abs(t))
    assert np.max(np.abs(y - tt)) <= 1e-5 * np.max(np.abs(tt))
    # eps must enter under the root: with eps = 0 channel 0 differs visibly
    t0 = gamma[0] * (x64.take(0, axis=1) - mean[0]) / np.sqrt(np.float64(var[0]))
    got0 = y.take(0, axis=1) - beta[0]
    if not relu:
        assert np.max(np.abs(got0 - t0)) > 1e-3 * np.max(np.abs(t0))


# ----------------------------------------------------------------------------- fp32 transposed convolution
CONVT_GRID = [
    dict(N=2, C=4, H=5, W=6, OC=6, k=(3, 3), s=(2, 2), p=(1, 1, 1, 1), d=(1, 1), g=1, op=(0, 0)),
    dict(N=1, C=6, H=4, W=4, OC=4, k=(2, 3), s=(3, 2), p=(0, 1, 0, 1), d=(2, 1), g=2, op=(1, 1)),
    dict(N=2, C=3, H=7, W=5, OC=5, k=(4, 4), s=(2, 2), p=(1, 1, 1, 1), d=(1, 1), g=1, op=(1, 0)),
    dict(N=3, C=64, H=14, W=14, OC=96, k=(4, 4), s=(2, 2), p=(1, 1, 1, 1), d=(1, 1), g=1, op=(0, 0)),
    dict(N=2, C=32, H=9, W=11, OC=32, k=(3, 3), s=(1, 1), p=(1, 1, 1, 1), d=(1, 1), g=4, op=(0, 0)),
    dict(N=1, C=8, H=6, W=6, OC=8, k=(3, 3), s=(2, 2), p=(2, 2, 2, 2), d=(1, 1), g=1, op=(1, 1)),
    dict(N=1, C=4, H=5, W=5, OC=4, k=(2, 2), s=(1, 1), p=(2, 2, 2, 2), d=(1, 1), g=1, op=(0, 0)),
    dict(N=1, C=2, H=3, W=40, OC=3, k=(1, 9), s=(1, 4), p=(0, 2, 0, 2), d=(1, 1), g=1, op=(0, 3)),
    dict(N=1, C=2, H=2, W=2, OC=2, k=(31, 31), s=(1, 1), p=(0, 0, 0, 0), d=(1, 1), g=1, op=(0, 0)),
    # begin pads that differ from the end pads (torch only knows symmetric ones: see the test)
    dict(N=2, C=4, H=6, W=5, OC=6, k=(3, 4), s=(2, 3), p=(0, 2, 1, 0), d=(1, 1), g=2, op=(1, 2)),
    dict(N=1, C=3, H=5, W=7, OC=2, k=(3, 3), s=(2, 1), p=(2, 0, 0, 1), d=(2, 2), g=1, op=(0, 0)),
]


def _convt_scatter64(x, w, bias, cfg):
    """The definition of ONNX ConvTranspose as a scatter in float64: every input value adds
    x * w[ic, oc, kh, kw] to y[oc, iy*stride + kh*dil - pad_begin, ...]; outputs outside [0, OH) are dropped."""
    N, C, H, W = x.shape
    g = cfg["g"]
    ocg = w.shape[1]
    kh, kw = cfg["k"]
    sh, sw = cfg["s"]
    dh, dw = cfg["d"]
    pt, pl, pb, pr = cfg["p"]
    OH = sh * (H - 1) + dh * (kh - 1) + 1 + cfg["op"][0] - pt - pb
    OW = sw * (W - 1) + dw * (kw - 1) + 1 + cfg["op"][1] - pl - pr
    y = np.zeros((N, ocg * g, OH, OW), np.float64)
    cg = C // g
    for ic in range(C):
        grp = ic // cg
        for a in range(kh):
            for b in range(kw):
                for iy in range(H):
                    oy = iy * sh + a * dh - pt
                    if not 0 <= oy < OH:
                        continue
                    for ix in range(W):
                        ox = ix * sw + b * dw - pl
                        if not 0 <= ox < OW:
                            continue
                        y[:, grp * ocg:(grp + 1) * ocg, oy, ox] += np.outer(x[:, ic, iy, ix].astype(np.float64),
                                                                            w[ic, :, a, b].astype(np.float64))
    if bias is not None:
        y += bias.astype(np.float64).reshape(1, -1, 1, 1)
    return y


@pytest.mark.parametrize("cfg", CONVT_GRID)
def test_conv_transpose2d_f32_against_torch_and_scatter(cfg):
    """or_conv_transpose2d_f32 over the grid of strides, dilations, groups, pads and output paddings that
    the GPU test compares the kernel with. Two independent answers: torch's conv_transpose2d on CPU in
    float64 (symmetric pads only: for begin != end pads torch is run without padding and the result cropped
    by the begin pads on the top/left and the end pads on the bottom/right, which is ONNX's definition) and
    the scatter definition written out in float64. The reference's fixtures only cover stride 1 without
    pads, groups, dilation or output padding."""
    r = rng(40 + cfg["C"] + cfg["H"])
    x = r.standard_normal((cfg["N"], cfg["C"], cfg["H"], cfg["W"])).astype(np.float32)
    w = (r.standard_normal((cfg["C"], cfg["OC"] // cfg["g"]) + cfg["k"]) * 0.2).astype(np.float32)
    b = r.standard_normal(cfg["OC"]).astype(np.float32)
    pt, pl, pb, pr = cfg["p"]
    for bias, relu in ((b, False), (None, True)):
        y = oracle.conv_transpose2d_f32(x, w, bias, cfg["p"], cfg["s"], cfg["d"], cfg["g"], cfg["op"], relu)
        full = F.conv_transpose2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(),
                                  None if bias is None else torch.from_numpy(bias).double(),
                                  stride=cfg["s"], padding=0, output_padding=0, groups=cfg["g"],
                                  dilation=cfg["d"]).numpy()
        # output padding appends rows/columns that receive no contribution (bias only)
        oph, opw = cfg["op"]
        full = np.pad(full, ((0, 0), (0, 0), (0, oph), (0, opw)))
        if bias is not None and (oph or opw):
            bb = bias.astype(np.float64).reshape(1, -1, 1, 1)
            if oph:
                full[:, :, -oph:, :] = bb
            if opw:
                full[:, :, :, -opw:] = bb
        t = full[:, :, pt:full.shape[2] - pb, pl:full.shape[3] - pr]
        s = _convt_scatter64(x, w, bias, cfg)
        if relu:
            t = np.maximum(t, 0)
            s = np.maximum(s, 0)
        assert y.shape == t.shape == s.shape
        scale = max(np.max(np.abs(t)), 1e-30)
        assert np.max(np.abs(s - t)) <= 1e-12 * scale            # the two truths agree
        assert np.max(np.abs(y - t)) <= 1e-5 * scale
        if pt == pb and pl == pr and oph < max(cfg["s"][0], cfg["d"][0]) and opw < max(cfg["s"][1], cfg["d"][1]):
            tsym = F.conv_transpose2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(),
                                      None if bias is None else torch.from_numpy(bias).double(),
                                      stride=cfg["s"], padding=(pt, pl), output_padding=cfg["op"],
                                      groups=cfg["g"], dilation=cfg["d"]).numpy()
            if relu:
                tsym = np.maximum(tsym, 0)
            assert np.max(np.abs(y - tsym)) <= 1e-5 * scale


# ----------------------------------------------------------------------------- the CPU baseline program
def _cpu_emitted(args, env=None):
    import json
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(oracle.__file__)), "cpu_emitted_bench")
    if not os.path.exists(exe):
        subprocess.run(["make", "-C", os.path.dirname(exe), "cpu_emitted_bench"], check=True, stdout=subprocess.DEVNULL)
    e = dict(os.environ)
    e.update(env or {})
    res = subprocess.run([exe] + args, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=e, timeout=300)
    assert res.returncode == 0, res.stderr
    return json.loads(res.stdout.strip().splitlines()[-1])


def _scipy_blas():
    import glob
    import importlib.util
    import os
    spec = importlib.util.find_spec("scipy")
    if spec is None:
        return None
    hits = glob.glob(os.path.join(os.path.dirname(os.path.dirname(spec.origin)), "scipy.libs", "libscipy_openblas-*.so"))
    return hits[0] if hits else None


def test_cpu_baseline_program_computes_what_the_oracle_computes(tmp_path):
    """oracle/cpu_emitted_bench.c (the reference's emitted call sequence for the fp32 MLP and convolution layer,
    timed by the benchmark as the CPU baseline) against the oracle's Gemm and Conv on the inputs it dumps, with
    its bundled loops and, where the image has one, with a BLAS bound at run time."""
    blas = _scipy_blas()
    variants = [[]] + ([["--blas", blas, "--prefix", "scipy_"]] if blas else [])
    for extra in variants:
        f = str(tmp_path / "mlp.bin")
        out = _cpu_emitted(["--workload", "mlp", "--calls", "2", "--dump", f] + extra, {"OMP_NUM_THREADS": "2"})
        assert out["selfcheck"] <= 1e-4
        raw = np.fromfile(f, np.float32)
        sizes = [256 * 64, 64 * 128, 128 * 64, 64 * 8, 256 * 8]
        x, w0, w1, w2, y = np.split(raw, np.cumsum(sizes)[:-1])
        h = oracle.gemm_f32(x.reshape(256, 64), w0.reshape(64, 128), np.zeros(128, np.float32), relu=True)
        h = oracle.gemm_f32(h, w1.reshape(128, 64), np.zeros(64, np.float32), relu=True)
        ref = oracle.gemm_f32(h, w2.reshape(64, 8), np.zeros(8, np.float32))
        assert np.max(np.abs(y.reshape(256, 8) - ref)) <= 1e-5 * np.max(np.abs(ref))
        # Glorot-uniform weights stay inside their limit, the input is roughly N(0,1)
        assert np.max(np.abs(w0)) <= np.sqrt(6.0 / 192) and abs(float(x.std()) - 1.0) < 0.05
        f = str(tmp_path / "conv.bin")
        out = _cpu_emitted(["--workload", "conv", "--images", "2", "--calls", "1", "--dump", f] + extra,
                           {"OMP_NUM_THREADS": "2"})
        raw = np.fromfile(f, np.float32)
        sizes = [2 * 64 * 56 * 56, 128 * 64 * 9, 128, 2 * 128 * 56 * 56]
        x, w, b, y = np.split(raw, np.cumsum(sizes)[:-1])
        ref = oracle.conv2d_f32(x.reshape(2, 64, 56, 56), w.reshape(128, 64, 3, 3), b, (1, 1), relu=True)
        assert np.max(np.abs(y.reshape(ref.shape) - ref)) <= 1e-5 * np.max(np.abs(ref))
        # the large Gemm: a few rows of the 4096 x 4096 x 4096 product with its bias row and ReLU
        f = str(tmp_path / "gemm.bin")
        rows = 3
        out = _cpu_emitted(["--workload", "gemm", "--images", str(rows), "--calls", "1", "--dump", f] + extra, {"OMP_NUM_THREADS": "2"})
        raw = np.fromfile(f, np.float32)
        sizes = [rows * 4096, 4096 * 4096, 4096, rows * 4096]
        assert raw.size == sum(sizes)
        x, w, b, y = np.split(raw, np.cumsum(sizes)[:-1])
        ref = oracle.gemm_f32(x.reshape(rows, 4096), w.reshape(4096, 4096), b, relu=True)
        assert np.max(np.abs(y.reshape(ref.shape) - ref)) <= 1e-5 * np.max(np.abs(ref))


def test_cpu_baseline_cnn_computes_what_the_oracle_computes(tmp_path):
    """The 'cnn' workload of oracle/cpu_emitted_bench.c (the reference's emitted fp32 sequence for the classifier of
    the batch-4096 configuration: Conv + Relu, the MaxPool loop, Gemm) against the oracle's convolution, pooling and
    Gemm on the tensors it dumps, with the bundled loops and with a BLAS bound at run time."""
    blas = _scipy_blas()
    variants = [[]] + ([["--blas", blas, "--prefix", "scipy_"]] if blas else [])
    n = 3
    for extra in variants:
        f = str(tmp_path / "cnn.bin")
        out = _cpu_emitted(["--workload", "cnn", "--images", str(n), "--calls", "1", "--dump", f] + extra, {"OMP_NUM_THREADS": "2"})
        assert out["images"] == n
        raw = np.fromfile(f, np.float32)
        sizes = [n * 1600, 32 * 9, 32, 64 * 32 * 9, 64, 128 * 64 * 9, 128, 12800 * 256, 256, 256 * 5, 5, n * 5]
        assert raw.size == sum(sizes)
        x, w1, b1, w2, b2, w3, b3, f1, c1, f2, c2, y = np.split(raw, np.cumsum(sizes)[:-1])
        h = oracle.conv2d_f32(x.reshape(n, 1, 40, 40), w1.reshape(32, 1, 3, 3), b1, (1, 1), relu=True)
        h = oracle.maxpool2d(h, (2, 2), (2, 2))
        h = oracle.conv2d_f32(h, w2.reshape(64, 32, 3, 3), b2, (1, 1), relu=True)
        h = oracle.maxpool2d(h, (2, 2), (2, 2))
        h = oracle.conv2d_f32(h, w3.reshape(128, 64, 3, 3), b3, (1, 1), relu=True)
        g = oracle.gemm_f32(h.reshape(n, 12800), f1.reshape(12800, 256), c1, relu=True)
        ref = oracle.gemm_f32(g, f2.reshape(256, 5), c2)
        assert np.max(np.abs(y.reshape(n, 5) - ref)) <= 1e-5 * np.max(np.abs(ref))


# ----------------------------------------------------------------------------- fp32 average pooling
@pytest.mark.parametrize("cfg", [
    dict(shape=(2, 3, 9, 8), k=(3, 2), s=(2, 1), p=(0, 0, 0, 0)),
    dict(shape=(1, 4, 7, 7), k=(3, 3), s=(1, 1), p=(1, 1, 1, 1)),
    dict(shape=(2, 2, 10, 11), k=(2, 4), s=(2, 3), p=(1, 2, 1, 2)),
    dict(shape=(3, 5, 6, 6), k=(6, 6), s=(1, 1), p=(0, 0, 0, 0)),      # the global average
])
def test_avgpool2d_against_torch_and_float64(cfg):
    """or_avgpool2d_f32 against torch's avg_pool2d on CPU with count_include_pad off and on (symmetric pads, which
    is what torch takes) and against a float64 mean of the cells inside the image."""
    r = rng(300 + cfg["shape"][2])
    x = r.standard_normal(cfg["shape"]).astype(np.float32)
    pt, pl, pb, pr = cfg["p"]
    for include in (False, True):
        y = oracle.avgpool2d(x, cfg["k"], cfg["s"], cfg["p"], include)
        t = F.avg_pool2d(torch.from_numpy(x).double(), cfg["k"], cfg["s"], (pt, pl), ceil_mode=False,
                         count_include_pad=include).numpy()
        assert y.shape == t.shape
        assert np.max(np.abs(y - t)) <= 1e-6 * max(np.max(np.abs(t)), 1.0)
    # brute force in float64 on one plane: mean over the cells inside the image
    y = oracle.avgpool2d(x, cfg["k"], cfg["s"], cfg["p"], False)
    H, W = cfg["shape"][2:]
    for oh in range(y.shape[2]):
        for ow in range(y.shape[3]):
            r0, c0 = oh * cfg["s"][0] - pt, ow * cfg["s"][1] - pl
            win = x[0, 0, max(r0, 0):min(r0 + cfg["k"][0], H), max(c0, 0):min(c0 + cfg["k"][1], W)].astype(np.float64)
            assert abs(y[0, 0, oh, ow] - win.mean()) <= 1e-6 * max(1.0, abs(win.mean()))


@pytest.mark.parametrize("cfg", [
    dict(shape=(2, 3, 6, 7, 8), k=(2, 3, 2), s=(2, 1, 2), p=(0, 0, 0, 0, 0, 0)),
    dict(shape=(1, 2, 5, 5, 5), k=(3, 3, 3), s=(1, 1, 1), p=(1, 1, 1, 1, 1, 1)),
    dict(shape=(2, 2, 7, 6, 9), k=(2, 2, 4), s=(1, 2, 3), p=(1, 0, 2, 1, 0, 2)),
    dict(shape=(1, 3, 6, 5, 7), k=(3, 2, 2), s=(2, 2, 1), p=(2, 0, 1, 0, 1, 0)),      # begin pads differ from end pads
])
def test_pool3d_against_torch_and_float64(cfg):
    """or_pool3d_f32: the maximum against torch's max_pool3d on the tensor padded with -inf by the six ONNX pads; the
    average with count_include_pad against avg_pool3d on the tensor padded with zeros, without it against avg_pool3d
    where the pads are symmetric (what torch takes) and against a float64 mean of the cells inside the volume."""
    r = rng(700 + cfg["shape"][2] + cfg["k"][2])
    x = r.standard_normal(cfg["shape"]).astype(np.float32)
    p = cfg["p"]
    tpad = (p[2], p[5], p[1], p[4], p[0], p[3])      # torch pads the last axis first
    xt = torch.from_numpy(x)
    ym = oracle.pool3d(x, cfg["k"], cfg["s"], p)
    tm = F.max_pool3d(F.pad(xt, tpad, value=float("-inf")), cfg["k"], cfg["s"]).numpy()
    assert ym.shape == tm.shape and np.array_equal(ym, tm)
    ya = oracle.pool3d(x, cfg["k"], cfg["s"], p, average=True, count_include_pad=True)
    ta = F.avg_pool3d(F.pad(xt.double(), tpad), cfg["k"], cfg["s"]).numpy()
    assert ya.shape == ta.shape and np.max(np.abs(ya - ta)) <= 1e-6 * max(np.max(np.abs(ta)), 1.0)
    yb = oracle.pool3d(x, cfg["k"], cfg["s"], p, average=True, count_include_pad=False)
    if p[:3] == p[3:]:
        tb = F.avg_pool3d(xt.double(), cfg["k"], cfg["s"], p[:3], count_include_pad=False).numpy()
        assert np.max(np.abs(yb - tb)) <= 1e-6 * max(np.max(np.abs(tb)), 1.0)
    D = cfg["shape"][2:]
    for idx in np.ndindex(*yb.shape[2:]):
        lo = [idx[i] * cfg["s"][i] - p[i] for i in range(3)]
        win = x[0, 0, max(lo[0], 0):min(lo[0] + cfg["k"][0], D[0]), max(lo[1], 0):min(lo[1] + cfg["k"][1], D[1]),
                max(lo[2], 0):min(lo[2] + cfg["k"][2], D[2])].astype(np.float64)
        assert abs(yb[(0, 0) + idx] - win.mean()) <= 1e-6 * max(1.0, abs(win.mean()))
