"""Seeded sweeps over random geometries: the HIP entry points against the oracle on shapes nobody picked by hand
(odd extents, unequal begin / end pads, strides, kernels up to 5x5, bands that cross image borders, ragged GEMM
tiles, K tails). Every output buffer sits between sentinel bands (sofie_amd.ops.Context), so a store past the edge
of a ragged tile fails the case that made it. Sizes are small enough for the C oracle to finish in seconds."""
import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from sofie_amd import ops as o
    return o


def _conv_geometry(r, max_hw, kmax=5):
    kh, kw = int(r.integers(1, kmax + 1)), int(r.integers(1, kmax + 1))
    sh, sw = int(r.integers(1, 4)), int(r.integers(1, 4))
    pads = tuple(int(v) for v in (r.integers(0, kh), r.integers(0, kw), r.integers(0, kh), r.integers(0, kw)))
    H = int(r.integers(max(1, kh - pads[0] - pads[2]), max_hw + 1))
    W = int(r.integers(max(1, kw - pads[1] - pads[3]), max_hw + 1))
    return (kh, kw), (sh, sw), pads, H, W


def _out_hw(H, W, k, s, p):
    return (H + p[0] + p[2] - k[0]) // s[0] + 1, (W + p[1] + p[3] - k[1]) // s[1] + 1


@pytest.mark.parametrize("seed", range(24))
def test_qconv2d_s8_matrix_core_shapes(ops, seed):
    """Channels-last operands with C % 32 == 0 and OC % 64 == 0: the matrix-core kernel (3x3 on 32 / 64 channels takes
    its unrolled form), or whatever the library falls back to when a band does not fit."""
    from sofie_amd import lib as L
    r = np.random.default_rng(9000 + seed)
    C = int(r.choice([32, 64, 96]))
    OC = int(r.choice([64, 128, 192]))
    if seed % 3 == 0:
        k, s, p = (3, 3), (1, 1), tuple(int(v) for v in r.integers(0, 3, 4))
        H, W = int(r.integers(3, 24)), int(r.integers(3, 24))
    else:
        k, s, p, H, W = _conv_geometry(r, 20)
    OH, OW = _out_hw(H, W, k, s, p)
    if OH < 1 or OW < 1:
        pytest.skip("empty output")
    N = int(r.integers(1, 9))
    x = r.integers(-128, 128, (N, H, W, C)).astype(np.int8)
    w = r.integers(-127, 128, (OC, C) + k).astype(np.int8)
    Kd = C * k[0] * k[1]
    scale = (r.uniform(20, 60, OC) / (73.3 * 73.3 * np.sqrt(Kd))).astype(np.float32)
    if seed % 5 == 0:
        scale[::7] *= -1.0
    bias = r.integers(-3000, 3000, OC).astype(np.int32)
    zpx, zpy, relu = int(r.choice([-128, 0, 5])), int(r.choice([-128, 3])), bool(r.integers(0, 2))
    ref = oracle.qconv2d_s8(x.transpose(0, 3, 1, 2), w, scale, bias, p, s, 1, zpx, zpy, relu)
    wh = np.ascontiguousarray(w.transpose(0, 2, 3, 1))
    y = ops.qconv2d_s8(x, wh, scale, bias, p, s, 1, zpx, zpy, relu, x_layout=L.LAYOUT_NHWC, y_layout=L.LAYOUT_NHWC,
                       w_layout=L.LAYOUT_NHWC)
    assert np.array_equal(y.transpose(0, 3, 1, 2), ref), (C, OC, k, s, p, H, W, N)
    if OH >= 2 and OW >= 2:
        pooled = oracle.maxpool2d(ref, (2, 2), (2, 2))
        yp = ops.qconv2d_pool_s8(x, wh, scale, bias, p, s, 1, zpx, zpy, relu, x_layout=L.LAYOUT_NHWC,
                                 y_layout=L.LAYOUT_NHWC, w_layout=L.LAYOUT_NHWC)
        assert np.array_equal(yp.transpose(0, 3, 1, 2), pooled), (C, OC, k, s, p, H, W, N, "pooled")


@pytest.mark.parametrize("seed", range(6))
def test_qconv2d_s8_many_small_images(ops, seed):
    """3x3 stride-1 layers on thousands of small images: every workgroup of the kernel that keeps a sliding window of
    input rows in LDS walks through several tiles and many image borders; with and without the fused pooling."""
    from sofie_amd import lib as L
    r = np.random.default_rng(9500 + seed)
    C, OC = (32, 128) if seed % 2 == 0 else (64, 128)
    H, W = int(r.integers(5, 10)), int(r.integers(5, 10))
    p = tuple(int(v) for v in r.integers(0, 3, 4))
    OH, OW = _out_hw(H, W, (3, 3), (1, 1), p)
    N = int(r.integers(70000, 110000)) // (OH * OW)        # 2 - 3 tiles of 256 pixels per workgroup
    x = r.integers(-128, 128, (N, H, W, C)).astype(np.int8)
    w = r.integers(-127, 128, (OC, C, 3, 3)).astype(np.int8)
    scale = (r.uniform(20, 60, OC) / (73.3 * 73.3 * np.sqrt(9.0 * C))).astype(np.float32)
    if seed % 3 == 0:
        scale[::7] *= -1.0
    bias = r.integers(-3000, 3000, OC).astype(np.int32)
    zpx, zpy, relu = int(r.choice([-128, 0, 5])), int(r.choice([-128, 3])), bool(r.integers(0, 2))
    ref = oracle.qconv2d_s8(x.transpose(0, 3, 1, 2), w, scale, bias, p, (1, 1), 1, zpx, zpy, relu)
    wh = np.ascontiguousarray(w.transpose(0, 2, 3, 1))
    y = ops.qconv2d_s8(x, wh, scale, bias, p, (1, 1), 1, zpx, zpy, relu, x_layout=L.LAYOUT_NHWC, y_layout=L.LAYOUT_NHWC,
                       w_layout=L.LAYOUT_NHWC)
    assert np.array_equal(y.transpose(0, 3, 1, 2), ref), (C, OC, p, H, W, N)
    pooled = oracle.maxpool2d(ref, (2, 2), (2, 2))
    yp = ops.qconv2d_pool_s8(x, wh, scale, bias, p, (1, 1), 1, zpx, zpy, relu, x_layout=L.LAYOUT_NHWC,
                             y_layout=L.LAYOUT_NHWC, w_layout=L.LAYOUT_NHWC)
    assert np.array_equal(yp.transpose(0, 3, 1, 2), pooled), (C, OC, p, H, W, N, "pooled")


@pytest.mark.parametrize("seed", range(16))
def test_qconv2d_s8_any_shape(ops, seed):
    """NCHW operands, any channel count and group count: the one-thread-per-output kernel and, for one input channel
    with a 3x3 kernel and pads of one, the first-layer kernel (with and without the fused quantisation)."""
    r = np.random.default_rng(9100 + seed)
    first = seed % 4 == 0
    if first:
        g, C, OC = 1, 1, int(r.choice([16, 32, 48]))
        k, s, p = (3, 3), (1, 1), (1, 1, 1, 1)
        H, W = int(r.integers(4, 30)), int(r.integers(4, 30))
    else:
        g = int(r.choice([1, 2, 3]))
        C, OC = g * int(r.integers(1, 6)), g * int(r.integers(1, 9))
        k, s, p, H, W = _conv_geometry(r, 14)
    OH, OW = _out_hw(H, W, k, s, p)
    if OH < 1 or OW < 1:
        pytest.skip("empty output")
    N = int(r.integers(1, 6))
    x = r.integers(-128, 128, (N, C, H, W)).astype(np.int8)
    w = r.integers(-127, 128, (OC, C // g) + k).astype(np.int8)
    Kd = C // g * k[0] * k[1]
    scale = (r.uniform(20, 60, OC) / (73.3 * 73.3 * np.sqrt(Kd))).astype(np.float32)
    bias = r.integers(-500, 500, OC).astype(np.int32)
    zpx, zpy, relu = int(r.choice([-128, 0, -7])), int(r.choice([-128, 0, 9])), bool(r.integers(0, 2))
    ref = oracle.qconv2d_s8(x, w, scale, bias, p, s, g, zpx, zpy, relu)
    assert np.array_equal(ops.qconv2d_s8(x, w, scale, bias, p, s, g, zpx, zpy, relu), ref), (C, OC, g, k, s, p, H, W, N)
    if first:
        xs = np.float32(1.0 / 255.0)
        xf = r.uniform(0.0, 1.0, (N, 1, H, W)).astype(np.float32)
        xq = oracle.quantize_f32_s8(xf, xs, -128)
        ref_q = oracle.qconv2d_s8(xq, w, scale, bias, p, s, 1, -128, zpy, relu)
        got = ops.quantize_qconv2d_s8(xf, xs, -128, w, scale, bias, p, s, 1, zpy, relu)
        assert np.array_equal(got, ref_q)
        if OH >= 2 and OW >= 2:
            got = ops.quantize_qconv2d_s8(xf, xs, -128, w, scale, bias, p, s, 1, zpy, relu, pool=(2, 2))
            assert np.array_equal(got, oracle.maxpool2d(ref_q, (2, 2), (2, 2)))


@pytest.mark.parametrize("seed", range(24))
def test_qgemm_s8_random_shapes(ops, seed):
    r = np.random.default_rng(9200 + seed)
    M, N = int(r.integers(1, 700)), int(r.integers(1, 700))
    K = int(r.integers(1, 1200)) if seed % 2 else 16 * int(r.integers(1, 80))
    if seed % 6 == 0:
        N = int(r.integers(1, 17))                    # the dot-product kernel
    if seed % 8 == 1:
        M, N, K = 128 * int(r.integers(1, 4)), 128 * int(r.integers(1, 3)), 8192 + 16 * int(r.integers(0, 40))   # K slices
    transB = bool(r.integers(0, 2))
    A = r.integers(-128, 128, (M, K)).astype(np.int8)
    B = r.integers(-127, 128, (N, K) if transB else (K, N)).astype(np.int8)
    scale = (r.uniform(20, 60, N) / (73.3 * 73.3 * np.sqrt(K))).astype(np.float32)
    bias = r.integers(-2000, 2000, N).astype(np.int32) if seed % 3 else None
    zpa, zpy, relu = int(r.choice([0, -128, 11])), int(r.choice([0, -128, -3])), bool(r.integers(0, 2))
    ref = oracle.qgemm_s8(A, B, scale, bias, transB, zpa, zpy, relu)
    got = ops.qgemm_s8(A, B, scale, bias, transB, zpa, zpy, relu)
    assert np.array_equal(got, ref), (M, N, K, transB, zpa, zpy, relu)
    assert np.array_equal(ops.igemm_s8(A, B, transB), oracle.igemm_s8(A, B, transB))


@pytest.mark.parametrize("seed", range(16))
def test_conv2d_f32_random_shapes(ops, seed):
    r = np.random.default_rng(9300 + seed)
    g = int(r.choice([1, 1, 2, 4]))
    C, OC = g * int(r.integers(1, 9)), g * int(r.integers(1, 12))
    k, s, p, H, W = _conv_geometry(r, 18, kmax=4)
    d = (int(r.integers(1, 3)), int(r.integers(1, 3)))
    ke = ((k[0] - 1) * d[0] + 1, (k[1] - 1) * d[1] + 1)
    H, W = max(H, ke[0]), max(W, ke[1])
    N = int(r.integers(1, 5))
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = (r.standard_normal((OC, C // g) + k) / np.sqrt(C // g * k[0] * k[1])).astype(np.float32)
    b = r.standard_normal(OC).astype(np.float32) if seed % 2 else None
    relu = bool(r.integers(0, 2))
    ref = oracle.conv2d_f32(x, w, b, p, s, d, g, relu)
    got = ops.conv2d_f32(x, w, b, p, s, d, g, relu)
    assert got.shape == ref.shape
    assert np.max(np.abs(got - ref)) <= 1e-5 * max(1.0, float(np.max(np.abs(ref)))), (C, OC, g, k, s, p, d, H, W, N)


@pytest.mark.parametrize("seed", range(12))
def test_pooling_random_shapes(ops, seed):
    r = np.random.default_rng(9400 + seed)
    k, s, p, H, W = _conv_geometry(r, 17, kmax=4)
    p = tuple(min(v, (k[i % 2] - 1) // 2) for i, v in enumerate(p))      # ONNX: a pad is smaller than the kernel
    H, W = max(H, k[0]), max(W, k[1])
    x = r.standard_normal((int(r.integers(1, 4)), int(r.integers(1, 7)), H, W)).astype(np.float32)
    assert np.array_equal(ops.maxpool2d(x, k, s, p), oracle.maxpool2d(x, k, s, p))
    for cip in (False, True):
        ref = oracle.avgpool2d(x, k, s, p, cip)
        got = ops.avgpool2d(x, k, s, p, cip)
        assert np.max(np.abs(got - ref)) <= 1e-6 * max(1.0, float(np.max(np.abs(ref))))


@pytest.mark.parametrize("seed", range(16))
def test_gemm_f32_random_shapes(ops, seed):
    r = np.random.default_rng(9500 + seed)
    M, N, K = int(r.integers(1, 400)), int(r.integers(1, 400)), int(r.integers(1, 500))
    tA, tB = bool(r.integers(0, 2)), bool(r.integers(0, 2))
    A = r.standard_normal((K, M) if tA else (M, K)).astype(np.float32)
    B = r.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
    bias = [None, r.standard_normal(N).astype(np.float32), r.standard_normal((M, N)).astype(np.float32)][seed % 3]
    alpha, beta, relu = float(r.choice([1.0, 0.5, -2.0])), float(r.choice([1.0, 0.25])), bool(r.integers(0, 2))
    if bias is None:
        beta = 0.0            # the reference refuses a non-zero beta without a bias tensor
    ref = oracle.gemm_f32(A, B, bias, alpha, beta, tA, tB, relu)
    got = ops.gemm_f32(A, B, bias, alpha, beta, tA, tB, relu)
    assert np.max(np.abs(got - ref)) <= 1e-5 * max(1.0, float(np.max(np.abs(ref)))), (M, N, K, tA, tB)


def _kernels_of(ops, call):
    """Names of the kernels `call` launches on the default context (sofie_hip_trace_begin / _end)."""
    import ctypes as C
    ctx = ops.default_context()
    buf = C.create_string_buffer(4096)
    n = C.c_int(-1)
    assert ctx.lib.sofie_hip_trace_begin(ctx.h) == 0
    try:
        out = call()
    finally:
        assert ctx.lib.sofie_hip_trace_end(ctx.h, buf, 4096, C.byref(n)) == 0
    return out, [l.split()[0] for l in buf.value.decode().splitlines()]


def test_gemm_f32_lds_dma_random_shapes(ops):
    """Random products of the shapes the LDS-DMA Gemm kernels take (K in whole stages of 32, rows of whole 16-byte
    chunks, at least 32 tiles of 64 x 64): ragged last tiles in M and N, both layouts of B, row bias or none, alpha,
    beta, ReLU; 1e-5 relative against the oracle. The trace names the kernel, and both tile sizes occur."""
    seen = {}
    for seed in range(14):
        r = np.random.default_rng(9900 + seed)
        big = seed % 3 == 2                       # 256 tiles of 128 x 128 or more: the 128 x 128-tile form
        M = int(r.integers(2049, 2400)) if big else int(r.integers(330, 1200))
        N = int(r.integers(2049, 2300)) if big else int(r.integers(330, 1200))
        K = 32 * int(r.integers(1, 5 if big else 12))
        tB = bool(r.integers(0, 2))
        if not tB:
            N -= N % 4
        A = r.standard_normal((M, K)).astype(np.float32)
        B = r.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
        bias = r.standard_normal(N).astype(np.float32) if seed % 2 else None
        alpha, relu = float(r.choice([1.0, 0.5, -2.0])), bool(r.integers(0, 2))
        beta = float(r.choice([1.0, 0.25])) if bias is not None else 0.0
        got, names = _kernels_of(ops, lambda: ops.gemm_f32(A, B, bias, alpha, beta, False, tB, relu))
        assert names in (["k_gemm_f32_dma"], ["k_gemm_f32_dma64"]), (names, M, N, K, tB)
        seen[names[0]] = seen.get(names[0], 0) + 1
        ref = oracle.gemm_f32(A, B, bias, alpha, beta, False, tB, relu)
        assert np.max(np.abs(got - ref)) <= 1e-5 * max(1.0, float(np.max(np.abs(ref)))), (M, N, K, tB)
    assert seen.get("k_gemm_f32_dma", 0) >= 3 and seen.get("k_gemm_f32_dma64", 0) >= 3, seen


def test_gemm_f32_few_rows_random_shapes(ops):
    """Random layers on a small batch (1 to 64 rows of A, K a multiple of 4, B of at least 64 K elements): the sliced pass
    over B (k_gemm_f32_skinny) against the oracle, 1e-5 relative; both layouts of B, every row-tile count, with and
    without the second pass over the slices."""
    seen = {}
    for seed in range(24):
        r = np.random.default_rng(9970 + seed)
        M = int(r.choice([1, 2, 7, 16, 17, 31, 32, 33, 50, 64]))
        tB = bool(r.integers(0, 2))
        N = int(r.integers(64, 2500))
        if not tB:
            N -= N % 4
        K = 4 * int(r.integers(16, 700))
        if N * K < 65536:
            K = 4 * (65536 // (4 * N) + 1)
        A = r.standard_normal((M, K)).astype(np.float32)
        B = r.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
        bias = r.standard_normal(N).astype(np.float32) if seed % 2 else None
        alpha, relu = float(r.choice([1.0, 0.5, -2.0])), bool(r.integers(0, 2))
        beta = float(r.choice([1.0, 0.25])) if bias is not None else 0.0
        got, names = _kernels_of(ops, lambda: ops.gemm_f32(A, B, bias, alpha, beta, False, tB, relu))
        assert names[0] == "k_gemm_f32_skinny" and len(names) <= 2, (names, M, N, K, tB)
        seen[len(names)] = seen.get(len(names), 0) + 1
        ref = oracle.gemm_f32(A, B, bias, alpha, beta, False, tB, relu)
        assert np.max(np.abs(got - ref)) <= 1e-5 * max(1.0, float(np.max(np.abs(ref)))), (M, N, K, tB)
    assert seen.get(1, 0) >= 1 and seen.get(2, 0) >= 3, seen


def test_conv2d_f32_lds_dma_random_shapes(ops):
    """Random layers with channel counts the LDS-DMA convolution kernel takes (even channel blocks with at least 18
    taps): kernels up to 4 x 4, strides, dilations, unequal pads, groups, ragged channel and pixel tiles; 1e-5 relative
    against the oracle. Both of its matrix loops (with and without the table of patch offsets) must have run."""
    seen = {}
    for seed in range(24):
        r = np.random.default_rng(9950 + seed)
        g = int(r.choice([1, 1, 2]))
        icg = int(r.choice([4, 6, 8, 10, 12, 16, 24, 32]))
        C, OC = g * icg, g * int(r.integers(1, 90))
        k, s, p, H, W = _conv_geometry(r, 26, kmax=4)
        d = (int(r.integers(1, 3)), int(r.integers(1, 3)))
        ke = ((k[0] - 1) * d[0] + 1, (k[1] - 1) * d[1] + 1)
        H, W = max(H, ke[0]), max(W, ke[1])
        N = int(r.integers(1, 4))
        x = r.standard_normal((N, C, H, W)).astype(np.float32)
        w = (r.standard_normal((OC, icg) + k) / np.sqrt(icg * k[0] * k[1])).astype(np.float32)
        b = r.standard_normal(OC).astype(np.float32) if seed % 2 else None
        relu = bool(r.integers(0, 2))
        got, names = _kernels_of(ops, lambda: ops.conv2d_f32(x, w, b, p, s, d, g, relu))
        seen[names[-1]] = seen.get(names[-1], 0) + 1
        ref = oracle.conv2d_f32(x, w, b, p, s, d, g, relu)
        assert got.shape == ref.shape
        assert np.max(np.abs(got - ref)) <= 1e-5 * max(1.0, float(np.max(np.abs(ref)))), (names, C, OC, g, k, s, p, d, H, W, N)
    assert seen.get("k_conv2d_f32_dma", 0) >= 3 and seen.get("k_conv2d_f32_dma_pairs", 0) >= 3, seen


@pytest.mark.parametrize("seed", range(12))
def test_conv_transpose2d_f32_random_shapes(ops, seed):
    r = np.random.default_rng(9600 + seed)
    g = int(r.choice([1, 1, 2]))
    C, OC = g * int(r.integers(1, 7)), g * int(r.integers(1, 7))
    k = (int(r.integers(1, 5)), int(r.integers(1, 5)))
    s = (int(r.integers(1, 4)), int(r.integers(1, 4)))
    d = (int(r.integers(1, 3)), int(r.integers(1, 3)))
    H, W = int(r.integers(1, 12)), int(r.integers(1, 12))
    p = tuple(int(v) for v in (r.integers(0, 2), r.integers(0, 2), r.integers(0, 2), r.integers(0, 2)))
    op = (int(r.integers(0, s[0])), int(r.integers(0, s[1])))
    OH = s[0] * (H - 1) + d[0] * (k[0] - 1) + 1 + op[0] - p[0] - p[2]
    OW = s[1] * (W - 1) + d[1] * (k[1] - 1) + 1 + op[1] - p[1] - p[3]
    if OH < 1 or OW < 1:
        pytest.skip("empty output")
    N = int(r.integers(1, 4))
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = r.standard_normal((C, OC // g) + k).astype(np.float32)
    b = r.standard_normal(OC).astype(np.float32) if seed % 2 else None
    ref = oracle.conv_transpose2d_f32(x, w, b, p, s, d, g, op)
    got = ops.conv_transpose2d_f32(x, w, b, p, s, d, g, op)
    assert got.shape == ref.shape
    assert np.max(np.abs(got - ref)) <= 1e-5 * max(1.0, float(np.max(np.abs(ref)))), (C, OC, g, k, s, d, p, op, H, W)


@pytest.mark.parametrize("seed", range(12))
def test_conv_transpose2d_f32_wide_layers(ops, seed):
    """Transposed convolutions with enough input channels that every output phase is a multiply of at least 16 taps x
    channels: the phases then run in the pipelined convolution kernel on gathered sub-kernels (uneven phases when the
    kernel size is not a multiple of the stride, groups, output padding, pads that differ begin to end)."""
    r = np.random.default_rng(9700 + seed)
    g = int(r.choice([1, 1, 2, 4]))
    C, OC = g * int(r.choice([4, 8, 12, 16, 32])), g * int(r.integers(1, 20))
    k = (int(r.integers(2, 6)), int(r.integers(2, 6)))
    s = (int(r.integers(1, 4)), int(r.integers(1, 4)))
    d = (1, 1) if seed % 4 else (int(r.integers(1, 3)), int(r.integers(1, 3)))
    H, W = int(r.integers(2, 24)), int(r.integers(2, 24))
    p = tuple(int(v) for v in r.integers(0, 3, 4))
    op = (int(r.integers(0, s[0])), int(r.integers(0, s[1])))
    OH = s[0] * (H - 1) + d[0] * (k[0] - 1) + 1 + op[0] - p[0] - p[2]
    OW = s[1] * (W - 1) + d[1] * (k[1] - 1) + 1 + op[1] - p[1] - p[3]
    if OH < 1 or OW < 1:
        pytest.skip("empty output")
    N = int(r.integers(1, 4))
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = r.standard_normal((C, OC // g) + k).astype(np.float32)
    b = r.standard_normal(OC).astype(np.float32) if seed % 2 else None
    ref = oracle.conv_transpose2d_f32(x, w, b, p, s, d, g, op)
    got = ops.conv_transpose2d_f32(x, w, b, p, s, d, g, op)
    assert got.shape == ref.shape
    assert np.max(np.abs(got - ref)) <= 1e-5 * max(1.0, float(np.max(np.abs(ref)))), (C, OC, g, k, s, d, p, op, H, W, N)


@pytest.mark.parametrize("seed", range(8))
def test_gemm_fp8_random_shapes(ops, seed):
    """The tolerance of the FP8 GEMM (one bf16 rounding of the result plus 7 * 2^-13 of the sum of magnitudes, against
    the float64-accumulated product of the same e4m3 operands) on random shapes and both layouts of B."""
    from sofie_amd import lib as L
    r = np.random.default_rng(9700 + seed)
    M, N = int(r.integers(1, 500)), 4 * int(r.integers(1, 120))
    K = 16 * int(r.integers(1, 70))
    transB = bool(r.integers(0, 2))
    a = r.standard_normal((M, K)).astype(np.float32)
    b = r.standard_normal((N, K) if transB else (K, N)).astype(np.float32)
    sa, sb = np.float32(np.abs(a).max() / 448.0), np.float32(np.abs(b).max() / 448.0)
    A, B = oracle.e4m3_encode(a / sa), oracle.e4m3_encode(b / sb)
    bias = r.standard_normal(N).astype(np.float32)
    yf = ops.gemm_fp8(A, B, sa, sb, bias, transB, out=L.OUT_F32)
    yb = ops.gemm_fp8(A, B, sa, sb, bias, transB)
    _, truth = oracle.gemm_fp8(A, B, sa, sb, bias, transB, acc64=True)
    da = np.abs(oracle.e4m3_decode(A)).astype(np.float64)
    db = np.abs(oracle.e4m3_decode(B)).astype(np.float64)
    # (seven products of a group of eight, each cut below 2^-13 of the group's largest: the matrix instruction's sums,
    # pinned in test_gpu_parity.py::test_fp8_matrix_instruction_sums_groups_of_eight)
    slack = 7 * 2.0 ** -13 * (da @ (db.T if transB else db)) * float(sa) * float(sb) + 1e-30
    assert np.all(np.abs(yf.astype(np.float64) - truth) <= slack + 2.0 ** -22 * np.abs(truth)), (M, N, K, transB)
    assert np.all(np.abs(oracle.bf16_decode(yb).astype(np.float64) - truth) <= 2.0 ** -8 * np.abs(truth) + slack)
    assert np.array_equal(yb, oracle.bf16_encode(yf))


@pytest.mark.parametrize("seed", range(14))
def test_mlp_f32_random_chains(ops, seed):
    """The one-launch chain of fully connected layers against the oracle's Gemm applied layer by layer."""
    r = np.random.default_rng(9800 + seed)
    n = int(r.integers(1, 6))
    dims = [int(r.integers(1, 300)) for _ in range(n + 1)]
    if seed == 0:
        n, dims = 3, [64, 128, 64, 8]                 # the benchmark's MLP
    if seed == 1:
        n, dims = 2, [700, 1024, 513]                 # wide layers: more than one pass of 256 columns
    M = int(r.choice([1, 7, 256, 700, 3000])) if seed > 1 else 256
    x = r.standard_normal((M, dims[0])).astype(np.float32)
    Ws = [(r.standard_normal((dims[i], dims[i + 1])) / np.sqrt(dims[i])).astype(np.float32) for i in range(n)]
    bs = [r.standard_normal(dims[i + 1]).astype(np.float32) if (seed + i) % 3 else None for i in range(n)]
    relus = [bool((seed + i) % 2) for i in range(n)]
    ref = x
    for i in range(n):
        ref = oracle.gemm_f32(ref, Ws[i], bs[i], 1.0, 1.0 if bs[i] is not None else 0.0, False, False, relus[i])
    got = ops.mlp_f32(x, Ws, bs, relus)
    assert got.shape == ref.shape
    assert np.max(np.abs(got - ref)) <= 1e-5 * max(1.0, float(np.max(np.abs(ref)))), (dims, M)


@pytest.mark.parametrize("M,K,N1,N2", [(4096, 12800, 256, 5), (512, 8192, 128, 8), (300, 8464, 64, 3), (1024, 16384, 32, 1),
                                        (700, 1040, 96, 4), (256, 8192, 256, 12), (64, 512, 100, 5)])
def test_qgemm_s8_pair(ops, M, K, N1, N2):
    """Two QLinearMatMul layers in one call against the two separate calls of the oracle: shapes whose first layer is
    cut into K slices (the second layer then rides on the pass that adds the slices) and shapes that take the two
    ordinary calls; int8 and float output."""
    from sofie_amd import lib as L
    r = np.random.default_rng(9900 + M + N1 + N2)
    A = r.integers(-128, 128, (M, K)).astype(np.int8)
    B1 = r.integers(-127, 128, (N1, K)).astype(np.int8)
    B2 = r.integers(-127, 128, (N2, N1)).astype(np.int8)
    s1 = (r.uniform(20, 60, N1) / (73.3 * 73.3 * np.sqrt(K))).astype(np.float32)
    s2 = (r.uniform(20, 60, N2) / (73.3 * 73.3 * np.sqrt(N1))).astype(np.float32)
    b1 = r.integers(-2000, 2000, N1).astype(np.int32)
    b2 = r.integers(-2000, 2000, N2).astype(np.int32)
    for zp_mid, relu1, zpy, relu2 in ((-128, True, 3, False), (5, False, -128, True)):
        T = oracle.qgemm_s8(A, B1, s1, b1, True, 0, zp_mid, relu1)
        q2 = ops.fold_zero_point_gemm(B2, b2, zp_mid, True)
        ref = oracle.qgemm_s8(T, B2, s2, q2, True, 0, zpy, relu2)
        got = ops.qgemm_s8_pair(A, B1, s1, b1, zp_mid, relu1, B2, s2, q2, zpy, relu2)
        assert np.array_equal(got, ref), (zp_mid, relu1, zpy, relu2)
        reff = oracle.qgemm_s8_f32out(T, B2, s2, q2, True, 0, relu2)
        gotf = ops.qgemm_s8_pair(A, B1, s1, b1, zp_mid, relu1, B2, s2, q2, 0, relu2, out=L.OUT_F32)
        assert np.array_equal(gotf, reff)
