"""Small graphs with seeded random attributes, for the tests that run the emitter's output against an implementation
that shares nothing with it: float graphs (Conv with groups, strides, dilations and four different pads, then Relu,
MaxPool, AveragePool or Flatten + Gemm) against torch on the CPU, quantized graphs (QuantizeLinear, QLinearConv with
per-channel scales, optional Relu and 2x2 MaxPool, DequantizeLinear) against the oracle's integer arithmetic."""
import numpy as np

from sofie_amd import emit

FLOAT_SEEDS = (1, 2, 7, 10, 13, 18, 22, 31)
QUANT_SEEDS = (0, 1, 3, 5, 6, 9)


def float_graph(seed, prefix="rg"):
    """(spec, input, expected flat output) or None when the seed's kernel does not fit its padded image."""
    import torch
    import torch.nn.functional as F
    r = np.random.default_rng(seed)
    g = int(r.choice([1, 1, 2, 4]))
    C, OC = g * int(r.integers(1, 5)), g * int(r.integers(1, 6))
    kh, kw = int(r.integers(1, 5)), int(r.integers(1, 5))
    sh, sw = int(r.integers(1, 4)), int(r.integers(1, 4))
    dh, dw = int(r.integers(1, 3)), int(r.integers(1, 3))
    pads = [int(v) for v in r.integers(0, 3, 4)]      # ONNX order: top, left, bottom, right
    N, H, W = int(r.integers(1, 4)), int(r.integers(6, 20)), int(r.integers(6, 20))
    if H + pads[0] + pads[2] < dh * (kh - 1) + 1 or W + pads[1] + pads[3] < dw * (kw - 1) + 1:
        return None
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = r.standard_normal((OC, C // g, kh, kw)).astype(np.float32)
    b = r.standard_normal(OC).astype(np.float32) if seed % 3 else None
    s = emit.ModelSpec("%s%d" % (prefix, seed))
    s.add_input("x", "FLOAT", x.shape)
    s.add_init("w", w)
    if b is not None:
        s.add_init("b", b)
    s.conv("x", "w", "b" if b is not None else None, "c", (kh, kw), tuple(pads), (sh, sw), (dh, dw), g)
    t = F.conv2d(F.pad(torch.from_numpy(x), (pads[1], pads[3], pads[0], pads[2])), torch.from_numpy(w),
                 None if b is None else torch.from_numpy(b), (sh, sw), 0, (dh, dw), g)
    cur = "c"
    if seed % 2:
        s.relu(cur, "r")
        cur, t = "r", torch.relu(t)
    mode = seed % 4
    if mode in (1, 2) and t.shape[2] >= 3 and t.shape[3] >= 3:
        k = (int(r.integers(1, 4)), int(r.integers(1, 4)))
        st = (int(r.integers(1, 3)), int(r.integers(1, 3)))
        pp = [int(v) for v in r.integers(0, 2, 4)]
        pp = [min(pp[0], k[0] - 1), min(pp[1], k[1] - 1), min(pp[2], k[0] - 1), min(pp[3], k[1] - 1)]
        around = (pp[1], pp[3], pp[0], pp[2])
        if mode == 1:
            s.maxpool(cur, "p", k, tuple(pp), st)
            t = F.max_pool2d(F.pad(t, around, value=float("-inf")), k, st)
        else:
            include = seed % 8 < 4
            s.avgpool(cur, "p", k, tuple(pp), st, include)
            sums = F.avg_pool2d(F.pad(t, around), k, st) * (k[0] * k[1])
            cells = F.avg_pool2d(F.pad(torch.ones_like(t), around), k, st) * (k[0] * k[1])
            t = sums / (k[0] * k[1]) if include else sums / cells
        cur = "p"
    if mode == 3:
        s.flatten(cur, "f")
        t = t.flatten(1)
        no = int(r.integers(1, 9))
        w2 = r.standard_normal((no, t.shape[1])).astype(np.float32)
        b2 = r.standard_normal(no).astype(np.float32)
        s.add_init("W2", w2)
        s.add_init("b2", b2)
        s.gemm("f", "W2", "b2", "y2", transB=1, relu=seed % 8 == 3)
        t = t @ torch.from_numpy(w2).T + torch.from_numpy(b2)
        t = torch.relu(t) if seed % 8 == 3 else t
        cur = "y2"
    s.set_output(cur)
    return s, x, t.numpy().reshape(-1)


def quantized_graph(seed, oracle, prefix="rq"):
    """(spec, float input, expected flat float output: exact, the output is a dequantised int8 tensor) or None."""
    r = np.random.default_rng(50000 + seed)
    g = int(r.choice([1, 1, 1, 2, 4]))
    C = g * int(r.choice([1, 2, 3, 8, 16]))
    if seed % 5 == 0:
        C, g = int(r.choice([32, 64])), 1            # the shapes of the ring kernel
    OC = g * int(r.integers(1, 20)) if seed % 4 else int(r.choice([64, 128]))
    k, st, pd = int(r.integers(1, 5)), int(r.integers(1, 3)), int(r.integers(0, 3))
    if seed % 5 == 0:
        k, st, pd = 3, 1, 1
    N, H, W = int(r.integers(1, 5)), int(r.integers(5, 24)), int(r.integers(5, 24))
    if H + 2 * pd < k or W + 2 * pd < k:
        return None
    x = r.uniform(-1, 1, (N, C, H, W)).astype(np.float32)
    w = r.integers(-127, 128, (OC, C // g, k, k)).astype(np.int8)
    sw = r.uniform(0.001, 0.003, OC).astype(np.float32)
    b = r.integers(-500, 500, OC).astype(np.int32) if seed % 3 else None
    sx, zx = np.float32(1 / 127.0), int(r.choice([0, 3, -128, 5]))
    sy, zy = np.float32(r.uniform(0.02, 0.08)), int(r.choice([0, -7, -128, 10]))
    relu, pool = bool(seed % 2), seed % 4 == 1
    s = emit.ModelSpec("%s%d" % (prefix, seed))
    s.add_input("x", "FLOAT", x.shape)
    s.add_scalar("sx", sx, np.float32)
    s.add_scalar("zx", zx, np.int8)
    s.add_scalar("sy", sy, np.float32)
    s.add_scalar("zy", zy, np.int8)
    s.add_init("w", w)
    s.add_init("sw", sw)
    if b is not None:
        s.add_init("b", b)
    s.quantize("x", "sx", "zx", "xq")
    s.qlinear_conv("xq", "sx", "zx", "w", "sw", None, "sy", "zy", "c", "b" if b is not None else None, (k, k),
                   (pd, pd, pd, pd), (st, st), group=g)
    cur = "c"
    xq = oracle.quantize_f32_s8(x, sx, zx)
    scale = ((sx * sw).astype(np.float32) / sy).astype(np.float32)
    c = oracle.qconv2d_s8(xq, w, scale, b, (pd, pd), (st, st), g, zx, zy, relu)
    if relu:
        s.relu(cur, "r")
        cur = "r"
    if pool and c.shape[2] >= 2 and c.shape[3] >= 2:
        s.maxpool(cur, "p", (2, 2), (0, 0, 0, 0), (2, 2))
        cur, c = "p", oracle.maxpool2d(c, (2, 2), (2, 2))
    s.dequantize(cur, "sy", "zy", "y")
    s.set_output("y")
    return s, x, oracle.dequantize_s8_f32(c, sy, zy).reshape(-1)
