"""The networks the tests and the benchmark push through the C++ emitter, with seeded weights, and the
CPU-oracle evaluation of each (test infrastructure)."""
import os

import numpy as np

from sofie_amd import emit, onnx_wire

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FIXTURES = ["Linear_16", "Linear_32", "Linear_64", "ConvWithPadding", "ConvWithoutPadding",
            "ConvWithAutopadSameLower", "ConvWithStridesPadding", "ConvWithStridesNoPadding",
            "ConvWithAsymmetricPadding", "MaxPool1d", "MaxPool2d", "MaxPool3d", "AvgPool", "ConvTranspose1d", "ConvTranspose2d", "ConvTransposeBias2d",
            "ConvTransposeBias2dBatched", "Einsum_matmul", "Einsum_dotprod", "Einsum_3", "Einsum_4"]


def fixture_spec(name):
    graph = onnx_wire.load(os.path.join(GOLD, "onnx", name + ".onnx"))
    return emit.spec_from_onnx(name, graph), graph


# ------------------------------------------------------------------------------------------ fp32 MLP
def mlp_weights(seed=0):
    """Glorot-uniform weights, zero biases, N(0,1) input; draw order W1, W2, W3, x."""
    r = np.random.default_rng(seed)
    dims = [(64, 128), (128, 64), (64, 8)]
    Ws = [r.uniform(-np.sqrt(6.0 / (a + b)), np.sqrt(6.0 / (a + b)), (a, b)).astype(np.float32) for a, b in dims]
    Bs = [np.zeros(b, np.float32) for _, b in dims]
    x = r.standard_normal((256, 64)).astype(np.float32)
    return Ws, Bs, x


def mlp_spec(name="mlp_c1", seed=0):
    Ws, Bs, x = mlp_weights(seed)
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", x.shape)
    for i, (W, B) in enumerate(zip(Ws, Bs)):
        s.add_init("W%d" % i, W)
        s.add_init("B%d" % i, B)
    s.gemm("x", "W0", "B0", "h0", relu=True)
    s.gemm("h0", "W1", "B1", "h1", relu=True)
    s.gemm("h1", "W2", "B2", "y")
    s.set_output("y")
    return s, x


def mlp_reference(oracle, seed=0):
    Ws, Bs, x = mlp_weights(seed)
    h = oracle.gemm_f32(x, Ws[0], Bs[0], relu=True)
    h = oracle.gemm_f32(h, Ws[1], Bs[1], relu=True)
    return oracle.gemm_f32(h, Ws[2], Bs[2])


# ------------------------------------------------------------------------------------------ CNN (fp32 and int8)
def cnn_float_params(seed=1):
    r = np.random.default_rng(seed)

    def kaiming(shape):
        fan = int(np.prod(shape[1:]))
        return (r.standard_normal(shape) * np.sqrt(2.0 / fan)).astype(np.float32)
    p = {"w1": kaiming((32, 1, 3, 3)), "w2": kaiming((64, 32, 3, 3)), "w3": kaiming((128, 64, 3, 3)),
         "fc1": kaiming((256, 12800)).T.copy(), "fc2": kaiming((5, 256)).T.copy()}
    for k, n in (("b1", 32), ("b2", 64), ("b3", 128), ("bf1", 256), ("bf2", 5)):
        p[k] = (r.standard_normal(n) * 0.05).astype(np.float32)
    return p


def cnn_input(batch, seed=2):
    return np.random.default_rng(seed).uniform(0, 1, (batch, 1, 40, 40)).astype(np.float32)


def cnn_f32_spec(batch, name="cnn_f32"):
    p = cnn_float_params()
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", (batch, 1, 40, 40))
    for k, v in p.items():
        s.add_init(k, v)
    s.conv("x", "w1", "b1", "c1", (3, 3), (1, 1, 1, 1), (1, 1)); s.relu("c1", "r1")
    s.maxpool("r1", "p1", (2, 2), (0, 0, 0, 0), (2, 2))
    s.conv("p1", "w2", "b2", "c2", (3, 3), (1, 1, 1, 1), (1, 1)); s.relu("c2", "r2")
    s.maxpool("r2", "p2", (2, 2), (0, 0, 0, 0), (2, 2))
    s.conv("p2", "w3", "b3", "c3", (3, 3), (1, 1, 1, 1), (1, 1)); s.relu("c3", "r3")
    s.flatten("r3", "f")
    s.gemm("f", "fc1", "bf1", "g1"); s.relu("g1", "rg1")
    s.gemm("rg1", "fc2", "bf2", "y")
    s.set_output("y")
    return s


def cnn_f32_stages(oracle, x):
    """Float activations after every layer (also used to calibrate the int8 network)."""
    p = cnn_float_params()
    a1 = oracle.conv2d_f32(x, p["w1"], p["b1"], (1, 1), relu=True)
    q1 = oracle.maxpool2d(a1, (2, 2), (2, 2))
    a2 = oracle.conv2d_f32(q1, p["w2"], p["b2"], (1, 1), relu=True)
    q2 = oracle.maxpool2d(a2, (2, 2), (2, 2))
    a3 = oracle.conv2d_f32(q2, p["w3"], p["b3"], (1, 1), relu=True)
    f = a3.reshape(a3.shape[0], -1)
    g1 = oracle.gemm_f32(f, p["fc1"], p["bf1"], relu=True)
    y = oracle.gemm_f32(g1, p["fc2"], p["bf2"])
    return {"a1": a1, "a2": a2, "a3": a3, "g1": g1, "y": y}


_QP = None


def qcnn_params(oracle):
    """Per-output-channel symmetric int8 weights, int32 biases, activation scales from a seeded
    calibration batch (max / 255 with zero-point -128, i.e. the uint8 range of a post-ReLU tensor)."""
    global _QP
    if _QP is not None:
        return _QP
    p = cnn_float_params()
    st = cnn_f32_stages(oracle, cnn_input(8, seed=3))
    q = {"sx": np.float32(1.0 / 255.0)}
    for k in ("a1", "a2", "a3", "g1"):
        q["s_" + k] = np.float32(float(st[k].max()) / 255.0)

    def qweights(w, axis_out):
        flat = w.reshape(w.shape[0], -1) if axis_out == 0 else w.T.reshape(w.shape[1], -1)
        sw = (np.abs(flat).max(axis=1) / 127.0).astype(np.float32)
        shape = [-1] + [1] * (w.ndim - 1) if axis_out == 0 else [1, -1]
        wq = np.clip(np.rint(w / sw.reshape(shape)), -127, 127).astype(np.int8)
        return wq, sw
    s_in = {"w1": q["sx"], "w2": q["s_a1"], "w3": q["s_a2"], "fc1": q["s_a3"], "fc2": q["s_g1"]}
    bias = {"w1": "b1", "w2": "b2", "w3": "b3", "fc1": "bf1", "fc2": "bf2"}
    for k in ("w1", "w2", "w3"):
        q[k], q["s_" + k] = qweights(p[k], 0)
    for k in ("fc1", "fc2"):
        q[k], q["s_" + k] = qweights(p[k], 1)      # [K,N], scale per column
    for k, b in bias.items():
        q[b] = np.rint(p[b] / (s_in[k] * q["s_" + k])).astype(np.int32)
    _QP = q
    return q


def qcnn_spec(oracle, batch, name="qcnn"):
    q = qcnn_params(oracle)
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", (batch, 1, 40, 40))
    s.add_scalar("sx", q["sx"], np.float32)
    s.add_scalar("zp", -128, np.int8)
    for k in ("a1", "a2", "a3", "g1"):
        s.add_scalar("s_" + k, q["s_" + k], np.float32)
    for k in ("w1", "w2", "w3", "fc1", "fc2"):
        s.add_init(k, q[k])
        s.add_init("s_" + k, q["s_" + k])
    for b in ("b1", "b2", "b3", "bf1", "bf2"):
        s.add_init(b, q[b])
    s.quantize("x", "sx", "zp", "xq")
    s.qlinear_conv("xq", "sx", "zp", "w1", "s_w1", None, "s_a1", "zp", "c1", "b1", (3, 3), (1, 1, 1, 1), (1, 1))
    s.relu("c1", "r1")
    s.maxpool("r1", "p1", (2, 2), (0, 0, 0, 0), (2, 2))
    s.qlinear_conv("p1", "s_a1", "zp", "w2", "s_w2", None, "s_a2", "zp", "c2", "b2", (3, 3), (1, 1, 1, 1), (1, 1))
    s.relu("c2", "r2")
    s.maxpool("r2", "p2", (2, 2), (0, 0, 0, 0), (2, 2))
    s.qlinear_conv("p2", "s_a2", "zp", "w3", "s_w3", None, "s_a3", "zp", "c3", "b3", (3, 3), (1, 1, 1, 1), (1, 1))
    s.relu("c3", "r3")
    s.flatten("r3", "f")
    s.qlinear_matmul("f", "s_a3", "zp", "fc1", "s_fc1", None, "s_g1", "zp", "g1", "bf1")
    s.relu("g1", "rg1")
    s.qlinear_matmul("rg1", "s_g1", "zp", "fc2", "s_fc2", None, None, None, "y", "bf2")
    s.set_output("y")
    return s


def qcnn_rt_spec(oracle, name="qcnn_rt"):
    """The int8 CNN with the batch as a shape parameter of the input ("bs"): generated with a capacity, run with any
    batch up to it."""
    s = qcnn_spec(oracle, "bs", name)
    s.batch, s.runtime_batch = 8, True
    return s


def cnn_f32_rt_spec(name="cnn_f32_rt"):
    s = cnn_f32_spec("bs", name)
    s.batch, s.runtime_batch = 8, True
    return s


def qcnn_reference(oracle, x):
    """The same network evaluated with the CPU oracle; per-channel scales are formed in fp32 in the
    emitter's order, (s_in * s_w[n]) / s_out."""
    q = qcnn_params(oracle)
    f32 = np.float32
    xq = oracle.quantize_f32_s8(x, q["sx"], -128)

    def conv(xi, w, b, s_in, s_out):
        scale = ((f32(s_in) * q["s_" + w]).astype(f32) / f32(s_out)).astype(f32)
        return oracle.qconv2d_s8(xi, q[w], scale, q[b], (1, 1), (1, 1), 1, -128, -128, True)
    c1 = oracle.maxpool2d(conv(xq, "w1", "b1", q["sx"], q["s_a1"]), (2, 2), (2, 2))
    c2 = oracle.maxpool2d(conv(c1, "w2", "b2", q["s_a1"], q["s_a2"]), (2, 2), (2, 2))
    c3 = conv(c2, "w3", "b3", q["s_a2"], q["s_a3"])
    f = c3.reshape(c3.shape[0], -1)
    s1 = ((f32(q["s_a3"]) * q["s_fc1"]).astype(f32) / f32(q["s_g1"])).astype(f32)
    g1 = oracle.qgemm_s8(f, q["fc1"], s1, q["bf1"], False, zpa=-128, zpy=-128, relu=True)
    s2 = (f32(q["s_g1"]) * q["s_fc2"]).astype(f32)
    bias2 = (q["bf2"].astype(np.int64) + 128 * q["fc2"].astype(np.int64).sum(axis=0)).astype(np.int32)
    acc = oracle.igemm_s8(g1, q["fc2"]).astype(np.int64) + bias2
    return (acc.astype(np.int32).astype(f32) * s2).astype(f32)


# ------------------------------------------------------------------------------------------ QDQ conv layer
def qdq_conv_params(seed=7):
    """One quantized conv layer between QuantizeLinear and DequantizeLinear: float [2,32,9,7] in, float
    [2,64,9,7] out. Exercises NCHW int8 input, channels-last output and the conversion back for float."""
    r = np.random.default_rng(seed)
    x = r.uniform(-1, 1, (2, 32, 9, 7)).astype(np.float32)
    w = r.integers(-127, 128, (64, 32, 3, 3)).astype(np.int8)
    sw = r.uniform(0.001, 0.003, 64).astype(np.float32)
    b = r.integers(-500, 500, 64).astype(np.int32)
    return {"x": x, "w": w, "sw": sw, "b": b, "sx": np.float32(1 / 127.0), "zx": 3, "sy": np.float32(0.05), "zy": -7}


def qdq_conv_spec(name="qdq_conv"):
    p = qdq_conv_params()
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", p["x"].shape)
    s.add_scalar("sx", p["sx"], np.float32)
    s.add_scalar("zx", p["zx"], np.int8)
    s.add_scalar("sy", p["sy"], np.float32)
    s.add_scalar("zy", p["zy"], np.int8)
    s.add_init("w", p["w"])
    s.add_init("sw", p["sw"])
    s.add_init("b", p["b"])
    s.quantize("x", "sx", "zx", "xq")
    s.qlinear_conv("xq", "sx", "zx", "w", "sw", None, "sy", "zy", "c", "b", (3, 3), (1, 1, 1, 1), (1, 1))
    s.dequantize("c", "sy", "zy", "y")
    s.set_output("y")
    return s


def qdq_conv_reference(oracle):
    p = qdq_conv_params()
    xq = oracle.quantize_f32_s8(p["x"], p["sx"], p["zx"])
    scale = ((p["sx"] * p["sw"]).astype(np.float32) / p["sy"]).astype(np.float32)
    c = oracle.qconv2d_s8(xq, p["w"], scale, p["b"], (1, 1), (1, 1), 1, p["zx"], p["zy"], False)
    return oracle.dequantize_s8_f32(c, p["sy"], p["zy"])


# ------------------------------------------------------------------------------------------ conv + batch norm
def convbn_params(seed=21):
    """Conv(3->16) -> BatchNormalization -> Relu -> MaxPool -> BatchNormalization -> ConvTranspose(16->4, stride 2) ->
    Relu on [4,3,12,12]: the first normalisation folds into the convolution, the second one runs as its own
    kernel (it follows a pooling), the transposed convolution takes the fused Relu."""
    r = np.random.default_rng(seed)
    p = {"x": r.standard_normal((4, 3, 12, 12)).astype(np.float32),
         "w1": (r.standard_normal((16, 3, 3, 3)) * 0.3).astype(np.float32), "b1": r.standard_normal(16).astype(np.float32),
         "wt": (r.standard_normal((16, 4, 4, 4)) * 0.2).astype(np.float32), "bt": r.standard_normal(4).astype(np.float32)}
    for k in ("1", "2"):
        p["g" + k] = r.uniform(0.5, 1.5, 16).astype(np.float32)
        p["beta" + k] = r.standard_normal(16).astype(np.float32)
        p["mean" + k] = r.standard_normal(16).astype(np.float32)
        p["var" + k] = r.uniform(0.2, 2.0, 16).astype(np.float32)
    return p


def convbn_spec(name="convbn"):
    p = convbn_params()
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", p["x"].shape)
    for k in ("w1", "b1", "wt", "bt", "g1", "beta1", "mean1", "var1", "g2", "beta2", "mean2", "var2"):
        s.add_init(k, p[k])
    s.conv("x", "w1", "b1", "c1", (3, 3), (1, 1, 1, 1), (1, 1))
    s.batchnorm("c1", "g1", "beta1", "mean1", "var1", "n1", 1e-5)
    s.relu("n1", "r1")
    s.maxpool("r1", "p1", (2, 2), (0, 0, 0, 0), (2, 2))
    s.batchnorm("p1", "g2", "beta2", "mean2", "var2", "n2", 1e-3)
    s.conv_transpose("n2", "wt", "bt", "t1", (), (1, 1, 1, 1), (2, 2))
    s.relu("t1", "y")
    s.set_output("y")
    return s


def convbn_reference(oracle):
    p = convbn_params()
    c1 = oracle.conv2d_f32(p["x"], p["w1"], p["b1"], (1, 1), (1, 1))
    r1 = oracle.batchnorm_f32(c1, p["g1"], p["beta1"], p["mean1"], p["var1"], 1e-5, relu=True)
    p1 = oracle.maxpool2d(r1, (2, 2), (2, 2))
    n2 = oracle.batchnorm_f32(p1, p["g2"], p["beta2"], p["mean2"], p["var2"], 1e-3)
    return oracle.conv_transpose2d_f32(n2, p["wt"], p["bt"], (1, 1, 1, 1), (2, 2), relu=True)


# ------------------------------------------------------------------------------------------ 1-D and 3-D convolutions
def conv1d_params(seed=51):
    r = np.random.default_rng(seed)
    return {"x": r.standard_normal((3, 4, 50)).astype(np.float32), "w": (r.standard_normal((6, 2, 5)) * 0.3).astype(np.float32),
            "b": r.standard_normal(6).astype(np.float32)}


def conv1d_spec(name="conv1d"):
    """Conv on [3,4,50] with a [6,2,5] kernel in two groups, stride 2, dilation 2, the default pads (1 per side), then Relu."""
    p = conv1d_params()
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", p["x"].shape)
    s.add_init("w", p["w"])
    s.add_init("b", p["b"])
    s.conv("x", "w", "b", "c", (), (), (2,), (2,), 2)
    s.relu("c", "y")
    s.set_output("y")
    return s


def conv1d_reference(oracle):
    p = conv1d_params()
    y = oracle.conv2d_f32(p["x"][:, :, None, :], p["w"][:, :, None, :], p["b"], (0, 1), (1, 2), (1, 2), 2, relu=True)
    return y[:, :, 0, :]


def conv3d_params(seed=52):
    r = np.random.default_rng(seed)
    return {"x": r.standard_normal((2, 4, 6, 9, 10)).astype(np.float32),
            "w": (r.standard_normal((6, 2, 3, 2, 3)) * 0.3).astype(np.float32), "b": r.standard_normal(6).astype(np.float32)}


def conv3d_spec(name="conv3d"):
    """Conv on [2,4,6,9,10] with a [6,2,3,2,3] kernel in two groups, strides (1,2,1), pads (1,0,2) on both sides."""
    p = conv3d_params()
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", p["x"].shape)
    s.add_init("w", p["w"])
    s.add_init("b", p["b"])
    s.conv("x", "w", "b", "y", (3, 2, 3), (1, 0, 2, 1, 0, 2), (1, 2, 1), (), 2)
    s.set_output("y")
    return s


def conv3d_reference(oracle):
    p = conv3d_params()
    return oracle.conv3d_f32(p["x"], p["w"], p["b"], (1, 0, 2), (1, 2, 1), (1, 1, 1), 2)


# ------------------------------------------------------------------------------------------ pooling over one and three axes
def pool1d_input(seed=53):
    return np.random.default_rng(seed).standard_normal((3, 4, 50)).astype(np.float32)


def pool1d_spec(name="pool1d"):
    """MaxPool on [3,4,50] (window 3, pads 1 and 1, stride 2) then AveragePool (window 4, pads 2 and 1, stride 1)."""
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", pool1d_input().shape)
    s.maxpool("x", "m", (3,), (1, 1), (2,))
    s.avgpool("m", "y", (4,), (2, 1), (1,))
    s.set_output("y")
    return s


def pool1d_reference(oracle):
    m = oracle.maxpool2d(pool1d_input()[:, :, None, :], (1, 3), (1, 2), (0, 1, 0, 1))
    return oracle.avgpool2d(m, (1, 4), (1, 1), (0, 2, 0, 1))[:, :, 0, :]


def pool3d_input(seed=54):
    return np.random.default_rng(seed).standard_normal((2, 3, 8, 9, 10)).astype(np.float32)


def pool3d_spec(name="pool3d"):
    """MaxPool on [2,3,8,9,10] (window 2x3x2, begin pads 1,0,1, end pads 0,1,0, strides 2,1,2) then AveragePool that
    counts the padding cells (window 2x2x3, begin pads 0,1,1, end pads 1,0,1, strides 1,2,1)."""
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", pool3d_input().shape)
    s.maxpool("x", "m", (2, 3, 2), (1, 0, 1, 0, 1, 0), (2, 1, 2))
    s.avgpool("m", "y", (2, 2, 3), (0, 1, 1, 1, 0, 1), (1, 2, 1), count_include_pad=True)
    s.set_output("y")
    return s


def pool3d_reference(oracle):
    m = oracle.pool3d(pool3d_input(), (2, 3, 2), (2, 1, 2), (1, 0, 1, 0, 1, 0))
    return oracle.pool3d(m, (2, 2, 3), (1, 2, 1), (0, 1, 1, 1, 0, 1), average=True, count_include_pad=True)


# ------------------------------------------------------------------------------------------ four-value model for SofieFunctor
def functor_params(seed=33):
    r = np.random.default_rng(seed)
    return {"W1": r.standard_normal((4, 8)).astype(np.float32), "B1": r.standard_normal(8).astype(np.float32),
            "W2": r.standard_normal((8, 1)).astype(np.float32), "B2": r.standard_normal(1).astype(np.float32),
            "rows": r.standard_normal((64, 4)).astype(np.float32)}


def functor_spec(name="functor4"):
    p = functor_params()
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", (1, 4))
    for k in ("W1", "B1", "W2", "B2"):
        s.add_init(k, p[k])
    s.gemm("x", "W1", "B1", "h", relu=True)
    s.gemm("h", "W2", "B2", "y")
    s.set_output("y")
    return s


def functor_reference(oracle):
    p = functor_params()
    h = oracle.gemm_f32(p["rows"], p["W1"], p["B1"], relu=True)
    return oracle.gemm_f32(h, p["W2"], p["B2"]).reshape(-1)


# ------------------------------------------------------------------------------------------ stacked MatMul
def stacked_params(seed=44):
    r = np.random.default_rng(seed)
    return {"x": r.standard_normal((2, 1, 4, 5)).astype(np.float32), "B1": r.standard_normal((3, 5, 6)).astype(np.float32),
            "B2": r.standard_normal((6, 2)).astype(np.float32)}


def stacked_spec(name="stacked"):
    """x [2,1,4,5] @ B1 [3,5,6] -> [2,3,4,6] (both operands broadcast over a leading dimension), then @ B2 [6,2]
    -> [2,3,4,2] (a plain matrix against a stack)."""
    p = stacked_params()
    s = emit.ModelSpec(name)
    s.add_input("x", "FLOAT", p["x"].shape)
    s.add_init("B1", p["B1"])
    s.add_init("B2", p["B2"])
    s.gemm("x", "B1", None, "h", 1.0, 0.0)
    s.gemm("h", "B2", None, "y", 1.0, 0.0)
    s.set_output("y")
    return s


def stacked_reference():
    p = stacked_params()
    return np.matmul(np.matmul(p["x"].astype(np.float64), p["B1"].astype(np.float64)), p["B2"].astype(np.float64))


# ------------------------------------------------------------------------------------------ several outputs
def two_heads_spec(name="two_heads", seed=0):
    """The MLP with its second hidden layer and its last layer both listed as outputs (one type: infer()
    returns a vector of vectors, as the reference's does)."""
    s, x = mlp_spec(name, seed)
    s.lines = [ln for ln in s.lines if not ln.startswith("output ")]
    s.output, s.outputs = None, []
    s.set_output("h1")
    s.set_output("y")
    return s, x


def two_heads_reference(oracle, seed=0):
    Ws, Bs, x = mlp_weights(seed)
    h = oracle.gemm_f32(x, Ws[0], Bs[0], relu=True)
    h1 = oracle.gemm_f32(h, Ws[1], Bs[1], relu=True)
    return h1, oracle.gemm_f32(h1, Ws[2], Bs[2])


MIXED_SCALE, MIXED_ZP = 0.05, 3


def mixed_outputs_spec(name="mixed_outputs", seed=0):
    """The MLP's float result and its QuantizeLinear image as two outputs (different types: infer() returns a
    tuple of vectors, as the reference's does)."""
    s, x = mlp_spec(name, seed)
    s.lines = [ln for ln in s.lines if not ln.startswith("output ")]
    s.output, s.outputs = None, []
    s.add_scalar("sq", MIXED_SCALE, np.float32)
    s.add_scalar("zq", MIXED_ZP, np.int8)
    s.quantize("y", "sq", "zq", "q")
    s.set_output("y")
    s.set_output("q", "INT8")
    return s, x


def mixed_outputs_reference(oracle, seed=0):
    y = mlp_reference(oracle, seed)
    return y, oracle.quantize_f32_s8(y, MIXED_SCALE, MIXED_ZP)


def mlp_nosession_spec(name="mlp_nosession", seed=0):
    """The MLP generated with Options::kNoSession: a free function infer, weights as literals."""
    s, x = mlp_spec(name, seed)
    s.no_session = True
    return s, x
