"""Host-side code generator (RModel / ROperator mirror): generation, fusion, memory plan, weight file
format and error behaviour. No GPU needed: the generated Sessions are only compiled here."""
import os
import re
import subprocess

import numpy as np
import pytest

import models
from oracle import oracle
from sofie_amd import emit


@pytest.fixture(scope="module", autouse=True)
def _emitter():
    emit.build_emitter()


def gen(spec, tmp_path, **kw):
    return spec.generate(str(tmp_path), **kw)


def test_weight_file_text_matches_the_reference_format(tmp_path):
    """`tensor_<name> <count>` header line, one value line, max_digits10 significant digits: the text the
    reference writes for B = [0.5, 0.5, -10, 0] and a 12-element W (RModel.cxx:1121-1158)."""
    s = emit.ModelSpec("probe")
    s.add_input("x", "FLOAT", (2, 3))
    s.add_init("B", np.array([0.5, 0.5, -10, 0], np.float32))
    s.add_init("W", np.array([1, 2, 3, -1, -2, -3, 0.5, 0.5, 0.5, 0, 0, 1], np.float32).reshape(4, 3))
    s.gemm("x", "W", "B", "y", transB=1, relu=True)
    s.set_output("y")
    hxx, dat, _ = gen(s, tmp_path)
    assert open(dat).read() == "tensor_B 4\n0.5 0.5 -10 0\ntensor_W 12\n1 2 3 -1 -2 -3 0.5 0.5 0.5 0 0 1\n"
    code = open(hxx).read()
    assert "namespace SOFIE_probe{" in code and "struct Session {" in code
    assert 'Session(std::string filename ="probe.dat"' in code
    assert "std::vector<float> infer(float* tensor_x)" in code
    # Gemm with transB, rank-1 bias broadcast in the epilogue (kind 1), fused ReLU
    assert re.search(r"sofie_hip_gemm_f32\(fCtx, 0, 1, 2, 4, 3, .*tensor_x, 3, tensor_W, 3, .*tensor_B, 1, tensor_y, 4, SOFIE_ACT_RELU\)", code)


def test_subnormal_weights_are_flushed_and_digits_round_trip(tmp_path):
    s = emit.ModelSpec("tiny")
    s.add_input("x", "FLOAT", (1, 2))
    w = np.array([[1e-42, 0.1], [np.float32(1) / 3, -2.5e-39]], np.float32)
    s.add_init("W", w)
    s.gemm("x", "W", None, "y", beta=0.0)
    s.set_output("y")
    _, dat, _ = gen(s, tmp_path)
    vals = np.array(open(dat).read().split("\n")[1].split(), np.float64).astype(np.float32)
    want = w.reshape(-1).copy()
    want[np.abs(want) < np.finfo(np.float32).tiny] = 0
    assert np.array_equal(vals, want)          # 9 significant digits reproduce every float32 exactly


def test_relu_after_gemm_and_conv_is_fused_and_flatten_is_a_view(tmp_path):
    spec = models.cnn_f32_spec(2, "cnn_small")
    hxx, _, res = gen(spec, tmp_path)
    code = open(hxx).read()
    assert code.count("sofie_hip_conv2d_f32(") == 3 and code.count("SOFIE_ACT_RELU") == 4
    assert "sofie_hip_relu_f32" not in code
    assert "tensor_f = reinterpret_cast<float*>(tensor_r3);" in code
    assert "tensor_r1 = reinterpret_cast<float*>(tensor_c1);" in code
    # liveness-based reuse: the pool is smaller than the sum of all intermediates
    sizes = {"c1": 2 * 32 * 40 * 40, "p1": 2 * 32 * 20 * 20, "c2": 2 * 64 * 20 * 20, "p2": 2 * 64 * 10 * 10,
             "c3": 2 * 128 * 10 * 10, "g1": 2 * 256, "y": 2 * 5}
    pool = int(re.search(r"intermediate pool (\d+) bytes", res.stdout).group(1))
    assert pool < 4 * sum(sizes.values())
    assert pool >= 4 * (sizes["c1"] + sizes["p1"])      # producer and consumer are live together


def test_pool_offsets_never_overlap_while_both_tensors_are_live(tmp_path):
    spec, _ = models.mlp_spec("mlp_plan")
    hxx, _, _ = gen(spec, tmp_path, layer_per_call=True)     # one call per Gemm: the tensors between the layers exist
    code = open(hxx).read()
    off = {m.group(1): int(m.group(2)) for m in re.finditer(r"tensor_(\w+) = reinterpret_cast<float\*>\(fIntermediateMemoryPool \+ (\d+)\)", code)}
    size = {"h0": 256 * 128 * 4, "h1": 256 * 64 * 4, "y": 256 * 8 * 4}
    assert set(off) == set(size)
    for a, b in (("h0", "h1"), ("h1", "y")):            # producer/consumer pairs
        assert off[a] + size[a] <= off[b] or off[b] + size[b] <= off[a]
    assert all(v % 256 == 0 for v in off.values())


def test_conv_default_pads_follow_the_reference(tmp_path):
    """auto_pad NOTSET and no pads attribute means 1 on every side (ROperator_Conv.hxx:136-139);
    SAME_LOWER with stride 2 on 5x5 gives the 3x3 output of the reference's fixture."""
    s = emit.ModelSpec("pads")
    s.add_input("x", "FLOAT", (1, 1, 5, 5))
    s.add_init("W", np.ones((1, 1, 3, 3), np.float32))
    s.conv("x", "W", None, "y", kernel=(3, 3))
    s.set_output("y")
    hxx, _, _ = gen(s, tmp_path)
    assert re.search(r"sofie_hip_conv2d_f32\(fCtx, tensor_x, tensor_W, nullptr, tensor_y, 1, 1, 5, 5, 1, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1,", open(hxx).read())
    spec, _ = models.fixture_spec("ConvWithAutopadSameLower")
    hxx, _, res = gen(spec, tmp_path)
    code = open(hxx).read()
    assert "std::vector<float> ret(9);" in code
    assert re.search(r"3, 3, 1, 1, 1, 1, 2, 2, 1, 1, 1, SOFIE_ACT_NONE", code)


@pytest.mark.parametrize("auto,kernel,stride,size,want_pads,want_out", [
    ("SAME_UPPER", 3, 1, 8, (1, 1, 1, 1), 8),      # odd kernel, stride 1: one on every side, the output keeps the size
    ("SAME_LOWER", 3, 1, 8, (1, 1, 1, 1), 8),
    ("SAME_UPPER", 4, 1, 8, (1, 1, 2, 2), 8),      # even kernel: the odd unit at the end ...
    ("SAME_LOWER", 4, 1, 8, (2, 2, 1, 1), 8),      # ... or at the begin
    ("SAME_UPPER", 3, 2, 8, (0, 0, 1, 1), 4),      # stride 2 on an even size needs one cell only
    ("SAME_LOWER", 3, 2, 8, (1, 1, 0, 0), 4),
    ("SAME_UPPER", 5, 3, 8, (1, 1, 2, 2), 3),
])
def test_conv_auto_pad_same_declares_the_output_the_kernel_writes(tmp_path, auto, kernel, stride, size, want_pads, want_out):
    """SAME_UPPER / SAME_LOWER: the declared output is ceil(in / stride) per axis and the emitted call carries the
    four pads that produce exactly that many windows (the library derives its output size from the same four
    numbers, so the Session's return vector and the kernel's stores agree)."""
    s = emit.ModelSpec("same")
    s.add_input("x", "FLOAT", (1, 1, size, size))
    s.add_init("W", np.ones((4, 1, kernel, kernel), np.float32))
    s.conv("x", "W", None, "y", kernel=(kernel, kernel), strides=(stride, stride), auto_pad=auto)
    s.set_output("y")
    hxx, _, _ = gen(s, tmp_path)
    code = open(hxx).read()
    assert "std::vector<float> ret(%d);" % (4 * want_out * want_out) in code
    call = "tensor_y, 1, 1, %d, %d, 4, %d, %d, %d, %d, %d, %d, %d, %d, 1, 1, 1, SOFIE_ACT_NONE" % (
        (size, size, kernel, kernel) + want_pads + (stride, stride))
    assert call in code
    pt, pl, pb, pr = want_pads
    assert (size + pt + pb - kernel) // stride + 1 == want_out


def test_conv_begin_and_end_pads_that_differ_are_kept(tmp_path):
    """pads = (0, 2, 1, 0): all four reach the library (the reference averages them while declaring the output by
    their sum); the declared output follows the sum, as the library's does."""
    s = emit.ModelSpec("asym")
    s.add_input("x", "FLOAT", (2, 3, 7, 6))
    s.add_init("W", np.ones((5, 3, 3, 2), np.float32))
    s.conv("x", "W", None, "y", kernel=(3, 2), pads=(0, 2, 1, 0))
    s.set_output("y")
    hxx, _, _ = gen(s, tmp_path)
    code = open(hxx).read()
    assert "tensor_y, 2, 3, 7, 6, 5, 3, 2, 0, 2, 1, 0, 1, 1, 1, 1, 1, SOFIE_ACT_NONE" in code
    assert "std::vector<float> ret(%d);" % (2 * 5 * 6 * 7) in code
    assert "average padding" not in code


def test_quantized_operators_fold_scales_and_zero_points(tmp_path):
    spec = models.qcnn_spec(oracle, 2, "qcnn_small")
    hxx, dat, _ = gen(spec, tmp_path)
    code = open(hxx).read()
    # conv1 and conv2 absorb their MaxPool; the unpooled tensors no longer exist. conv2 (with its pooling) and conv3 are
    # the two layers of one chain call, whose descriptors carry what the two separate calls would
    assert code.count("sofie_hip_qconv2d_s8_chain(fCtx, tensor_p1, SOFIE_LAYOUT_NHWC, 2, 2, layers)") == 1
    assert "sofie_hip_qconv2d_pool_s8(" not in code and "sofie_hip_qconv2d_s8(" not in code
    assert ("{tensor_w2_ohwi, SOFIE_LAYOUT_NHWC, tensor_c2_qbias, tensor_c2_qscale, tensor_p2, SOFIE_LAYOUT_NHWC, 32, 20, 20, 64, 3, 3, "
            "1, 1, 1, 1, 1, 1, 1, -128, -128, SOFIE_ACT_RELU, 2, 2, 2, 2}") in code
    assert ("{tensor_w3_ohwi, SOFIE_LAYOUT_NHWC, tensor_c3_qbias, tensor_c3_qscale, tensor_c3, SOFIE_LAYOUT_NHWC, 64, 10, 10, 128, 3, 3, "
            "1, 1, 1, 1, 1, 1, 1, -128, -128, SOFIE_ACT_RELU, 0, 0, 0, 0}") in code
    assert code.count("sofie_hip_quantize_qconv2d_s8(") == 1
    assert "sofie_hip_maxpool2d_s8" not in code and "tensor_c1" not in code.replace("tensor_c1_q", "") and "tensor_r2" not in code
    # the two fully connected layers are one call (the second one has five columns); one call each with kLayerPerCall
    assert code.count("sofie_hip_qgemm_s8_pair(") == 1 and code.count("sofie_hip_qgemm_s8(") == 0
    assert re.search(r"sofie_hip_qgemm_s8_pair\(fCtx, 2, 12800, tensor_f, 12800, 256, tensor_fc1_nk_cl, 12800, tensor_g1_qscale, "
                     r"tensor_g1_qbias, -128, SOFIE_ACT_RELU, tensor_g1, 256, 5, tensor_fc2_nk, 256, tensor_y_qscale, tensor_y_qbias, 0, "
                     r"SOFIE_ACT_NONE, tensor_y, 5, SOFIE_OUT_F32\)", code)
    code_lpc = open(gen(spec, tmp_path, layer_per_call=True)[0]).read()
    assert code_lpc.count("sofie_hip_qgemm_s8(") == 2 and "sofie_hip_qgemm_s8_pair(" not in code_lpc
    assert code_lpc.count("sofie_hip_qconv2d_pool_s8(") == 1 and code_lpc.count("sofie_hip_qconv2d_s8(") == 1 and "_chain(" not in code_lpc
    # the chain's input and both of its outputs are alive together: none of them shares arena bytes with another
    offs = {m.group(1): int(m.group(2)) for m in re.finditer(r"tensor_(p1|p2|c3) = reinterpret_cast<int8_t\*>\(fIntermediateMemoryPool \+ (\d+)\)", code)}
    sizes = {"p1": 2 * 400 * 32, "p2": 2 * 100 * 64, "c3": 2 * 100 * 128}
    spans = sorted((offs[k], offs[k] + sizes[k]) for k in ("p1", "p2", "c3"))
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    assert "int8_t * tensor_fc1_nk_cl" in code and "tensor_fc1 =" not in code   # transposed once, original dropped
    assert "tensor_w2_ohwi, SOFIE_LAYOUT_NHWC" in code and "tensor_w2 =" not in code
    # conv1 reads the one-channel quantized input as it is, everything after it is channels-last
    # the first layer also absorbs the QuantizeLinear in front of it: it reads the float input
    assert "sofie_hip_quantize_f32_s8" not in code and "tensor_xq" not in code
    assert "sofie_hip_quantize_qconv2d_s8(fCtx, tensor_x, static_cast<float>(0.00392156886), -128, tensor_w1_ohwi" in code
    assert "tensor_p1, SOFIE_LAYOUT_NHWC, 2, 1, 40, 40, 32, 3, 3, 1, 1, 1, 1, 1, 1, 1, -128, SOFIE_ACT_RELU, 2, 2, 2, 2)" in code
    assert "SOFIE_OUT_F32" in code and "std::vector<float> infer(float* tensor_x)" in code
    q = models.qcnn_params(oracle)
    text = open(dat).read().split("\n")
    rec = {text[i].split()[0]: text[i + 1] for i in range(0, len(text) - 1, 2)}
    scale = np.array(rec["tensor_c1_qscale"].split(), np.float64).astype(np.float32)
    want = ((np.float32(q["sx"]) * q["s_w1"]).astype(np.float32) / np.float32(q["s_a1"])).astype(np.float32)
    assert np.array_equal(scale, want)
    qb = np.array(rec["tensor_c1_qbias"].split(), np.int64)
    assert np.array_equal(qb, q["b1"].astype(np.int64) + 128 * q["w1"].astype(np.int64).reshape(32, -1).sum(axis=1))
    # fc1 consumes the flattened channels-last conv3 output: rows reordered from (c,h,w) to (h,w,c)
    fc1 = np.array(rec["tensor_fc1_nk_cl"].split(), np.int64).reshape(256, 12800)
    want_fc1 = q["fc1"].T.reshape(256, 128, 100).transpose(0, 2, 1).reshape(256, 12800)
    assert np.array_equal(fc1, want_fc1)
    w2 = np.array(rec["tensor_w2_ohwi"].split(), np.int64).reshape(64, 3, 3, 32)
    assert np.array_equal(w2, q["w2"].transpose(0, 2, 3, 1))


def emit_error(spec, tmp_path):
    _, _, res = spec.generate(str(tmp_path), check=False)
    assert res.returncode != 0
    return res.stderr


def test_error_messages_follow_the_reference(tmp_path):
    s = emit.ModelSpec("e1")
    s.add_input("x", "FLOAT", (2, 3))
    s.add_init("W", np.ones((3, 4), np.float32))
    s.gemm("x", "W", None, "y", beta=1.0)
    s.set_output("y")
    assert "Bias tensor is not present but beta value in Gemm is not zero" in emit_error(s, tmp_path)

    s = emit.ModelSpec("e2")
    s.add_input("x", "FLOAT", (2, 3))
    s.gemm("x", "nope", None, "y", beta=0.0)
    s.set_output("y")
    assert "TMVA SOFIE Gemm Op Input Tensor x or nope is not found in model" in emit_error(s, tmp_path)

    s = emit.ModelSpec("e3")
    s.add_input("x", "FLOAT", (1, 2, 5, 5))
    s.add_init("W", np.ones((4, 2, 3, 3), np.float32))
    s.add_init("B", np.ones(3, np.float32))
    s.conv("x", "W", "B", "y", (3, 3), (1, 1, 1, 1))
    s.set_output("y")
    assert "TMVA SOFIE Conv op: Bias Tensor has wrong shape" in emit_error(s, tmp_path)

    s = emit.ModelSpec("e4")
    s.add_input("x", "FLOAT", (2, 3))
    s.add_init("W", np.ones((5, 4), np.float32))
    s.gemm("x", "W", None, "y", beta=0.0)
    s.set_output("y")
    assert "has invalid shape" in emit_error(s, tmp_path)


def test_no_weight_file_option_embeds_literals(tmp_path):
    s = emit.ModelSpec("lit")
    s.add_input("x", "FLOAT", (1, 2))
    s.add_init("W", np.array([[1.5, -2.0], [0.25, 3.0]], np.float32))
    s.gemm("x", "W", None, "y", beta=0.0)
    s.set_output("y")
    hxx, dat, _ = gen(s, tmp_path, no_weight_file=True)
    code = open(hxx).read()
    assert "static const float host[4] = {1.5f, -2.f, 0.25f, 3.f};" in code
    assert not os.path.exists(dat)
    # the generated header compiles against the C ABI
    exe = s.compile_runner(str(tmp_path))
    assert os.path.exists(exe)


def _onnx_emit(path, outdir):
    exe = os.path.join(emit.GEN_DIR, "emit_from_onnx")
    return subprocess.run([exe, path, str(outdir)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)


def _body(path):
    return [line for line in open(path).read().split("\n") if not line.startswith("//Code generated")]


@pytest.mark.parametrize("name", models.FIXTURES)
def test_cpp_onnx_front_end_on_reference_fixtures(name, tmp_path):
    """RModelParser_ONNX::Parse -> Generate on the reference's own .onnx files gives the same Session code and the
    same weight file as the description-driven route the GPU tests run (so those results hold for it too)."""
    res = _onnx_emit(os.path.join(models.GOLD, "onnx", name + ".onnx"), tmp_path)
    assert res.returncode == 0, res.stderr
    spec, _ = models.fixture_spec(name)
    sub = tmp_path / "spec"
    sub.mkdir()
    hxx, dat, _ = spec.generate(str(sub))
    assert _body(str(tmp_path / (name + ".hxx"))) == _body(hxx)
    assert open(str(tmp_path / (name + ".dat"))).read() == open(dat).read()


def test_cpp_onnx_front_end_quantized_graph_and_fusions(tmp_path):
    """A hand-written ONNX file with int8 / int32 initializers (QuantizeLinear -> QLinearConv -> DequantizeLinear,
    which the reference's parser rejects) and a MatMul -> Add -> Relu chain: same code as the description route,
    MatMul + Add becomes one Gemm call."""
    import onnx_write as ow
    p = models.qdq_conv_params()
    init = {"sx": np.array(p["sx"], np.float32), "zx": np.array(p["zx"], np.int8), "sy": np.array(p["sy"], np.float32),
            "zy": np.array(p["zy"], np.int8), "w": p["w"], "sw": p["sw"], "b": p["b"]}
    nodes = [ow.node("QuantizeLinear", ["x", "sx", "zx"], ["xq"]),
             ow.node("QLinearConv", ["xq", "sx", "zx", "w", "sw", "", "sy", "zy", "b"], ["c"], kernel_shape=[3, 3],
                     pads=[1, 1, 1, 1], strides=[1, 1]),
             ow.node("DequantizeLinear", ["c", "sy", "zy"], ["y"])]
    path = tmp_path / "qdq_conv.onnx"
    path.write_bytes(ow.model(nodes, init, [("x", 1, p["x"].shape)], [("y", 1, (2, 64, 9, 7))]))
    res = _onnx_emit(str(path), tmp_path)
    assert res.returncode == 0, res.stderr
    sub = tmp_path / "spec"
    sub.mkdir()
    hxx, dat, _ = models.qdq_conv_spec().generate(str(sub))
    assert _body(str(tmp_path / "qdq_conv.hxx")) == _body(hxx)
    assert open(str(tmp_path / "qdq_conv.dat")).read() == open(dat).read()

    r = np.random.default_rng(5)
    init = {"W": r.standard_normal((6, 4)).astype(np.float32), "B": r.standard_normal(4).astype(np.float32)}
    nodes = [ow.node("MatMul", ["x", "W"], ["m"]), ow.node("Add", ["m", "B"], ["a"]), ow.node("Relu", ["a"], ["y"])]
    path = tmp_path / "mm_add.onnx"
    path.write_bytes(ow.model(nodes, init, [("x", 1, (3, 6))], [("y", 1, (3, 4))]))
    res = _onnx_emit(str(path), tmp_path)
    assert res.returncode == 0, res.stderr
    code = open(str(tmp_path / "mm_add.hxx")).read()
    assert code.count("sofie_hip_gemm_f32(") == 1 and "tensor_B, 1, tensor_a, 4, SOFIE_ACT_RELU" in code

    # an operator outside the path is reported the way the reference words it
    path = tmp_path / "bad.onnx"
    path.write_bytes(ow.model([ow.node("Softmax", ["x"], ["y"])], {}, [("x", 1, (3, 6))], [("y", 1, (3, 6))]))
    res = _onnx_emit(str(path), tmp_path)
    assert res.returncode != 0 and "Operator type Softmax is not yet supported" in res.stderr


def test_cpp_onnx_front_end_fuses_qdq_groups(tmp_path):
    """The same layer written in the QDQ format (DequantizeLinear -> Conv -> QuantizeLinear around float operators,
    int8 weights and int32 bias behind their own DequantizeLinear) parses into the code of the QLinearConv form;
    a DequantizeLinear -> Gemm(transB) -> Relu -> QuantizeLinear group with a float bias becomes one int8 GEMM call
    whose bias is quantized with x_scale * w_scale[n]."""
    import onnx_write as ow
    p = models.qdq_conv_params()
    init = {"sx": np.array(p["sx"], np.float32), "zx": np.array(p["zx"], np.int8), "sy": np.array(p["sy"], np.float32),
            "zy": np.array(p["zy"], np.int8), "w": p["w"], "sw": p["sw"], "b": p["b"],
            "sb": (p["sx"] * p["sw"]).astype(np.float32), "zw": np.zeros(64, np.int8)}
    nodes = [ow.node("QuantizeLinear", ["x", "sx", "zx"], ["xq"]),
             ow.node("DequantizeLinear", ["xq", "sx", "zx"], ["xf"]),
             ow.node("DequantizeLinear", ["w", "sw"], ["wf"], axis=0),
             ow.node("DequantizeLinear", ["b", "sb"], ["bf"], axis=0),
             ow.node("Conv", ["xf", "wf", "bf"], ["cf"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1]),
             ow.node("QuantizeLinear", ["cf", "sy", "zy"], ["c"]),
             ow.node("DequantizeLinear", ["c", "sy", "zy"], ["y"])]
    path = tmp_path / "qdq_conv.onnx"
    path.write_bytes(ow.model(nodes, init, [("x", 1, p["x"].shape)], [("y", 1, (2, 64, 9, 7))]))
    res = _onnx_emit(str(path), tmp_path)
    assert res.returncode == 0, res.stderr
    sub = tmp_path / "spec"
    sub.mkdir()
    hxx, dat, _ = models.qdq_conv_spec().generate(str(sub))
    assert _body(str(tmp_path / "qdq_conv.hxx")) == _body(hxx)
    assert open(str(tmp_path / "qdq_conv.dat")).read() == open(dat).read()

    r = np.random.default_rng(11)
    M, K, N = 4, 32, 16
    w = r.integers(-127, 128, (N, K)).astype(np.int8)
    sw = r.uniform(0.01, 0.02, N).astype(np.float32)
    sa = np.float32(0.05)
    bf = r.uniform(-3, 3, N).astype(np.float32)
    init = {"sa": np.array(sa, np.float32), "za": np.array(-5, np.int8), "w": w, "sw": sw, "bf": bf,
            "sy": np.array(0.1, np.float32), "zy": np.array(-128, np.int8)}
    nodes = [ow.node("DequantizeLinear", ["a", "sa", "za"], ["af"]),
             ow.node("DequantizeLinear", ["w", "sw"], ["wf"], axis=0),
             ow.node("Gemm", ["af", "wf", "bf"], ["g"], transB=1),
             ow.node("Relu", ["g"], ["r"]),
             ow.node("QuantizeLinear", ["r", "sy", "zy"], ["y"])]
    path = tmp_path / "qdq_fc.onnx"
    path.write_bytes(ow.model(nodes, init, [("a", 3, (M, K))], [("y", 3, (M, N))]))
    res = _onnx_emit(str(path), tmp_path)
    assert res.returncode == 0, res.stderr
    code = open(str(tmp_path / "qdq_fc.hxx")).read()
    assert code.count("sofie_hip_qgemm_s8(") == 1 and "SOFIE_ACT_RELU" in code
    assert "dequantize" not in code and "sofie_hip_gemm_f32" not in code
    dat = open(str(tmp_path / "qdq_fc.dat")).read().split("\n")
    # the folded bias: rne(bf / (sa * sw)) - za * sum_k w[n, k]
    sb = (sa * sw).astype(np.float32)
    want = np.rint(bf.astype(np.float64) / sb.astype(np.float64)).astype(np.int64) + 5 * w.astype(np.int64).sum(axis=1)
    line = [i for i, l in enumerate(dat) if l.startswith("tensor_y_qbias ")][0]
    got = np.array(dat[line + 1].split(), dtype=np.int64)
    assert np.array_equal(got, want)

    # a per-channel scale along the wrong axis is not a QDQ group: the float operators stay
    nodes[1] = ow.node("DequantizeLinear", ["w", "sw"], ["wf"], axis=1)
    path = tmp_path / "qdq_bad_axis.onnx"
    path.write_bytes(ow.model(nodes, init, [("a", 3, (M, K))], [("y", 3, (M, N))]))
    res = _onnx_emit(str(path), tmp_path)
    assert res.returncode != 0 or "sofie_hip_qgemm_s8(" not in open(str(tmp_path / "qdq_bad_axis.hxx")).read()


def test_batchnorm_folds_into_conv_or_runs_alone(tmp_path):
    """Conv -> BatchNormalization -> Relu becomes one convolution call whose weights and bias carry the
    normalisation (W * s, (b - mean) * s + beta with s = gamma / sqrt(var + eps)); a BatchNormalization that does not
    follow a convolution is one call of its own kernel with the folded per-channel scale; the tensors only the
    absorbed operator read are not written to the weight file."""
    spec = models.convbn_spec("convbn_t")
    hxx, dat, _ = spec.generate(str(tmp_path))
    code = open(hxx).read()
    assert code.count("sofie_hip_conv2d_f32(") == 1 and code.count("sofie_hip_batchnorm_f32(") == 1
    assert "tensor_n1_bnw, tensor_n1_bnb, tensor_n1, " in code and "SOFIE_ACT_RELU), \"Conv" in code
    assert code.count("sofie_hip_conv_transpose2d_f32(") == 1 and code.count("sofie_hip_relu_f32(") == 0
    lines = open(dat).read().split("\n")
    names = [l.split()[0] for l in lines if l.startswith("tensor_")]
    for gone in ("tensor_w1", "tensor_b1", "tensor_g1", "tensor_var1", "tensor_mean1", "tensor_beta1", "tensor_g2", "tensor_var2"):
        assert gone not in names
    for kept in ("tensor_n1_bnw", "tensor_n1_bnb", "tensor_n2_bnscale", "tensor_mean2", "tensor_beta2", "tensor_wt"):
        assert kept in names
    p = models.convbn_params()
    s1 = p["g1"] * (1.0 / np.sqrt((p["var1"] + np.float32(1e-5)).astype(np.float64))).astype(np.float32)
    got_w = np.array(lines[[i for i, l in enumerate(lines) if l.startswith("tensor_n1_bnw ")][0] + 1].split(), np.float32)
    got_b = np.array(lines[[i for i, l in enumerate(lines) if l.startswith("tensor_n1_bnb ")][0] + 1].split(), np.float32)
    assert np.array_equal(got_w, (p["w1"] * s1[:, None, None, None]).reshape(-1))
    assert np.array_equal(got_b, (p["b1"] - p["mean1"]) * s1 + p["beta1"])


def test_parametric_batch_dimension_is_fixed_at_generation_time(tmp_path):
    """An input whose first dimension is the parameter "bs" (or a -1) is given its value through the batch size
    argument of Generate, as with the reference; without a value the device emission refuses, in words that say
    what to do."""
    import onnx_write as ow
    r = np.random.default_rng(3)
    init = {"W": r.standard_normal((6, 4)).astype(np.float32), "B": r.standard_normal(4).astype(np.float32)}
    nodes = [ow.node("Gemm", ["x", "W", "B"], ["g"]), ow.node("Relu", ["g"], ["y"])]
    for first in ("bs", -1):
        path = tmp_path / "dyn.onnx"
        path.write_bytes(ow.model(nodes, init, [("x", 1, (first, 6))], [("y", 1, (first, 4))]))
        exe = os.path.join(emit.GEN_DIR, "emit_from_onnx")
        res = subprocess.run([exe, str(path), str(tmp_path), "--batch", "7"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        assert res.returncode == 0, res.stderr
        code = open(str(tmp_path / "dyn.hxx")).read()
        assert "sofie_hip_gemm_f32(fCtx, 0, 0, 7, 4, 6," in code
        res = _onnx_emit(str(path), tmp_path)
        assert res.returncode != 0 and "parametric shape" in res.stderr and "pass the batch size" in res.stderr
        # the same file with the value as a capacity: the Gemm -> Relu pair prints the Session's batch member
        res = subprocess.run([exe, str(path), str(tmp_path), "--batch", "7", "--runtime"], stdout=subprocess.PIPE,
                             stderr=subprocess.PIPE, text=True)
        assert res.returncode == 0, res.stderr
        code = open(str(tmp_path / "dyn.hxx")).read()
        assert "sofie_hip_gemm_f32(fCtx, 0, 0, fBatch, 4, 6," in code and "size_t fBatch = 7;" in code


def test_stacked_matmul_shapes_and_offsets(tmp_path):
    """Leading dimensions broadcast as in numpy.matmul; one launch per stacked operator, with the element strides of A
    and B along every leading dimension (0 where the operand is broadcast)."""
    hxx, _, _ = models.stacked_spec("stacked_t").generate(str(tmp_path))
    code = open(hxx).read()
    # x [2,1,4,5] @ B1 [3,5,6]: leading dimensions (2, 3); A advances with the first only, B with the second only
    assert "_lead[] = {2, 3};" in code and "_sa[] = {20, 0};" in code and "_sb[] = {0, 30};" in code
    # h [2,3,4,6] @ B2 [6,2]: B is one matrix
    assert "_sa[] = {72, 24};" in code and "_sb[] = {0, 0};" in code
    assert code.count("sofie_hip_gemm_f32_stacked(") == 2 and "sofie_hip_gemm_f32(" not in code
    assert "tensor_x, 5, tensor_B1, 6, tensor_h, 6, 2, " in code
    bad = emit.ModelSpec("bad_stack")
    bad.add_input("x", "FLOAT", (2, 4, 5))
    bad.add_init("B", np.zeros((3, 5, 6), np.float32))
    bad.gemm("x", "B", None, "y", 1.0, 0.0)
    bad.set_output("y")
    with pytest.raises(RuntimeError, match="invalid input shapes 2 and 3"):
        bad.generate(str(tmp_path))


def _einsum_spec(name, equation, shapes):
    s = emit.ModelSpec(name)
    xs = ["x%d" % i for i in range(len(shapes))]
    for n, shape in zip(xs, shapes):
        s.add_input(n, "FLOAT", shape)
    s.einsum(equation, xs, "y")
    s.set_output("y")
    return s


def test_einsum_matrix_products_become_gemm_calls_everything_else_one_kernel_call(tmp_path):
    """The reference's four cases of a matrix product (ROperator_Einsum.hxx:181-197) map to transA / transB of
    one Gemm call per stacked matrix; an equation whose free labels come out in another order, which the reference
    would hand to sgemm_ all the same, takes the general kernel."""
    def code(name, eq, shapes):
        return open(_einsum_spec(name, eq, shapes).generate(str(tmp_path))[0]).read()
    c = code("es_nn", "ik,kj->ij", [(4, 5), (5, 6)])
    assert "sofie_hip_gemm_f32(fCtx, 0, 0, 4, 6, 5, 1.0f, tensor_x0, 5, tensor_x1, 6," in c
    c = code("es_tn", "ki,kj->ij", [(5, 4), (5, 6)])
    assert "sofie_hip_gemm_f32(fCtx, 1, 0, 4, 6, 5, 1.0f, tensor_x0, 4, tensor_x1, 6," in c
    c = code("es_nt", "bik,bjk->bij", [(3, 4, 5), (3, 6, 5)])
    assert "sofie_hip_gemm_f32(fCtx, 0, 1, 4, 6, 5," in c and "_a[] = {0, 20, 40};" in c and "_b[] = {0, 30, 60};" in c
    c = code("es_tt", "ki,jk->ij", [(5, 4), (6, 5)])
    assert "sofie_hip_gemm_f32(fCtx, 1, 1, 4, 6, 5, 1.0f, tensor_x0, 4, tensor_x1, 5," in c
    # a stacked label that only one operand carries: the other operand's matrix repeats
    c = code("es_bc", "abik,bkj->abij", [(2, 3, 4, 5), (3, 5, 6)])
    assert "_a[] = {0, 20, 40, 60, 80, 100};" in c and "_b[] = {0, 30, 60, 0, 30, 60};" in c
    # free labels swapped in the output: not a row-major product of these operands
    c = code("es_sw", "ik,kj->ji", [(4, 5), (5, 6)])
    assert "sofie_hip_gemm_f32" not in c
    assert "_extent[] = {6, 4, 5};" in c and "_stride[] = {0, 5, 1, 1, 0, 6};" in c
    assert "sofie_hip_einsum_f32(fCtx, 2, op_0_x, 3, 2, op_0_extent, op_0_stride, tensor_y)" in c
    # two summed labels run in the order of their characters; a scalar result has no output label
    c = code("es_2", "abc,abd->ad", [(2, 2, 3), (2, 2, 3)])
    assert "_extent[] = {2, 3, 2, 3};" in c and "_stride[] = {6, 0, 3, 1, 6, 1, 3, 0};" in c
    c = code("es_dot", "i,i->", [(7,), (7,)])
    assert "sofie_hip_einsum_f32(fCtx, 2, op_0_x, 1, 0," in c and "std::vector<float> ret(1);" in c
    # a repeated label walks the diagonal: its strides add up
    c = code("es_diag", "ii->i", [(5, 5)])
    assert "_stride[] = {6};" in c


def test_runtime_batch_session(tmp_path):
    """Options::kRuntimeBatch: the batch given to Generate is a capacity (buffers and the arena are sized for it); every
    operator prints the Session's fBatch member where it would print the leading dimension, and infer(n, ...) moves
    n rows in and out."""
    hxx, _, _ = models.cnn_f32_rt_spec("rt_t").generate(str(tmp_path))
    c = open(hxx).read()
    assert "size_t fBatch = 8;" in c
    assert "sofie_hip_conv2d_f32(fCtx, tensor_x, tensor_w1, tensor_b1, tensor_c1, fBatch, 1, 40, 40, 32, 3, 3," in c
    assert "sofie_hip_maxpool2d_f32(fCtx, tensor_r1, tensor_p1, (fBatch * 32), 40, 40," in c
    assert "sofie_hip_gemm_f32(fCtx, 0, 0, fBatch, 256, 12800," in c
    assert "std::vector<float> infer(size_t batch, float* tensor_x){" in c
    assert "sofie_hip_upload(fCtx, fInput_x, tensor_x, fBatch * 6400)" in c and "std::vector<float> ret(fBatch * 5);" in c
    assert "std::vector<float> infer(float* tensor_x){ return infer(8, tensor_x); }" in c
    assert "the batch must be between 1 and 8" in c
    # the arena is the one of the fixed batch of 8
    fixed = open(models.cnn_f32_spec(8, "rt_f").generate(str(tmp_path))[0]).read()
    pool = re.search(r"fIntermediateMemoryPool\), (\d+)\)", c).group(1)
    assert pool == re.search(r"fIntermediateMemoryPool\), (\d+)\)", fixed).group(1)
    assert "fBatch" not in fixed

    # without a shape parameter there is no batch to vary; without a capacity there is nothing to size
    s, _ = models.mlp_spec("rt_e1")
    s.runtime_batch = True
    s.batch = 4
    assert "needs an input whose leading dimension is a parameter" in emit_error(s, tmp_path)
    s = models.cnn_f32_spec("bs", "rt_e2")
    s.runtime_batch = True
    assert "needs the largest batch" in emit_error(s, tmp_path)
    # an operator that cannot tell which of its dimensions is the batch refuses
    s = emit.ModelSpec("rt_e3")
    s.add_input("a", "FLOAT", ("bs", 4))
    s.add_init("b", np.ones((4, 3), np.float32))
    s.einsum("ik,kj->ij", ["a", "b"], "y")
    s.set_output("y")
    s.batch, s.runtime_batch = 6, True
    assert "this Einsum operator cannot run on fewer rows" in emit_error(s, tmp_path)
    # the same parameter resolved at generation time only: a plain Session for that batch
    s = emit.ModelSpec("rt_fix")
    s.add_input("a", "FLOAT", ("bs", 4))
    s.add_init("b", np.ones((4, 3), np.float32))
    s.gemm("a", "b", None, "y", 1.0, 0.0)
    s.set_output("y")
    s.batch = 6
    c = open(s.generate(str(tmp_path))[0]).read()
    assert "sofie_hip_gemm_f32(fCtx, 0, 0, 6, 3, 4," in c and "fBatch" not in c


def test_two_shape_parameters_get_their_values_by_name(tmp_path):
    """An input with two named dimensions ([bs, seq, 8]): RModel::Initialize(map) gives each its value, as in the
    reference (RModel.cxx:408-463); a MatMul of rank 3 against a [8, 4] matrix then has its sizes at generation time.
    A parameter left without a value is an error that names the tensor."""
    def spec(name):
        s = emit.ModelSpec(name)
        s.add_input("x", "FLOAT", ("bs", "seq", 8))
        s.add_init("w", np.arange(32, dtype=np.float32).reshape(8, 4))
        s.gemm("x", "w", None, "y", beta=0.0)
        s.set_output("y")
        return s
    c = open(spec("two_params").generate(str(tmp_path), params={"bs": 3, "seq": 5})[0]).read()
    assert "std::vector<float> ret(60);" in c            # 3 * 5 * 4
    c = open(spec("two_params_b").generate(str(tmp_path), batch=2, params={"seq": 7})[0]).read()
    assert "std::vector<float> ret(56);" in c            # the batch number answers for "bs"
    with pytest.raises(RuntimeError, match="parametric shape"):
        spec("two_params_c").generate(str(tmp_path), batch=2)


def test_session_promises_constant_weights(tmp_path):
    """A Session's weights are uploaded in its constructor and never written again: it tells the library so, right
    behind the creation of the context, and the library keeps its own layouts of them."""
    c = open(models.conv1d_spec("cw_t").generate(str(tmp_path))[0]).read()
    create = c.index("sofie_hip_create(&fCtx.p, device, nullptr)")
    promise = c.index("Check(sofie_hip_constant_weights(fCtx, 1), \"Session construction\");")
    upload = c.index("sofie_hip_upload(fCtx, tensor_w")
    assert create < promise < upload


def test_pool_1d_and_3d_emission(tmp_path):
    """Pooling over one spatial axis (ROperator_Pool.hxx:329-370) is emitted as the two-axis call on a plane of height
    one; over three axes (:417-470) as the calls that take the geometry as arrays, pads in ONNX order."""
    c = open(models.pool1d_spec("p1d_t").generate(str(tmp_path))[0]).read()
    # [3,4,50] -> (50 + 2 - 3) / 2 + 1 = 25 -> (25 + 3 - 4) + 1 = 25
    assert "sofie_hip_maxpool2d_f32(fCtx, tensor_x, tensor_m, 12, 1, 50, 1, 3, 0, 1, 0, 1, 1, 2)" in c
    assert "sofie_hip_avgpool2d_f32(fCtx, tensor_m, tensor_y, 12, 1, 25, 1, 4, 0, 2, 0, 1, 1, 1, 0)" in c
    assert "std::vector<float> ret(300);" in c
    c = open(models.pool3d_spec("p3d_t").generate(str(tmp_path))[0]).read()
    assert "const int dims[3] = {8, 9, 10}, kernel[3] = {2, 3, 2}, pads[6] = {1, 0, 1, 0, 1, 0}, strides[3] = {2, 1, 2};" in c
    assert "sofie_hip_maxpool3d_f32(fCtx, tensor_x, tensor_m, 6, dims, kernel, pads, strides)" in c
    # (8 + 1 - 2) / 2 + 1 = 4, (9 + 1 - 3) + 1 = 8, (10 + 1 - 2) / 2 + 1 = 5
    assert "const int dims[3] = {4, 8, 5}, kernel[3] = {2, 2, 3}, pads[6] = {0, 1, 1, 1, 0, 1}, strides[3] = {1, 2, 1};" in c
    assert "sofie_hip_avgpool3d_f32(fCtx, tensor_m, tensor_y, 6, dims, kernel, pads, strides, 1)" in c
    # (4 + 1 - 2) + 1 = 4, (8 + 1 - 2) / 2 + 1 = 4, (5 + 2 - 3) + 1 = 5
    assert "std::vector<float> ret(%d);" % (2 * 3 * 4 * 4 * 5) in c
    # refused at generation time: a kernel of the wrong rank, an average over inside cells with a pad as large as the window
    s = emit.ModelSpec("p3d_bad")
    s.add_input("x", "FLOAT", (1, 1, 4, 4, 4))
    s.maxpool("x", "y", (2, 2), (0, 0, 0, 0), (1, 1))
    s.set_output("y")
    with pytest.raises(RuntimeError, match="invalid inputs"):
        s.generate(str(tmp_path))
    s = emit.ModelSpec("p1d_bad")
    s.add_input("x", "FLOAT", (1, 1, 9))
    s.avgpool("x", "y", (2,), (2, 0), (1,))
    s.set_output("y")
    with pytest.raises(RuntimeError, match="without a cell"):
        s.generate(str(tmp_path))


def test_conv_1d_and_3d_emission(tmp_path):
    """One spatial dimension runs as the 2-D call with a height of one; three as the 3-D call. Absent pads mean one
    on every side of every dimension, as in the reference (ROperator_Conv.hxx:136-139)."""
    c = open(models.conv1d_spec("c1d_t").generate(str(tmp_path))[0]).read()
    # [3,4,50], kernel 5 dilated by 2 (extent 9), pads 1+1, stride 2: (50 + 2 - 9) / 2 + 1 = 22
    assert "sofie_hip_conv2d_f32(fCtx, tensor_x, tensor_w, tensor_b, tensor_c, 3, 4, 1, 50, 6, 1, 5, 0, 1, 0, 1, 1, 2, 1, 2, 2, SOFIE_ACT_RELU)" in c
    assert "std::vector<float> ret(396);" in c
    c = open(models.conv3d_spec("c3d_t").generate(str(tmp_path))[0]).read()
    assert ("sofie_hip_conv3d_f32(fCtx, tensor_x, tensor_w, tensor_b, tensor_y, 2, 4, 6, 9, 10, 6, 3, 2, 3, 1, 0, 2, 1, 2, 1, 1, 1, 1, 2, "
            "SOFIE_ACT_NONE)") in c
    # (6 + 2 - 3) + 1 = 6, (9 - 2) / 2 + 1 = 4, (10 + 4 - 3) + 1 = 12
    assert "std::vector<float> ret(%d);" % (2 * 6 * 6 * 4 * 12) in c
    s = emit.ModelSpec("c3d_def")
    s.add_input("x", "FLOAT", (1, 1, 4, 4, 4))
    s.add_init("w", np.ones((2, 1, 3, 3, 3), np.float32))
    s.conv("x", "w", None, "y")
    s.set_output("y")
    c = open(s.generate(str(tmp_path))[0]).read()
    assert "1, 1, 4, 4, 4, 2, 3, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, SOFIE_ACT_NONE" in c
    bad = emit.ModelSpec("c_rank")
    bad.add_input("x", "FLOAT", (1, 1, 4, 4))
    bad.add_init("w", np.ones((2, 1, 3), np.float32))
    bad.conv("x", "w", None, "y")
    bad.set_output("y")
    assert "is not of 3,4 or 5 dimensions" in emit_error(bad, tmp_path)


def test_einsum_errors(tmp_path):
    assert "Error parsing the equation ik,kj" in emit_error(_einsum_spec("ee1", "ik,kj", [(2, 3), (3, 2)]), tmp_path)
    assert "Error parsing the equation" in emit_error(_einsum_spec("ee2", "ik->i", [(2, 3), (3, 2)]), tmp_path)
    assert "output label z is not present in inputs" in emit_error(_einsum_spec("ee3", "ik,kj->iz", [(2, 3), (3, 2)]), tmp_path)
    assert "label k has two sizes, 3 and 4" in emit_error(_einsum_spec("ee4", "ik,kj->ij", [(2, 3), (4, 2)]), tmp_path)
    assert "invalid label or shape" in emit_error(_einsum_spec("ee5", "ik,kj->ij", [(2, 3, 1), (3, 2)]), tmp_path)


def test_binary_weight_file_holds_the_same_tensors(tmp_path):
    """Options::kBinaryWeightFile: the .bin file carries the records of the .dat file (same names, order, lengths and
    values, typed and raw) and the generated constructor defaults to it; its reader takes either format."""
    import struct
    spec = models.qdq_conv_spec("qdq_bin")
    hxx_b, binf, _ = spec.generate(str(tmp_path), binary_weight_file=True)
    sub = tmp_path / "text"
    sub.mkdir()
    hxx_t, dat, _ = models.qdq_conv_spec("qdq_bin").generate(str(sub))
    assert 'Session(std::string filename ="qdq_bin.bin"' in open(hxx_b).read()
    assert 'Session(std::string filename ="qdq_bin.dat"' in open(hxx_t).read()
    # apart from that default the two headers are the same code: the reader recognises the format from the file
    strip = lambda path: [l for l in _body(path) if "Session(std::string filename" not in l]
    assert strip(hxx_b) == strip(hxx_t)
    raw = open(binf, "rb").read()
    assert raw[:8] == b"SOFIEBIN" and struct.unpack_from("<II", raw, 8)[0] == 1
    count = struct.unpack_from("<II", raw, 8)[1]
    lines = open(dat).read().split("\n")
    text = {}
    for i in range(0, len(lines) - 1, 2):
        name, length = lines[i].split()
        text[name] = (int(length), lines[i + 1].split())
    assert count == len(text)
    off, np_types = 16, {1: np.float32, 3: np.int8, 6: np.int32, 2: np.uint8}
    order = []
    for _ in range(count):
        (nlen,) = struct.unpack_from("<I", raw, off)
        name = raw[off + 4:off + 4 + nlen].decode()
        type_code, length = struct.unpack_from("<IQ", raw, off + 4 + nlen)
        off += 4 + nlen + 12
        dt = np.dtype(np_types[type_code])
        vals = np.frombuffer(raw, dt, length, off)
        off += length * dt.itemsize
        off += (8 - (length * dt.itemsize) % 8) % 8
        assert text[name][0] == length
        assert np.array_equal(vals, np.array(text[name][1], dtype=np.float64).astype(dt))
        order.append(name)
    assert off == len(raw) and order == [l.split()[0] for l in lines[0:-1:2]]


def test_every_prebuilt_session_compiles():
    """tests/build_generated.py output (made by build()): header, weights and runner of each network."""
    import build_generated
    for spec in build_generated.all_specs(with_large=True):
        for ext in (".hxx",):
            assert os.path.exists(os.path.join(emit.GEN_DIR, spec.name + ext)), spec.name
        assert os.path.exists(os.path.join(emit.GEN_DIR, "run_" + spec.name)), spec.name


def test_several_outputs_follow_the_reference_return_convention(tmp_path):
    """Outputs of one type come back as a vector of vectors, outputs of different types as a tuple of vectors, in
    the order of the output list (RModel.cxx:744-801); an intermediate that is an output keeps its place in the
    pool until the end; the generated code compiles against the runner."""
    spec, _ = models.two_heads_spec("two_heads_probe")
    hxx, _, _ = gen(spec, tmp_path, layer_per_call=True)   # one call per layer, so that the first hidden layer is a tensor
    code = open(hxx).read()
    assert "std::vector<std::vector<float>> infer(float* tensor_x)" in code
    assert "return std::vector<std::vector<float>>{std::move(ret_0), std::move(ret_1)};" in code
    assert "std::tuple<const float*,const float*> infer_device(const float* tensor_x)" in code
    off = {m.group(1): int(m.group(2)) for m in re.finditer(r"tensor_(\w+) = reinterpret_cast<float\*>\(fIntermediateMemoryPool \+ (\d+)\)", code)}
    assert off["y"] == off["h0"]                       # the last layer reuses the dead first hidden layer ...
    assert off["h1"] >= off["h0"] + 256 * 128 * 4       # ... and never the hidden layer that is an output
    spec.compile_runner(str(tmp_path))

    spec, _ = models.mixed_outputs_spec("mixed_probe")
    hxx, _, _ = gen(spec, tmp_path)
    code = open(hxx).read()
    assert "std::tuple<std::vector<float>,std::vector<int8_t>> infer(float* tensor_x)" in code
    assert "std::tuple<const float*,const int8_t*> infer_device(const float* tensor_x)" in code
    assert code.index("tensor_y, ret_0.size()") < code.index("tensor_q, ret_1.size()")
    spec.compile_runner(str(tmp_path))


def test_no_session_option_emits_a_free_infer_over_literal_weights(tmp_path):
    """Options::kNoSession: no weight file is written, the weights are literals and the namespace has a free
    function infer (the reference's no-session form); the runner compiles against it."""
    spec, _ = models.mlp_nosession_spec("nosession_probe")
    hxx, dat, _ = gen(spec, tmp_path)
    assert not os.path.exists(dat)
    code = open(hxx).read()
    assert "static const float host[" in code
    assert 'inline Session& DefaultSession() { static Session session(""); return session; }' in code
    assert "inline auto infer(float* tensor_x){ return DefaultSession().infer(tensor_x); }" in code
    spec.compile_runner(str(tmp_path))


def test_cpp_onnx_front_end_graph_with_two_outputs(tmp_path):
    """An ONNX graph that lists a hidden Gemm result and the final result as outputs: the parser keeps both in the
    file's order, the Gemm -> Relu pair is not fused over the tensor that is an output, and infer() returns a
    vector of two vectors."""
    import onnx_write as ow
    r = np.random.default_rng(6)
    init = {"W0": r.standard_normal((6, 4)).astype(np.float32), "B0": r.standard_normal(4).astype(np.float32),
            "W1": r.standard_normal((4, 3)).astype(np.float32), "B1": r.standard_normal(3).astype(np.float32)}
    nodes = [ow.node("Gemm", ["x", "W0", "B0"], ["h"]), ow.node("Relu", ["h"], ["hr"]),
             ow.node("Gemm", ["hr", "W1", "B1"], ["y"])]
    path = tmp_path / "two_out.onnx"
    path.write_bytes(ow.model(nodes, init, [("x", 1, (5, 6))], [("h", 1, (5, 4)), ("y", 1, (5, 3))]))
    res = _onnx_emit(str(path), tmp_path)
    assert res.returncode == 0, res.stderr
    code = open(str(tmp_path / "two_out.hxx")).read()
    assert "std::vector<std::vector<float>> infer(float* tensor_x)" in code
    assert code.index("tensor_h, ret_0.size()") < code.index("tensor_y, ret_1.size()")
    # the pre-activation tensor h is an output: its Gemm keeps no fused ReLU, the Relu runs as its own call
    first = re.search(r"sofie_hip_gemm_f32\([^;]*tensor_h, 4, (SOFIE_ACT_\w+)\)", code)
    assert first and first.group(1) == "SOFIE_ACT_NONE"
    assert "sofie_hip_relu_f32(" in code


def test_cpp_onnx_front_end_refuses_ceil_mode_pooling(tmp_path):
    """MaxPool with ceil_mode = 1 has a different output size than the floor rule the kernels implement: refused
    at generation time (as auto_pad and dilations of a pooling are), not silently computed with the floor rule."""
    import onnx_write as ow
    nodes = [ow.node("MaxPool", ["x"], ["y"], kernel_shape=[2, 2], strides=[2, 2], ceil_mode=1)]
    path = tmp_path / "ceil.onnx"
    path.write_bytes(ow.model(nodes, {}, [("x", 1, (1, 2, 5, 5))], [("y", 1, (1, 2, 3, 3))]))
    res = _onnx_emit(str(path), tmp_path)
    assert res.returncode != 0
    assert "ceil_mode is not supported" in res.stderr + res.stdout


def test_generated_weight_reader_checks_the_element_type(tmp_path):
    """Every ReadTensor call of the generated constructor names the element type it expects and the binary reader
    compares it with the record's type field."""
    spec = models.qdq_conv_spec("qdq_type")
    hxx, _, _ = spec.generate(str(tmp_path), binary_weight_file=True)
    code = open(hxx).read()
    calls = re.findall(r'ReadTensor\(f, binary, "tensor_(\w+)", (\d+), (\d+), host\.data\(\)\);', code)
    assert calls and {int(c[2]) for c in calls} <= {1, 2, 3, 6}          # FLOAT, UINT8, INT8, INT32
    assert any(int(c[2]) == 3 for c in calls) and any(int(c[2]) == 1 for c in calls)
    assert "type != expected_type" in code and "failed to read the correct tensor type" in code


def test_gemm_chain_becomes_one_call(tmp_path):
    """Gemm -> Relu -> Gemm -> Relu -> Gemm on small constant matrices: one sofie_hip_mlp_f32 call, no tensor between the
    layers, weights given [N, K] rewritten as [K, N] in the weight file; Options::kLayerPerCall keeps the three calls."""
    spec, _ = models.mlp_spec("mlp_chain")
    hxx, _, _ = gen(spec, tmp_path)
    code = open(hxx).read()
    assert code.count("sofie_hip_mlp_f32(") == 1 and "sofie_hip_gemm_f32(" not in code
    assert re.search(r"_dims\[\] = \{64, 128, 64, 8\};", code)
    assert re.search(r"_act\[\] = \{SOFIE_ACT_RELU, SOFIE_ACT_RELU, SOFIE_ACT_NONE\};", code)
    assert "tensor_h0" not in code and "tensor_h1" not in code
    hxx, _, _ = gen(spec, tmp_path, layer_per_call=True)
    code = open(hxx).read()
    assert code.count("sofie_hip_gemm_f32(") == 3 and "sofie_hip_mlp_f32(" not in code

    # a layer whose output is also a model output ends the chain; a transposed matrix read by two layers is not rewritten
    r = np.random.default_rng(0)
    s2 = emit.ModelSpec("chain_breaks")
    s2.add_input("x", "FLOAT", (4, 6))
    s2.add_init("W", r.standard_normal((6, 6)).astype(np.float32))
    s2.add_init("V", r.standard_normal((3, 6)).astype(np.float32))
    s2.gemm("x", "W", None, "a", beta=0.0, transB=True)
    s2.gemm("a", "W", None, "b", beta=0.0, transB=True)
    s2.gemm("b", "V", None, "c", beta=0.0, transB=True)
    s2.gemm("c", "V", None, "d", beta=0.0)
    s2.set_output("d")
    hxx, dat, _ = gen(s2, tmp_path)
    code = open(hxx).read()
    # W and V are transposed operands read by two layers each: rewriting them as [K, N] for one reader would break
    # the other, so every layer keeps its own call
    assert code.count("sofie_hip_gemm_f32(") == 4 and "sofie_hip_mlp_f32(" not in code
    s3 = emit.ModelSpec("chain_to_output")
    s3.add_input("x", "FLOAT", (4, 6))
    for n_, shape in (("A", (6, 5)), ("B", (5, 7)), ("C", (7, 2))):
        s3.add_init(n_, r.standard_normal(shape).astype(np.float32))
    s3.gemm("x", "A", None, "p", beta=0.0)
    s3.gemm("p", "B", None, "q", beta=0.0)
    s3.gemm("q", "C", None, "t", beta=0.0)
    s3.set_output("q")
    s3.set_output("t")
    hxx, _, _ = gen(s3, tmp_path)
    code = open(hxx).read()
    # q is a model output: the chain x -> p -> q ends there and the last layer is a call of its own
    assert code.count("sofie_hip_mlp_f32(") == 1 and code.count("sofie_hip_gemm_f32(") == 1
    assert re.search(r"_dims\[\] = \{6, 5, 7\};", code)


@pytest.mark.parametrize("host_code", [False, True])
def test_generated_sessions_compile_without_warnings(host_code, tmp_path):
    """What the emitter writes is code a user compiles into a program of their own: -Wall -Wextra -Wshadow -Werror on
    the Sessions of the benchmark's networks, the quantized models, a weightless pooling graph, ConvTranspose and
    Einsum, for the device and for the host cores."""
    specs = [models.mlp_spec()[0], models.cnn_f32_spec(8), models.qcnn_spec(oracle, 8), models.qdq_conv_spec(),
             models.convbn_spec(), models.conv3d_spec(), models.pool3d_spec(), models.cnn_f32_rt_spec()]
    specs += [models.fixture_spec(n)[0] for n in ("ConvTransposeBias2d", "Einsum_3", "Einsum_4", "AvgPool", "MaxPool1d")]
    for spec in specs:
        d = tmp_path / (spec.name + ("_host" if host_code else "_dev"))
        d.mkdir()
        hxx, _, _ = spec.generate(str(d), host_code=host_code)
        src = d / "unit.cxx"
        src.write_text('#include "%s"\nint main() { return 0; }\n' % os.path.basename(hxx))
        res = subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Wshadow", "-Werror", "-fsyntax-only", "-I" + str(d),
                              "-I" + os.path.join(emit.ROOT, "include"), "-I" + os.path.join(emit.ROOT, "sofie_amd", "host", "inc"), str(src)],
                             stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        assert res.returncode == 0, spec.name + "\n" + res.stdout
