"""Options::kHostCode: RModel::Generate emits the Session for the host cores, the way the reference does (bias
copy + BLAS::sgemm_ for Gemm, Im2col + sgemm_ + saxpy_ per image for Conv, the Relu and pooling loops; reference
src/SOFIE_core/inc/SOFIE/ROperator_Gemm.hxx:292-390, ROperator_Conv.hxx:302-522, ROperator_Pool.hxx:266-476,
ROperator_Relu.hxx:54-66). The generated code is compiled with g++ and run here, without a GPU and without the kernel
library, against the answers the reference's own tests hold for its fixtures and against the oracle."""
import json
import os
import subprocess

import numpy as np
import pytest

import models
import random_graphs
import replay
from oracle import oracle
from sofie_amd import emit

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
HOST_FIXTURES = ["Linear_16", "Linear_32", "Linear_64", "ConvWithPadding", "ConvWithoutPadding", "ConvWithAutopadSameLower",
                 "ConvWithStridesPadding", "ConvWithStridesNoPadding", "ConvWithAsymmetricPadding", "MaxPool1d", "MaxPool2d",
                 "MaxPool3d", "AvgPool", "ConvTranspose1d", "ConvTranspose2d", "ConvTransposeBias2d", "ConvTransposeBias2dBatched",
                 "Einsum_matmul", "Einsum_dotprod", "Einsum_3", "Einsum_4"]
MKL = "/opt/conda/lib/libmkl_rt.so.1"


def run_host(spec, xs, outdir, env=None, iters=0, **generate_args):
    """Generate the host Session of `spec` into outdir, compile its runner, run it on the inputs; returns the output."""
    outdir = str(outdir)
    hxx, dat, res = spec.generate(outdir, host_code=True, **generate_args)
    text = open(hxx).read()
    assert "sofie_hip" not in text   # host code only: no call into the kernel library
    exe = emit.compile_host_runner(spec.name, outdir, num_inputs=len(xs))
    names = []
    for i, a in enumerate(xs):
        names.append(os.path.join(outdir, "in%d.bin" % i))
        np.ascontiguousarray(a, np.float32).tofile(names[-1])
    fout = os.path.join(outdir, "out.bin")
    cmd = [exe, dat, ",".join(names), fout] + ([str(iters)] if iters else [])
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300,
                       env=dict(os.environ, **(env or {})))
    assert r.returncode == 0, r.stderr
    y = np.fromfile(fout, np.float32)
    return (y, json.loads(r.stdout)) if iters else y


def rel_err(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) / max(float(np.max(np.abs(b))), 1e-30))


@pytest.mark.parametrize("name", HOST_FIXTURES)
def test_reference_fixture_through_host_session(name, tmp_path):
    """The reference's fixtures through the generated host code: its expected outputs within its own tolerance, the
    oracle's replay of the graph within 1e-5."""
    entry = json.load(open(os.path.join(GOLD, "expected.json")))[name]
    spec, graph = models.fixture_spec(name)
    feeds = replay.fixture_feeds(entry, graph)
    xs = [feeds[i[0]] for i in graph["inputs"]]
    y = run_host(spec, xs, tmp_path)
    want = np.array(entry["expected"], np.float32)
    assert y.size == want.size
    assert np.max(np.abs(y - want)) <= 1e-3
    yo = replay.run_graph(graph, feeds, oracle)
    assert rel_err(y, yo.reshape(-1)) <= 1e-5


def test_mlp_and_cnn_host_sessions(tmp_path):
    """The benchmark's fp32 networks (MLP 64-128-64-8 on 256 rows; the CNN classifier on 8 images) as host code."""
    spec, x = models.mlp_spec()
    y = run_host(spec, [x], tmp_path / "mlp")
    assert rel_err(y, models.mlp_reference(oracle).reshape(-1)) <= 1e-5
    x = models.cnn_input(8)
    y = run_host(models.cnn_f32_spec(8), [x], tmp_path / "cnn")
    assert rel_err(y, models.cnn_f32_stages(oracle, x)["y"].reshape(-1)) <= 1e-5


def test_quantized_models_as_host_code_are_bit_exact(tmp_path):
    """The quantized operators have a host form as well (the reference has no quantized operators: the generated CPU
    code of an int8 model is this emission): QuantizeLinear, QLinearConv with a ReLU behind it, int8 MaxPool, Flatten,
    QLinearMatMul with int8 and with float output, DequantizeLinear of a channels-last tensor. Integer sums and one
    rounding rule: the int8 CNN's logits and the dequantised convolution equal the oracle's bit for bit."""
    x = models.cnn_input(8)
    y = run_host(models.qcnn_spec(oracle, 8), [x], tmp_path / "qcnn")
    assert np.array_equal(y, models.qcnn_reference(oracle, x).reshape(-1))
    p = models.qdq_conv_params()
    y = run_host(models.qdq_conv_spec(), [p["x"]], tmp_path / "qdq")
    assert np.array_equal(y, models.qdq_conv_reference(oracle).reshape(-1))
    # weights as literals (int8, int32 and float tensors in the header)
    y = run_host(models.qdq_conv_spec(), [p["x"]], tmp_path / "qdq_lit", no_weight_file=True)
    assert np.array_equal(y, models.qdq_conv_reference(oracle).reshape(-1))


def test_host_session_options(tmp_path):
    """Weights as literals, a binary weight file, and a run-time batch give the same numbers as the plain host Session."""
    spec, x = models.mlp_spec()
    ref = models.mlp_reference(oracle).reshape(-1)
    assert rel_err(run_host(spec, [x], tmp_path / "lit", no_weight_file=True), ref) <= 1e-5
    assert rel_err(run_host(models.mlp_spec()[0], [x], tmp_path / "bin", binary_weight_file=True), ref) <= 1e-5
    x8 = models.cnn_input(8)
    y = run_host(models.cnn_f32_rt_spec(), [x8], tmp_path / "rt")      # infer(float*) runs the whole capacity
    assert rel_err(y, models.cnn_f32_stages(oracle, x8)["y"].reshape(-1)) <= 1e-5


def test_host_session_with_a_blas_library(tmp_path):
    """sgemm_ / saxpy_ bound to a BLAS library at run time (SOFIE_BLAS) instead of the runner's loops."""
    if not os.path.exists(MKL):
        pytest.skip("no MKL in this image")
    x = models.cnn_input(8)
    y, timing = run_host(models.cnn_f32_spec(8), [x], tmp_path, env={"SOFIE_BLAS": MKL, "MKL_NUM_THREADS": "2"}, iters=3)
    assert timing["blas"] == MKL and timing["host_ms"] > 0
    assert rel_err(y, models.cnn_f32_stages(oracle, x)["y"].reshape(-1)) <= 1e-5


def test_operators_without_a_host_form_say_so(tmp_path):
    """GemmFP8 is the one operator of the device path without a host form."""
    s = emit.ModelSpec("fp8")
    s.add_input("a", "FLOAT8E4M3FN", (4, 16))
    s.add_init("b", np.zeros((16, 8), np.uint8), "FLOAT8E4M3FN")
    s.add_scalar("sa", 1.0, np.float32)
    s.add_scalar("sb", 1.0, np.float32)
    s.gemm_fp8("a", "sa", "b", "sb", None, "y")
    s.set_output("y", "BFLOAT16")
    _, _, res = s.generate(str(tmp_path), host_code=True, check=False)
    assert res.returncode != 0 and "no host emission" in res.stderr


def test_batchnorm_conv_transpose_and_stacked_products_as_host_code(tmp_path):
    """Conv + BatchNormalization + Relu (the normalisation is its own loop here: no folding pass runs), a 1-D
    convolution, pooling over one and three axes, stacked MatMul: 1e-5 relative against the oracle's references."""
    p = models.convbn_params()
    assert rel_err(run_host(models.convbn_spec(), [p["x"]], tmp_path / "bn"), models.convbn_reference(oracle).reshape(-1)) <= 1e-5
    p = models.conv1d_params()
    assert rel_err(run_host(models.conv1d_spec(), [p["x"]], tmp_path / "c1"), models.conv1d_reference(oracle).reshape(-1)) <= 1e-5
    p = models.conv3d_params()
    assert rel_err(run_host(models.conv3d_spec(), [p["x"]], tmp_path / "c3"), models.conv3d_reference(oracle).reshape(-1)) <= 1e-5
    assert rel_err(run_host(models.pool1d_spec(), [models.pool1d_input()], tmp_path / "p1"), models.pool1d_reference(oracle).reshape(-1)) <= 1e-5
    assert rel_err(run_host(models.pool3d_spec(), [models.pool3d_input()], tmp_path / "p3"), models.pool3d_reference(oracle).reshape(-1)) <= 1e-5


@pytest.mark.parametrize("seed", random_graphs.FLOAT_SEEDS)
def test_random_float_graphs_against_torch(seed, tmp_path):
    """Conv with random groups, strides, dilations and four different pads, then Relu / MaxPool / AveragePool (with and
    without the padding cells in the count) / Flatten + Gemm: the generated host Session against torch's CPU operators,
    which share nothing with the emitter or the oracle. 1e-5 of the largest output."""
    spec, x, want = random_graphs.float_graph(seed)
    y = run_host(spec, [x], tmp_path)
    assert y.size == want.size
    assert np.max(np.abs(y - want)) <= 1e-5 * max(1.0, float(np.max(np.abs(want))))


@pytest.mark.parametrize("seed", random_graphs.QUANT_SEEDS)
def test_random_quantized_graphs_are_bit_exact(seed, tmp_path):
    """QuantizeLinear, QLinearConv with random channels, groups, kernel, stride, pads, zero-points and per-channel
    scales, optional Relu and 2x2 MaxPool, DequantizeLinear: the generated host Session equals the oracle bit for bit."""
    spec, x, want = random_graphs.quantized_graph(seed, oracle)
    y = run_host(spec, [x], tmp_path)
    assert np.array_equal(y, want)


@pytest.mark.parametrize("name", ["Linear_16", "ConvWithPadding", "MaxPool2d"])
def test_onnx_file_to_host_session(name, tmp_path):
    """The C++ ONNX front end with --host: the reference's fixture file straight to a host Session, same numbers as the
    reference's expected output."""
    emit.build_emitter()
    entry = json.load(open(os.path.join(GOLD, "expected.json")))[name]
    _, graph = models.fixture_spec(name)
    feeds = replay.fixture_feeds(entry, graph)
    xs = [feeds[i[0]] for i in graph["inputs"]]
    out = str(tmp_path)
    r = subprocess.run([os.path.join(emit.GEN_DIR, "emit_from_onnx"), os.path.join(GOLD, "onnx", name + ".onnx"), out, "--host"],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert r.returncode == 0, r.stderr
    assert "sofie_hip" not in open(os.path.join(out, name + ".hxx")).read()
    exe = emit.compile_host_runner(name, out, num_inputs=len(xs))
    names = []
    for i, a in enumerate(xs):
        names.append(os.path.join(out, "in%d.bin" % i))
        np.ascontiguousarray(a, np.float32).tofile(names[-1])
    fout = os.path.join(out, "out.bin")
    r = subprocess.run([exe, os.path.join(out, name + ".dat"), ",".join(names), fout], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert r.returncode == 0, r.stderr
    y = np.fromfile(fout, np.float32)
    want = np.array(entry["expected"], np.float32)
    assert y.size == want.size and np.max(np.abs(y - want)) <= 1e-3
