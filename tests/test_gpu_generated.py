"""Generated Sessions on the GPU: the code the C++ emitter wrote (prebuilt by tests/build_generated.py) is run
as its own process, the way a user of the generated header runs it, and its output is compared with the
reference's expected vectors and with the CPU oracle.

Bars: fp32 networks 1e-5 relative (max |d| / max |ref|); int8 network logits identical, since they are an exact
int32 accumulator times an fp32 scale."""
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

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def run_session(name, x, tmp_path, out_dtype=np.float32, dat=None, iters=0):
    exe = os.path.join(emit.GEN_DIR, "run_" + name)
    if not os.path.exists(exe):
        raise RuntimeError("%s is missing: run python tests/build_generated.py on the build machine" % exe)
    fout = str(tmp_path / "out.bin")
    if isinstance(x, (list, tuple)):
        # one file per input of the model, in the order of infer()'s arguments
        names = [str(tmp_path / ("in%d.bin" % i)) for i in range(len(x))]
        for f, a in zip(names, x):
            np.ascontiguousarray(a).tofile(f)
        fin = ",".join(names)
    else:
        fin = str(tmp_path / "in.bin")
        np.ascontiguousarray(x).tofile(fin)
    cmd = [exe, os.path.join(emit.GEN_DIR, (dat or name) + ".dat"), fin, fout] + ([str(iters)] if iters else [])
    print("running", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=110)
    assert res.returncode == 0, res.stderr
    y = np.fromfile(fout, out_dtype)
    return (y, json.loads(res.stdout)) if iters else y


def run_session_outputs(name, x, tmp_path, out_dtypes):
    """Runner of a model with several outputs: one raw file per output, in the order of the output list."""
    exe = os.path.join(emit.GEN_DIR, "run_" + name)
    if not os.path.exists(exe):
        raise RuntimeError("%s is missing: run python tests/build_generated.py on the build machine" % exe)
    fin = str(tmp_path / "in.bin")
    np.ascontiguousarray(x).tofile(fin)
    fouts = [str(tmp_path / ("out%d.bin" % i)) for i in range(len(out_dtypes))]
    cmd = [exe, os.path.join(emit.GEN_DIR, name + ".dat"), fin, ",".join(fouts)]
    print("running", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=110)
    assert res.returncode == 0, res.stderr
    return [np.fromfile(f, d) for f, d in zip(fouts, out_dtypes)]


def rel_err(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) / max(float(np.max(np.abs(b))), 1e-30))


@pytest.mark.parametrize("name", models.FIXTURES)
def test_reference_fixture_through_generated_session(name, tmp_path):
    entry = json.load(open(os.path.join(GOLD, "expected.json")))[name]
    _, graph = models.fixture_spec(name)
    feeds = replay.fixture_feeds(entry, graph)
    xs = [feeds[i[0]] for i in graph["inputs"]]
    y = run_session(name, xs if len(xs) > 1 else xs[0], tmp_path)
    want = np.array(entry["expected"], np.float32)
    assert y.size == want.size
    assert np.max(np.abs(y - want)) <= 1e-3             # the reference's own tolerance
    yo = replay.run_graph(graph, feeds, oracle)
    assert rel_err(y, yo.reshape(-1)) <= 1e-5


@pytest.mark.parametrize("seed", random_graphs.FLOAT_SEEDS)
def test_random_float_graph_sessions_against_torch(seed, tmp_path):
    """Generated device Sessions of graphs with random attributes (Conv with groups, strides, dilations, four different
    pads; Relu, MaxPool, AveragePool, Flatten + Gemm behind it) against torch's CPU operators: 1e-5 of the largest
    output."""
    spec, x, want = random_graphs.float_graph(seed)
    y = run_session(spec.name, x, tmp_path)
    assert y.size == want.size
    assert np.max(np.abs(y - want)) <= 1e-5 * max(1.0, float(np.max(np.abs(want))))


@pytest.mark.parametrize("seed", random_graphs.QUANT_SEEDS)
def test_random_quantized_graph_sessions_are_bit_exact(seed, tmp_path):
    """QuantizeLinear, QLinearConv (random channels, groups, kernel, stride, pads, zero-points, per-channel scales),
    optional Relu and 2x2 MaxPool, DequantizeLinear as generated device Sessions: the oracle's output bit for bit."""
    spec, x, want = random_graphs.quantized_graph(seed, oracle)
    y = run_session(spec.name, x, tmp_path)
    assert np.array_equal(y, want)


def test_mlp_session(tmp_path):
    _, x = models.mlp_spec()
    y = run_session("mlp_c1", x, tmp_path)
    ref = models.mlp_reference(oracle)
    assert rel_err(y, ref.reshape(-1)) <= 1e-5


def test_cnn_f32_session(tmp_path):
    x = models.cnn_input(8)
    y = run_session("cnn_f32", x, tmp_path)
    ref = models.cnn_f32_stages(oracle, x)["y"]
    assert rel_err(y, ref.reshape(-1)) <= 1e-5


@pytest.mark.parametrize("name,weights", [("mlp_c1", "mlp_c1"), ("cnn_f32", "cnn_f32"), ("qcnn", "qcnn")])
def test_host_and_device_emission_agree(name, weights, tmp_path):
    """The same model generated twice, as calls into the kernel library and as code for the host cores
    (Options::kHostCode: the reference's BLAS calls and loops; for the quantized operators, which the reference does
    not have, loops with int32 sums and the same rounding rule), on the same seeded input: within 1e-5 relative for the
    float networks, bit for bit for the int8 network."""
    x = models.mlp_spec()[1] if name == "mlp_c1" else models.cnn_input(8)
    y_device = run_session(name, x, tmp_path)
    exe = os.path.join(emit.GEN_DIR, "host", "run_host_" + name)
    if not os.path.exists(exe):
        raise RuntimeError("%s is missing: run python tests/build_generated.py on the build machine" % exe)
    fout = str(tmp_path / "host_out.bin")
    res = subprocess.run([exe, os.path.join(emit.GEN_DIR, weights + ".dat"), str(tmp_path / "in.bin"), fout],
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=110)
    assert res.returncode == 0, res.stderr
    y_host = np.fromfile(fout, np.float32)
    assert y_host.size == y_device.size
    if name == "qcnn":
        assert np.array_equal(y_device, y_host)
    else:
        assert rel_err(y_device, y_host) <= 1e-5


def test_runtime_batch_sessions(tmp_path):
    """Sessions generated with a batch capacity of 8 run 8, 3 and 1 images through infer(n, ...): the int8 network's
    logits are those of the oracle on the same images bit for bit, the float network's within 1e-5."""
    x = models.cnn_input(8)
    for n in (8, 3, 1):
        exe = os.path.join(emit.GEN_DIR, "run_qcnn_rt")
        fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
        np.ascontiguousarray(x[:n]).tofile(fin)
        cmd = [exe, os.path.join(emit.GEN_DIR, "qcnn.dat"), fin, fout, str(n)]   # the weight file of the fixed-batch Session
        print("running", " ".join(cmd), flush=True)
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=110)
        assert res.returncode == 0, res.stderr
        y = np.fromfile(fout, np.float32)
        ref = models.qcnn_reference(oracle, x[:n])
        assert y.size == ref.size and np.array_equal(y, ref.reshape(-1))
    n = 5
    exe = os.path.join(emit.GEN_DIR, "run_cnn_f32_rt")
    fin, fout = str(tmp_path / "inf.bin"), str(tmp_path / "outf.bin")
    np.ascontiguousarray(x[:n]).tofile(fin)
    res = subprocess.run([exe, os.path.join(emit.GEN_DIR, "cnn_f32.dat"), fin, fout, str(n)], stdout=subprocess.PIPE,
                         stderr=subprocess.PIPE, text=True, timeout=110)
    assert res.returncode == 0, res.stderr
    y = np.fromfile(fout, np.float32)
    ref = models.cnn_f32_stages(oracle, x[:n])["y"]
    assert y.size == ref.size and rel_err(y, ref.reshape(-1)) <= 1e-5
    # a batch beyond the capacity is refused by the Session
    np.ascontiguousarray(np.concatenate([x, x[:1]])).tofile(fin)
    res = subprocess.run([exe, os.path.join(emit.GEN_DIR, "cnn_f32.dat"), fin, fout, "9"], stdout=subprocess.PIPE,
                         stderr=subprocess.PIPE, text=True, timeout=110)
    assert res.returncode != 0 and "the batch must be between 1 and 8" in res.stderr


def test_conv_1d_and_3d_sessions(tmp_path):
    """A 1-D convolution runs on the 2-D kernel with a height of one (1e-5 relative); the 3-D kernel sums in the
    order of the reference's column matrix, so it equals the oracle exactly."""
    y = run_session("conv1d", models.conv1d_params()["x"], tmp_path)
    ref = models.conv1d_reference(oracle)
    assert y.size == ref.size and rel_err(y, ref.reshape(-1)) <= 1e-5
    y = run_session("conv3d", models.conv3d_params()["x"], tmp_path)
    ref = models.conv3d_reference(oracle)
    assert y.size == ref.size and np.array_equal(y, ref.reshape(-1))


def test_pooling_over_one_and_three_axes_sessions(tmp_path):
    """MaxPool and AveragePool on [N,C,W] (the two-axis kernels with a height of one) and on [N,C,D,H,W] (kernels of
    their own) with begin pads that differ from the end pads: the maximum is exact, the average sums in the oracle's
    order and is exact too."""
    y = run_session("pool1d", models.pool1d_input(), tmp_path)
    ref = models.pool1d_reference(oracle)
    assert y.size == ref.size and np.array_equal(y, ref.reshape(-1))
    y = run_session("pool3d", models.pool3d_input(), tmp_path)
    ref = models.pool3d_reference(oracle)
    assert y.size == ref.size and np.array_equal(y, ref.reshape(-1))


def test_conv_batchnorm_convtranspose_session(tmp_path):
    """Conv -> BatchNormalization -> Relu (folded into the convolution at generation time) -> MaxPool ->
    BatchNormalization (its own kernel) -> ConvTranspose -> Relu against the unfused oracle steps; 1e-5 relative
    (folding the scale into the weights rounds differently from scaling the sum)."""
    p = models.convbn_params()
    y = run_session("convbn", p["x"], tmp_path)
    ref = models.convbn_reference(oracle)
    assert y.size == ref.size
    assert rel_err(y, ref.reshape(-1)) <= 1e-5


@pytest.mark.parametrize("name,make_input", [
    ("mlp_c1", lambda: models.mlp_spec()[1]), ("cnn_f32", lambda: models.cnn_input(8)), ("qcnn", lambda: models.cnn_input(8)),
    ("qdq_conv", lambda: models.qdq_conv_params()["x"]), ("convbn", lambda: models.convbn_params()["x"]),
    ("stacked", lambda: models.stacked_params()["x"]), ("qcnn_b4096", lambda: models.cnn_input(4096))])
def test_graph_replay_matches_eager(name, make_input, tmp_path):
    """Session::use_graph: the operator sequence recorded into a HIP graph at the first infer() and replayed afterwards
    gives the same bytes as the eager sequence, on four replays with eager runs and synchronisations in between."""
    _, timing = run_session(name, make_input(), tmp_path, iters=5, dat="qcnn" if name == "qcnn_b4096" else None)
    assert timing["graph_matches"] is True
    assert timing["graph_ms"] > 0
    assert timing["pinned_matches"] is True and timing["host_pinned_ms"] > 0   # infer() on the page-locked input buffer
    # two Sessions of the model in flight at once (own contexts and streams, a host thread each) give the same bytes
    assert timing["sessions_in_flight"] == 2 and timing["two_sessions_match"] is True and timing["two_sessions_ms_per_batch"] > 0
    # one entry per launch of the sequence, timed by the events the library records behind its launches; their sum is
    # the time of the sequence on the device (the five batches here are too few for the two to agree closely)
    assert len(timing["kernels"]) >= 1 and all(k["us"] > 0 and k["kernel"].startswith("k_") for k in timing["kernels"])
    if name == "qcnn_b4096":
        # (the second and third convolution are one launch at this batch)
        assert [k["kernel"] for k in timing["kernels"]] == ["k_qconv_first", "k_qconv_ring_pair", "k_gemm_bytes", "k_splitk_finish_pair"]


def test_stacked_matmul_session(tmp_path):
    """MatMul on stacked operands (numpy.matmul broadcasting of the leading dimensions): every product reads its
    own matrices; against the float64 product, 1e-5 relative."""
    p = models.stacked_params()
    y = run_session("stacked", p["x"], tmp_path)
    ref = models.stacked_reference()
    assert y.size == ref.size
    assert rel_err(y, ref.reshape(-1)) <= 1e-5


def test_sofie_functor_slots_from_threads(tmp_path):
    """SofieFunctor<4, Session> with three slots, each called from its own thread (one device context and stream
    per Session): every row equals the oracle's two-layer network, and one slot gives the same numbers."""
    p = models.functor_params()
    ref = models.functor_reference(oracle)
    fin = str(tmp_path / "rows.bin")
    p["rows"].tofile(fin)
    exe = os.path.join(emit.GEN_DIR, "run_functor")
    outs = []
    for slots in (3, 0):
        fout = str(tmp_path / ("out%d.bin" % slots))
        res = subprocess.run([exe, os.path.join(emit.GEN_DIR, "functor4.dat"), str(slots), fin, fout], stdout=subprocess.PIPE,
                             stderr=subprocess.PIPE, text=True, timeout=110)
        assert res.returncode == 0, res.stderr
        outs.append(np.fromfile(fout, np.float64))
    assert outs[0].size == ref.size and np.array_equal(outs[0], outs[1])
    assert rel_err(outs[0], ref) <= 1e-5


def test_binary_weight_file_gives_the_same_session(tmp_path):
    """The Session built from the binary weight file computes the same bytes as the one built from the text file."""
    p = models.convbn_params()
    y_text = run_session("convbn", p["x"], tmp_path)
    exe = os.path.join(emit.GEN_DIR, "run_convbn")
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out_b.bin")
    res = subprocess.run([exe, os.path.join(emit.GEN_DIR, "convbn.bin"), fin, fout], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                         text=True, timeout=110)
    assert res.returncode == 0, res.stderr
    assert np.array_equal(np.fromfile(fout, np.float32), y_text)


def test_int8_cnn_session_is_bit_exact(tmp_path):
    x = models.cnn_input(8)
    y = run_session("qcnn", x, tmp_path)
    ref = models.qcnn_reference(oracle, x)
    assert np.array_equal(y, ref.reshape(-1))
    # and it classifies like the float network it was quantized from
    f = models.cnn_f32_stages(oracle, x)["y"]
    assert np.array_equal(np.argmax(y.reshape(8, 5), 1), np.argmax(f, 1)) or rel_err(y, f.reshape(-1)) < 0.1


def test_quantize_conv_dequantize_session(tmp_path):
    """NCHW int8 into the conv, channels-last out of it, converted back for the float consumer: the floats are
    exact products of an int8 and the output scale, so they equal the oracle's bit for bit."""
    p = models.qdq_conv_params()
    y = run_session("qdq_conv", p["x"], tmp_path)
    ref = models.qdq_conv_reference(oracle)
    assert np.array_equal(y, ref.reshape(-1))


def test_int8_cnn_batch_4096_matches_the_oracle_on_a_sample_and_is_batch_invariant(tmp_path):
    """Full benchmark batch: every image is computed independently of its neighbours, so the first 8 rows
    equal the batch-8 Session's output, and 256 images spread over the batch equal the oracle."""
    x = models.cnn_input(4096)
    y = run_session("qcnn_b4096", x, tmp_path, dat="qcnn").reshape(4096, 5)
    pick = np.arange(0, 4096, 16) + (np.arange(256) % 16)          # one image of every group of 16, every position in a group
    ref = models.qcnn_reference(oracle, x[pick])
    assert np.array_equal(y[pick], ref)
    y8 = run_session("qcnn", x[:8], tmp_path).reshape(8, 5)
    assert np.array_equal(y[:8], y8)


def test_sessions_with_several_outputs(tmp_path):
    """Two float outputs (vector of vectors) and a float plus an int8 output (tuple): every output equals the
    oracle's tensor, the hidden layer that is an output is intact after the layers behind it ran."""
    _, x = models.two_heads_spec()
    h1, y = run_session_outputs("two_heads", x, tmp_path, (np.float32, np.float32))
    rh1, ry = models.two_heads_reference(oracle)
    assert h1.size == rh1.size and y.size == ry.size
    assert rel_err(h1, rh1.reshape(-1)) <= 1e-5 and rel_err(y, ry.reshape(-1)) <= 1e-5

    y, q = run_session_outputs("mixed_outputs", x, tmp_path, (np.float32, np.int8))
    ry, _ = models.mixed_outputs_reference(oracle)
    assert rel_err(y, ry.reshape(-1)) <= 1e-5
    # the int8 output is the quantisation of the float output the device computed, bit for bit
    assert np.array_equal(q, oracle.quantize_f32_s8(y, models.MIXED_SCALE, models.MIXED_ZP))


def test_no_session_free_function(tmp_path):
    """A model generated with Options::kNoSession: the free function infer (called twice, on the one Session it
    creates at its first call) gives the MLP's result."""
    _, x = models.mlp_nosession_spec()
    y = run_session("mlp_nosession", x, tmp_path, dat="unused")
    assert rel_err(y, models.mlp_reference(oracle).reshape(-1)) <= 1e-5


def test_binary_weight_file_with_another_element_type_is_refused(tmp_path):
    """A record with the right name and count but another type code would be reinterpreted byte for byte: the
    generated constructor throws instead (the process ends with a non-zero status before any kernel runs)."""
    import struct
    raw = bytearray(open(os.path.join(emit.GEN_DIR, "convbn.bin"), "rb").read())
    (nlen,) = struct.unpack_from("<I", raw, 16)
    (type_code,) = struct.unpack_from("<I", raw, 16 + 4 + nlen)
    assert type_code == 1
    struct.pack_into("<I", raw, 16 + 4 + nlen, 6)          # FLOAT -> INT32: same size, another meaning
    bad = tmp_path / "bad.bin"
    bad.write_bytes(bytes(raw))
    p = models.convbn_params()
    fin, fout = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    np.ascontiguousarray(p["x"], np.float32).tofile(fin)
    res = subprocess.run([os.path.join(emit.GEN_DIR, "run_convbn"), str(bad), fin, fout], stdout=subprocess.PIPE,
                         stderr=subprocess.PIPE, text=True, timeout=110)
    assert res.returncode != 0
    assert "correct tensor type" in res.stderr + res.stdout
