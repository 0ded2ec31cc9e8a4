"""CPU-side safety net: the host emitter, the ONNX wire parser and the oracle built with AddressSanitizer and
UndefinedBehaviorSanitizer (`make -C sofie_amd/host SAN=1`, `make -C oracle san`), run over the fixtures, over every
model description of the GPU tests and over mutated ONNX bytes. A parser may reject a damaged file (exit status 1
with a message) or accept it; it may never crash, read out of bounds or overflow. The code the emitter generates for
the host cores is compiled with the same sanitizers and run as well."""
import os
import subprocess
import sys

import numpy as np
import pytest

from sofie_amd import emit
import models

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SAN_DIR = os.path.join(emit.GEN_DIR, "san")
GOLD = os.path.join(ROOT, "tests", "golden", "onnx")
SAN_ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:exitcode=99", UBSAN_OPTIONS="print_stacktrace=1")


@pytest.fixture(scope="module")
def san_tools():
    res = subprocess.run(["make", "-C", os.path.join(ROOT, "sofie_amd", "host"), "SAN=1", "-j4"], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout[-2000:]
    return os.path.join(SAN_DIR, "emit_from_spec"), os.path.join(SAN_DIR, "emit_from_onnx")


def _clean(res):
    text = res.stdout + res.stderr
    assert res.returncode in (0, 1), "exit status %d\n%s" % (res.returncode, text[-3000:])
    assert "AddressSanitizer" not in text and "runtime error:" not in text and "LeakSanitizer" not in text, text[-3000:]


def test_emitters_are_clean_on_every_model(san_tools, tmp_path):
    """Every fixture through the ONNX front end and every model description of the GPU tests through the
    description-driven emitter, under the sanitizers; the generated code equals the ordinary build's."""
    spec_exe, onnx_exe = san_tools
    for name in models.FIXTURES:
        res = subprocess.run([onnx_exe, os.path.join(GOLD, name + ".onnx"), str(tmp_path)], stdout=subprocess.PIPE,
                             stderr=subprocess.PIPE, text=True, env=SAN_ENV, timeout=120)
        _clean(res)
        assert res.returncode == 0, res.stderr
    import build_generated
    from oracle import oracle
    for spec in build_generated.all_specs(with_large=False):
        sub = tmp_path / spec.name
        sub.mkdir()
        hxx, dat, res0 = spec.generate(str(sub))
        out2 = tmp_path / (spec.name + "_san")
        out2.mkdir()
        hxx2, _, res = spec.generate(str(out2), check=False, emitter=spec_exe, env=SAN_ENV)
        _clean(res)
        assert res.returncode == 0, res.stderr[-2000:]
        strip = lambda path: [l for l in open(path).read().split("\n") if not l.startswith("//Code generated")]
        assert strip(hxx) == strip(hxx2)
    # the host emission (Options::kHostCode) of the fixtures, under the sanitizers too: a model whose operators all
    # have a host form generates, any other is refused with a message
    for name in models.FIXTURES:
        res = subprocess.run([onnx_exe, os.path.join(GOLD, name + ".onnx"), str(tmp_path), "--host"], stdout=subprocess.PIPE,
                             stderr=subprocess.PIPE, text=True, env=SAN_ENV, timeout=120)
        _clean(res)
        assert res.returncode == 0 or "has no host emission" in res.stderr, res.stderr


def test_onnx_parser_survives_mutated_files(san_tools, tmp_path):
    """Byte flips, truncations, length-field damage and random splices of the golden .onnx files: the front end
    rejects or parses, under the sanitizers, and never takes longer than a few seconds."""
    _, onnx_exe = san_tools
    r = np.random.default_rng(11)
    names = ["Linear_16", "ConvWithPadding", "ConvTransposeBias2d", "MaxPool2d", "ConvWithAutopadSameLower"]
    blobs = {n: open(os.path.join(GOLD, n + ".onnx"), "rb").read() for n in names}
    cases = 0
    for name, blob in blobs.items():
        head = min(len(blob), 600)          # structure lives in the first bytes and in the tail; weights in between
        variants = []
        for _ in range(40):
            b = bytearray(blob)
            kind = r.integers(0, 5)
            if kind == 0:                     # flip a few bytes near the structure
                for _ in range(int(r.integers(1, 6))):
                    pos = int(r.integers(0, head)) if r.random() < 0.5 else int(r.integers(len(b) - head, len(b)))
                    b[pos] = int(r.integers(0, 256))
            elif kind == 1:                   # truncate
                b = b[:int(r.integers(1, len(b)))]
            elif kind == 2:                   # a huge varint where a length or a dimension stood
                pos = int(r.integers(0, head))
                b[pos:pos + 1] = b"\xff\xff\xff\xff\xff\xff\xff\xff\x7f"
            elif kind == 3:                   # splice a piece of the file into another place
                a0, a1 = sorted(int(v) for v in r.integers(0, len(b), 2))
                pos = int(r.integers(0, len(b)))
                b[pos:pos] = b[a0:min(a1, a0 + 200)]
            else:                             # zero a window
                pos = int(r.integers(0, len(b) - 8))
                b[pos:pos + 8] = bytes(8)
            variants.append(bytes(b))
        for i, v in enumerate(variants):
            path = tmp_path / ("%s_%d.onnx" % (name, i))
            path.write_bytes(v)
            res = subprocess.run([onnx_exe, str(path), str(tmp_path)], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                                 text=True, env=SAN_ENV, timeout=60)
            _clean(res)
            os.remove(path)
            cases += 1
    assert cases == 200


def test_oracle_is_clean_under_the_sanitizers():
    """The oracle's own tests once more against liboracle_san.so, in a child Python with libasan preloaded."""
    res = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "san"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout[-2000:]
    asan = subprocess.run(["gcc", "-print-file-name=libasan.so"], stdout=subprocess.PIPE, text=True).stdout.strip()
    if not os.path.isabs(asan) or not os.path.exists(asan):
        pytest.skip("libasan.so not found next to gcc")
    env = dict(os.environ, LD_PRELOAD=asan, ASAN_OPTIONS="detect_leaks=0:exitcode=99",
               SOFIE_ORACLE_LIB=os.path.join(ROOT, "oracle", "liboracle_san.so"))
    res = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider",
                          os.path.join(ROOT, "tests", "test_oracle_golden.py"),
                          os.path.join(ROOT, "tests", "test_oracle_math.py"), "-k", "not cpu_baseline_program"],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=900, cwd=ROOT)
    text = res.stdout
    assert "AddressSanitizer" not in text and "runtime error:" not in text, text[-3000:]
    assert res.returncode == 0, text[-3000:]


def test_generated_host_sessions_run_clean(tmp_path):
    """The code the emitter writes for the host cores, compiled with AddressSanitizer and UndefinedBehaviorSanitizer and
    run: the fp32 CNN, the int8 CNN (QuantizeLinear, QLinearConv + pooling, QLinearMatMul), quantize -> conv ->
    dequantize, graphs with random attributes, a transposed convolution and an Einsum. Same outputs as the ordinary
    build checks elsewhere; here no report from either sanitizer."""
    import random_graphs
    import replay
    import json
    from oracle import oracle
    cases = []
    x2 = models.cnn_input(2)
    cases.append((models.cnn_f32_spec(2, "cnn_f32_b2"), [x2], models.cnn_f32_stages(oracle, x2)["y"].reshape(-1), 1e-5))
    cases.append((models.qcnn_spec(oracle, 2, "qcnn_b2"), [x2], models.qcnn_reference(oracle, x2).reshape(-1), 0.0))
    cases.append((models.qdq_conv_spec(), [models.qdq_conv_params()["x"]], models.qdq_conv_reference(oracle).reshape(-1), 0.0))
    for seed in random_graphs.FLOAT_SEEDS[:3]:
        s, x, want = random_graphs.float_graph(seed)
        cases.append((s, [x], want, 1e-5))
    for seed in random_graphs.QUANT_SEEDS[1:3]:
        s, x, want = random_graphs.quantized_graph(seed, oracle)
        cases.append((s, [x], want, 0.0))
    expected = json.load(open(os.path.join(ROOT, "tests", "golden", "expected.json")))
    for name in ("ConvTransposeBias2dBatched", "Einsum_3"):
        spec, graph = models.fixture_spec(name)
        feeds = replay.fixture_feeds(expected[name], graph)
        cases.append((spec, [feeds[i[0]] for i in graph["inputs"]], np.array(expected[name]["expected"], np.float32), 1e-3))
    for spec, xs, want, tol in cases:
        d = tmp_path / spec.name
        d.mkdir()
        hxx, dat, _ = spec.generate(str(d), host_code=True)
        exe = str(d / "run")
        cmd = ["g++", "-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
               "-fno-sanitize-recover=undefined", "-I" + str(d), "-DSOFIE_MODEL_HEADER=\"%s.hxx\"" % spec.name,
               "-DSOFIE_MODEL_NS=SOFIE_%s" % spec.name, "-DSOFIE_NUM_INPUTS=%d" % len(xs),
               os.path.join(ROOT, "sofie_amd", "host", "examples", "run_host_session.cxx"), "-o", exe, "-ldl"]
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        assert res.returncode == 0, res.stdout[-2000:]
        names = []
        for i, a in enumerate(xs):
            names.append(str(d / ("in%d.bin" % i)))
            np.ascontiguousarray(a, np.float32).tofile(names[-1])
        res = subprocess.run([exe, dat, ",".join(names), str(d / "out.bin")], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                             env=SAN_ENV, timeout=300)
        _clean(res)
        assert res.returncode == 0, spec.name + "\n" + res.stderr[-2000:]
        y = np.fromfile(str(d / "out.bin"), np.float32)
        assert y.size == want.size, spec.name
        if tol == 0.0:
            assert np.array_equal(y, want), spec.name
        else:
            assert np.max(np.abs(y - want)) <= tol * max(1.0, float(np.max(np.abs(want)))), spec.name
