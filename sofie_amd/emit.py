"""Describe a network to the C++ emitter (RModel / ROperator), generate its Session header and
weight file, and compile a runner for it.

The C++ emit program (sofie_amd/host/examples/emit_from_spec.cxx) reads a line-based description
plus raw tensor files; this module writes those from numpy arrays or from a decoded ONNX graph
(sofie_amd.onnx_wire), applying the same operator fusions the reference's parser applies
(Gemm followed by a single-consumer Relu -> Gemm with RELU activation,
src/SOFIE_parsers/src/RModelParser_ONNX.cxx:316-321).
"""
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_HERE)
GEN_DIR = os.path.join(_HERE, "generated")
EMIT = os.path.join(GEN_DIR, "emit_from_spec")

_TYPE = {np.dtype(np.float32): "FLOAT", np.dtype(np.int8): "INT8", np.dtype(np.uint8): "UINT8",
         np.dtype(np.int32): "INT32", np.dtype(np.int64): "INT64"}
_CTYPE = {"FLOAT": "float", "INT8": "int8_t", "UINT8": "uint8_t", "INT32": "int32_t", "FLOAT8E4M3FN": "uint8_t",
          "BFLOAT16": "uint16_t"}


def build_emitter():
    subprocess.run(["make", "-C", os.path.join(_HERE, "host"), "-j4"], check=True, stdout=subprocess.DEVNULL)
    return EMIT


def _lst(v):
    v = list(v)
    return "%d %s" % (len(v), " ".join(str(x) if isinstance(x, str) else str(int(x)) for x in v)) if v else "0"


class ModelSpec:
    """Accumulates the statements of one model description."""

    def __init__(self, name):
        self.name = name
        self.lines = ["model %s" % name]
        self.tensors = {}
        self.input = None      # the first input (single-input runners)
        self.inputs = []
        self.output = None     # the first output
        self.out_type = "FLOAT"
        self.outputs = []      # (name, type) of every output, in the order infer() returns them
        self.batch = None            # value of the inputs' shape parameters at generation time
        self.runtime_batch = False   # ... as a capacity: the Session also takes infer(n, ...)
        self.no_session = False      # Options::kNoSession: free function infer, weights as literals

    def add_input(self, name, dtype, shape):
        t = dtype if isinstance(dtype, str) else _TYPE[np.dtype(dtype)]
        self.lines.append("input %s %s %s" % (name, t, _lst(shape)))
        if self.input is None:
            self.input = (name, t, tuple(shape))
        self.inputs.append((name, t, tuple(shape)))

    def add_init(self, name, array, type_name=None):
        array = np.ascontiguousarray(array)
        t = type_name or _TYPE[array.dtype]
        fname = "%s__%s.bin" % (self.name, "".join(c if c.isalnum() else "_" for c in name))
        self.tensors[fname] = array
        self.lines.append("init %s %s %s %s" % (name, t, _lst(array.shape), fname))

    def add_scalar(self, name, value, dtype):
        self.add_init(name, np.array([value], dtype))

    def set_output(self, name, type_name="FLOAT"):
        self.lines.append("output %s" % name)
        if self.output is None:
            self.output = name
            self.out_type = type_name
        self.outputs.append((name, type_name))

    # ---- operators -------------------------------------------------------------------------
    def gemm(self, a, b, c, y, alpha=1.0, beta=1.0, transA=0, transB=0, relu=False):
        self.lines.append("op Gemm %r %r %d %d %s %s %s %s %d" % (float(alpha), float(beta), transA, transB, a, b,
                                                                 c or "-", y, int(relu)))

    def conv(self, x, w, b, y, kernel=(), pads=(), strides=(), dilations=(), group=1, auto_pad="NOTSET"):
        self.lines.append("op Conv %s %d %s %s %s %s %s %s %s %s" % (auto_pad, group, _lst(kernel), _lst(pads),
                                                                    _lst(strides), _lst(dilations), x, w, b or "-", y))

    def conv_transpose(self, x, w, b, y, kernel=(), pads=(), strides=(), dilations=(), group=0, output_padding=(),
                       output_shape=(), auto_pad="NOTSET"):
        self.lines.append("op ConvTranspose %s %d %s %s %s %s %s %s %s %s %s %s" % (
            auto_pad, group, _lst(kernel), _lst(pads), _lst(strides), _lst(dilations), _lst(output_padding),
            _lst(output_shape), x, w, b or "-", y))

    def batchnorm(self, x, scale, b, mean, var, y, epsilon=1e-5):
        self.lines.append("op BatchNormalization %r %s %s %s %s %s %s" % (float(epsilon), x, scale, b, mean, var, y))

    def einsum(self, equation, xs, y):
        self.lines.append("op Einsum %s %d %s %s" % (equation.replace(" ", ""), len(xs), " ".join(xs), y))

    def relu(self, x, y):
        self.lines.append("op Relu %s %s" % (x, y))

    def avgpool(self, x, y, kernel, pads=(0, 0, 0, 0), strides=(1, 1), count_include_pad=False):
        self.lines.append("op %s %s %s %s %s %s" % ("AveragePoolIncludePad" if count_include_pad else "AveragePool", _lst(kernel),
                                                    _lst(pads), _lst(strides), x, y))

    def global_avgpool(self, x, y):
        self.lines.append("op GlobalAveragePool %s %s" % (x, y))

    def maxpool(self, x, y, kernel, pads=(0, 0, 0, 0), strides=(1, 1)):
        self.lines.append("op MaxPool %s %s %s %s %s" % (_lst(kernel), _lst(pads), _lst(strides), x, y))

    def flatten(self, x, y, axis=1):
        self.lines.append("op Flatten %d %s %s" % (axis, x, y))

    def quantize(self, x, scale, zp, y):
        self.lines.append("op QuantizeLinear %s %s %s %s" % (x, scale, zp or "-", y))

    def dequantize(self, x, scale, zp, y):
        self.lines.append("op DequantizeLinear %s %s %s %s" % (x, scale, zp or "-", y))

    def qlinear_matmul(self, a, a_scale, a_zp, b, b_scale, b_zp, y_scale, y_zp, y, bias=None, transB=0):
        self.lines.append("op QLinearMatMul %s %s %s %s %s %s %s %s %s %s %d" % (
            a, a_scale, a_zp or "-", b, b_scale, b_zp or "-", y_scale or "-", y_zp or "-", bias or "-", y, transB))

    def qlinear_conv(self, x, x_scale, x_zp, w, w_scale, w_zp, y_scale, y_zp, y, bias=None, kernel=(), pads=(),
                     strides=(), group=1, auto_pad="NOTSET"):
        self.lines.append("op QLinearConv %s %d %s %s %s %s %s %s %s %s %s %s %s %s %s" % (
            auto_pad, group, _lst(kernel), _lst(pads), _lst(strides), x, x_scale, x_zp or "-", w, w_scale,
            w_zp or "-", y_scale, y_zp or "-", bias or "-", y))

    def gemm_fp8(self, a, a_scale, b, b_scale, bias, y, transB=0):
        self.lines.append("op GemmFP8 %s %s %s %s %s %s %d" % (a, a_scale, b, b_scale, bias or "-", y, transB))

    # ---- generation ------------------------------------------------------------------------
    def generate(self, outdir=GEN_DIR, no_weight_file=False, check=True, binary_weight_file=False, batch=None,
                 runtime_batch=False, no_session=False, emitter=None, env=None, layer_per_call=False, params=None,
                 host_code=False):
        """Run the C++ emitter. Returns (header path, weight file path, CompletedProcess). `batch` gives the shape
        parameters of the inputs (dimensions written as names) their value; with `runtime_batch` it is a capacity and
        the generated Session also takes infer(n, ...) for any n up to it. `emitter` names another build of the emit
        program (the sanitizer build), `env` its environment. `host_code` asks for Options::kHostCode: the Session for
        the host cores (BLAS calls and loops, as the reference generates it) instead of calls into the kernel library."""
        os.makedirs(outdir, exist_ok=True)
        tdir = os.path.join(outdir, "tensors")
        os.makedirs(tdir, exist_ok=True)
        for fname, arr in self.tensors.items():
            arr.tofile(os.path.join(tdir, fname))
        spec = os.path.join(outdir, self.name + ".spec")
        with open(spec, "w") as f:
            flag = " noweightfile" if no_weight_file else (" binaryweightfile" if binary_weight_file else "")
            if no_session or self.no_session:
                flag = " nosession"
            batch = self.batch if batch is None else batch
            if batch is not None:
                flag += " batch %d" % batch
            for pname, value in (params or {}).items():      # shape parameters by name (RModel::Initialize(map))
                flag += " param %s %d" % (pname, value)
            if runtime_batch or self.runtime_batch:
                flag += " runtimebatch"
            if layer_per_call:
                flag += " layerpercall"       # Options::kLayerPerCall: no chains of fully connected layers in one launch
            if host_code:
                flag += " hostcode"
            f.write("\n".join(self.lines + ["generate" + flag]) + "\n")
        if emitter is None and not os.path.exists(EMIT):
            build_emitter()
        res = subprocess.run([emitter or EMIT, spec, tdir, outdir], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                             env=env)
        if check and res.returncode:
            raise RuntimeError("emitter failed: " + res.stderr)
        for fname in self.tensors:
            os.remove(os.path.join(tdir, fname))
        return (os.path.join(outdir, self.name + ".hxx"),
                os.path.join(outdir, self.name + (".bin" if binary_weight_file else ".dat")), res)

    def compile_runner(self, outdir=GEN_DIR, runtime_batch=False):
        """g++ the generic runner against the generated header and libsofie_hip.so. With runtime_batch the runner's
        fourth argument is the batch it hands to infer(n, ...)."""
        exe = os.path.join(outdir, "run_" + self.name)
        cmd = ["g++", "-std=c++17", "-O2", "-pthread", "-I" + os.path.join(ROOT, "include"), "-I" + outdir,
               "-DSOFIE_MODEL_HEADER=\"%s.hxx\"" % self.name, "-DSOFIE_MODEL_NS=SOFIE_%s" % self.name,
               "-DSOFIE_IN_T=%s" % _CTYPE[self.input[1]], "-DSOFIE_OUT_T=%s" % _CTYPE[self.out_type],
               "-DSOFIE_INPUT_MEMBER=fInput_%s" % self.input[0], "-DSOFIE_PINNED_INPUT=pinned_input_%s" % self.input[0], "-DSOFIE_NUM_INPUTS=%d" % len(self.inputs),
               "-DSOFIE_NUM_OUTPUTS=%d" % max(1, len(self.outputs))] + \
              (["-DSOFIE_RUNTIME_BATCH"] if (runtime_batch or self.runtime_batch) else []) + \
              (["-DSOFIE_NO_SESSION"] if self.no_session else []) + [
               os.path.join(_HERE, "host", "examples", "run_session.cxx"), "-o", exe,
               "-L" + _HERE, "-lsofie_hip", "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + _HERE]
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode:
            raise RuntimeError("compiling the generated Session failed:\n" + res.stdout)
        return exe


def compile_host_runner(model, outdir, num_inputs=1):
    """g++ host/examples/run_host_session.cxx against a header generated with host_code=True: a program for the host
    cores only (no kernel library, no GPU). Its sgemm_ / saxpy_ are the runner's own loops unless SOFIE_BLAS names a
    library at run time."""
    exe = os.path.join(outdir, "run_host_" + model)
    cmd = ["g++", "-std=c++17", "-O2", "-I" + outdir, "-DSOFIE_MODEL_HEADER=\"%s.hxx\"" % model,
           "-DSOFIE_MODEL_NS=SOFIE_%s" % model, "-DSOFIE_NUM_INPUTS=%d" % num_inputs,
           os.path.join(_HERE, "host", "examples", "run_host_session.cxx"), "-o", exe, "-ldl"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode:
        raise RuntimeError("compiling the generated host Session failed:\n" + res.stdout)
    return exe


def compile_example(source, model, exe_name, outdir=GEN_DIR):
    """g++ one of host/examples/*.cxx against the generated header of `model` and libsofie_hip.so."""
    exe = os.path.join(outdir, exe_name)
    cmd = ["g++", "-std=c++17", "-O2", "-pthread", "-I" + os.path.join(ROOT, "include"), "-I" + outdir,
           "-I" + os.path.join(_HERE, "host", "inc"), "-DSOFIE_MODEL_HEADER=\"%s.hxx\"" % model,
           "-DSOFIE_MODEL_NS=SOFIE_%s" % model, os.path.join(_HERE, "host", "examples", source), "-o", exe,
           "-L" + _HERE, "-lsofie_hip", "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + _HERE]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode:
        raise RuntimeError("compiling %s failed:\n%s" % (source, res.stdout))
    return exe


def clean(name):
    return "".join(c if (c.isalnum() or c == "_") else ("_" if c == "-" else "") for c in name)


def spec_from_onnx(name, graph):
    """Gemm / Relu / Conv / MaxPool / Flatten graph (sofie_amd.onnx_wire.load) -> ModelSpec."""
    spec = ModelSpec(name)
    for iname, _, ishape in graph["inputs"]:
        spec.add_input(clean(iname), "FLOAT", ishape)
    for k, v in graph["initializers"].items():
        spec.add_init(clean(k), v)
    nodes = graph["nodes"]
    consumers = {}
    for nd in nodes:
        for i in nd["inputs"]:
            consumers[i] = consumers.get(i, 0) + 1
    skip = set()
    for idx, nd in enumerate(nodes):
        if idx in skip:
            continue
        op, a, ins, out = nd["op_type"], nd["attrs"], [clean(i) for i in nd["inputs"]], clean(nd["outputs"][0])
        if op == "Gemm":
            relu = False
            # the parser's Gemm -> Relu fusion when the Gemm output has a single consumer
            if idx + 1 < len(nodes) and nodes[idx + 1]["op_type"] == "Relu" and \
                    nodes[idx + 1]["inputs"][0] == nd["outputs"][0] and consumers.get(nd["outputs"][0], 0) == 1:
                relu = True
                out = clean(nodes[idx + 1]["outputs"][0])
                skip.add(idx + 1)
            spec.gemm(ins[0], ins[1], ins[2] if len(ins) > 2 else None, out, a.get("alpha", 1.0),
                      a.get("beta", 1.0) if len(ins) > 2 else 0.0, a.get("transA", 0), a.get("transB", 0), relu)
        elif op == "Relu":
            spec.relu(ins[0], out)
        elif op == "Conv":
            spec.conv(ins[0], ins[1], ins[2] if len(ins) > 2 else None, out, a.get("kernel_shape", ()),
                      a.get("pads", ()), a.get("strides", ()), a.get("dilations", ()), a.get("group", 1),
                      a.get("auto_pad", "NOTSET"))
        elif op == "ConvTranspose":
            spec.conv_transpose(ins[0], ins[1], ins[2] if len(ins) > 2 else None, out, a.get("kernel_shape", ()),
                                a.get("pads", ()), a.get("strides", ()), a.get("dilations", ()), a.get("group", 0),
                                a.get("output_padding", ()), a.get("output_shape", ()), a.get("auto_pad", "NOTSET"))
        elif op == "Einsum":
            eq = a["equation"]
            spec.einsum(eq.decode() if isinstance(eq, bytes) else eq, ins, out)
        elif op == "BatchNormalization":
            spec.batchnorm(ins[0], ins[1], ins[2], ins[3], ins[4], out, a.get("epsilon", 1e-5))
        elif op == "MaxPool":
            spec.maxpool(ins[0], out, a["kernel_shape"], a.get("pads", ()), a.get("strides", ()))
        elif op == "AveragePool":
            spec.avgpool(ins[0], out, a["kernel_shape"], a.get("pads", ()), a.get("strides", ()),
                         bool(a.get("count_include_pad", 0)))
        elif op == "GlobalAveragePool":
            spec.global_avgpool(ins[0], out)
        elif op == "Flatten":
            spec.flatten(ins[0], out, a.get("axis", 1))
        else:
            raise NotImplementedError(op)
    spec.set_output(clean(graph["outputs"][0][0]))
    return spec
