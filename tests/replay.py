"""Replay a decoded ONNX graph (Gemm / Relu / Conv / ConvTranspose / Einsum / MaxPool / Flatten) through a backend.

A backend is any object with the methods gemm_f32, relu_f32, conv2d_f32, conv_transpose2d_f32, einsum_f32 and maxpool2d
(pool3d for pooling over three axes) taking and returning numpy arrays: the CPU oracle module, or the HIP library wrapper.
The attribute handling restates what the reference's operators do at Initialize time.
"""
import numpy as np


def conv_pads(attrs, kshape, in_hw, strides, dilations):
    """Pads (top, left, bottom, right) of a Conv node as this build's emitter resolves them.

    Absent pads with auto_pad NOTSET mean 1 on every side, the reference's rule (ROperator_Conv.hxx:136-139).
    SAME_UPPER / SAME_LOWER are ONNX's: the total that makes the output ceil(in / stride), the odd unit at the
    end / at the begin (the reference's own rule, :140-158, declares an output larger than its code writes).
    Begin and end pads that differ are kept (the reference averages them, :387-401).
    """
    auto = attrs.get("auto_pad", "NOTSET")
    pads = list(attrs.get("pads", []))
    if auto == "NOTSET":
        if not pads:
            pads = [1, 1, 1, 1]
    elif auto in ("SAME_UPPER", "SAME_LOWER"):
        pads = [0, 0, 0, 0]
        for i in range(2):
            extent = dilations[i] * (kshape[i] - 1) + 1
            covered = (-(-in_hw[i] // strides[i]) - 1) * strides[i] + extent
            total = max(covered - in_hw[i], 0)
            small, large = total // 2, total - total // 2
            pads[i], pads[2 + i] = (small, large) if auto == "SAME_UPPER" else (large, small)
    elif auto == "VALID":
        pads = [0, 0, 0, 0]
    else:
        raise RuntimeError("TMVA SOFIE Conv Op invalid fAutopad")
    return tuple(pads)


def run_graph(graph, feeds, backend):
    """Evaluate the nodes in file order; returns the first graph output as numpy."""
    env = dict(graph["initializers"])
    env.update(feeds)
    for node in graph["nodes"]:
        op, a, ins = node["op_type"], node["attrs"], node["inputs"]
        if op == "Gemm":
            bias = env[ins[2]] if len(ins) > 2 else None
            y = backend.gemm_f32(env[ins[0]], env[ins[1]], bias, alpha=a.get("alpha", 1.0),
                                 beta=a.get("beta", 1.0) if bias is not None else 0.0,
                                 transA=bool(a.get("transA", 0)), transB=bool(a.get("transB", 0)))
        elif op == "Relu":
            y = backend.relu_f32(env[ins[0]])
        elif op == "Conv":
            w = env[ins[1]]
            strides = tuple(a.get("strides", [1, 1]))
            pads = conv_pads(a, w.shape[2:], env[ins[0]].shape[2:], strides, tuple(a.get("dilations", [1, 1])))
            bias = env[ins[2]] if len(ins) > 2 else None
            y = backend.conv2d_f32(env[ins[0]], w, bias, pads=pads,
                                   strides=strides,
                                   dilations=tuple(a.get("dilations", [1, 1])),
                                   groups=a.get("group", 1))
        elif op == "ConvTranspose":
            # ROperator_ConvTranspose.icc:14-103: strides / dilations default to 1, pads and output_padding to 0;
            # begin/end pads that differ are kept as they are (the reference averages them for the scatter, :318-346,
            # while the output keeps the size the shape rule gave it). A 1-D operator runs as a 2-D one with a height of one.
            x, w = env[ins[0]], env[ins[1]]
            dim = x.ndim - 2
            strides = list(a.get("strides", [1] * dim))
            dil = list(a.get("dilations", [1] * dim))
            pads = list(a.get("pads", [0] * (2 * dim)))
            opad = list(a.get("output_padding", [0] * dim))
            out = [strides[i] * (x.shape[2 + i] - 1) + dil[i] * (w.shape[2 + i] - 1) + 1 + opad[i] - pads[i] - pads[dim + i]
                   for i in range(dim)]
            begin = [pads[i] for i in range(dim)]
            if dim == 1:
                x, w = x[:, :, None, :], w[:, :, None, :]
                strides, dil, begin, out = [1] + strides, [1] + dil, [0] + begin, [1] + out
            # hand the backend pads whose end part reproduces the output size of the shape rule
            full = [strides[i] * (x.shape[2 + i] - 1) + dil[i] * (w.shape[2 + i] - 1) + 1 for i in range(2)]
            end = [full[i] - begin[i] - out[i] for i in range(2)]
            extra = [max(0, -e) for e in end]
            end = [max(0, e) for e in end]
            bias = env[ins[2]] if len(ins) > 2 else None
            y = backend.conv_transpose2d_f32(x, w, bias, pads=(begin[0], begin[1], end[0], end[1]), strides=tuple(strides),
                                             dilations=tuple(dil), groups=max(1, a.get("group", 1)),
                                             output_padding=tuple(extra))
            if dim == 1:
                y = y[:, :, 0, :]
        elif op == "Einsum":
            eq = a["equation"]
            y = backend.einsum_f32(eq.decode() if isinstance(eq, bytes) else eq, [env[i] for i in ins])
        elif op in ("MaxPool", "AveragePool"):
            # one spatial axis runs as two with a height of one, three through the backend's pool3d
            x = env[ins[0]]
            dim = x.ndim - 2
            k = tuple(a["kernel_shape"])
            st = tuple(a.get("strides", [1] * dim))
            pads = tuple(a.get("pads", [0] * (2 * dim)))
            include = bool(a.get("count_include_pad", 0))
            if dim == 3:
                y = backend.pool3d(x, k, st, pads, average=op == "AveragePool", count_include_pad=include)
            else:
                if dim == 1:
                    x, k, st, pads = x[:, :, None, :], (1,) + k, (1,) + st, (0, pads[0], 0, pads[1])
                y = backend.maxpool2d(x, k, st, pads) if op == "MaxPool" else backend.avgpool2d(x, k, st, pads, include)
                if dim == 1:
                    y = y[:, :, 0, :]
        elif op == "GlobalAveragePool":
            x = env[ins[0]]
            y = backend.avgpool2d(x, tuple(x.shape[2:]), (1, 1))
        elif op == "Flatten":
            x = env[ins[0]]
            y = np.ascontiguousarray(x).reshape(x.shape[0], -1)
        else:
            raise NotImplementedError(op)
        env[node["outputs"][0]] = y
    return env[graph["outputs"][0][0]]


def fixture_feeds(entry, graph):
    """{graph input name: array} for a fixture entry."""
    if entry["input_kind"] == "literals":
        return {name: np.array(vals, np.float32).reshape(shape)
                for (name, _, shape), vals in zip(graph["inputs"], entry["inputs"])}
    return {graph["inputs"][0][0]: fixture_input(entry)}


def fixture_input(entry):
    shape = entry["input_shape"]
    n = int(np.prod(shape))
    kind = entry["input_kind"]
    if kind == "ones":
        x = np.ones(n, np.float32)
    elif kind == "iota":
        x = np.arange(n, dtype=np.float32)
    else:
        x = np.array(entry["input"], np.float32)
    return x.reshape(shape)
