"""Seeded writers for the ONNX graphs of the benchmark configurations.

No `onnx` package is needed: a small protobuf encoder/decoder for the handful of ONNX
messages the descriptor runner reads (field numbers of the reference's scripts/onnx.proto:
ModelProto:357-400, GraphProto:456-477, NodeProto:208-224, AttributeProto:122-185,
TensorProto:499-618).  Weights are random-initialised from numpy's default_rng with a seed
per tensor, so the same bytes are produced on every machine.

Graphs (the shapes follow example/benchmark/make_models.py:142-162 of the reference and the
five benchmark configurations):
    gemm_model      Gemm A[M,K] . B[N,K]^T + C[N]
    ffn_model       MatMul -> Add -> Relu -> MatMul -> Add(residual)
    conv_model      Conv 3x3 -> Relu
    resnet50_model  ResNet-50 v1 with BatchNorm folded into the conv bias
    detr_model      DETR-R50-style detector: ResNet-50 trunk, 1x1 projection, 6+6 transformer layers
"""
import struct

import numpy as np

FLOAT, INT32, INT64 = 1, 6, 7
ATTR_FLOAT, ATTR_INT, ATTR_STRING, ATTR_TENSOR, ATTR_FLOATS, ATTR_INTS = 1, 2, 3, 4, 6, 7


# ------------------------------------------------------------------ protobuf wire format
def _varint(v):
    if v < 0:
        v += 1 << 64
    out = bytearray()
    while v > 0x7F:
        out.append((v & 0x7F) | 0x80)
        v >>= 7
    out.append(v)
    return bytes(out)


def _tag(field, wire):
    return _varint(field << 3 | wire)


def _len(field, payload):
    return _tag(field, 2) + _varint(len(payload)) + payload


def _int(field, v):
    return _tag(field, 0) + _varint(int(v))


def _str(field, s):
    return _len(field, s.encode("utf-8"))


def _packed_ints(field, values):
    return _len(field, b"".join(_varint(int(v)) for v in values)) if len(values) else b""


def tensor_proto(name, array):
    array = np.asarray(array)
    if array.dtype == np.float32:
        dt = FLOAT
    elif array.dtype == np.int64:
        dt = INT64
    elif array.dtype == np.int32:
        dt = INT32
    else:
        raise TypeError("unsupported initializer dtype %s" % array.dtype)
    return (_packed_ints(1, array.shape) + _int(2, dt) + _str(8, name)
            + _len(9, np.ascontiguousarray(array).tobytes()))


def attribute(name, value):
    out = _str(1, name)
    if isinstance(value, float):
        return out + _tag(2, 5) + struct.pack("<f", value) + _int(20, ATTR_FLOAT)
    if isinstance(value, (int, np.integer)):
        return out + _int(3, value) + _int(20, ATTR_INT)
    if isinstance(value, str):
        return out + _len(4, value.encode("utf-8")) + _int(20, ATTR_STRING)
    if isinstance(value, (list, tuple)):
        return out + _packed_ints(8, value) + _int(20, ATTR_INTS)
    if isinstance(value, np.ndarray):
        return out + _len(5, tensor_proto("", value)) + _int(20, ATTR_TENSOR)
    raise TypeError("unsupported attribute %r" % (value,))


def node(op_type, inputs, outputs, name, **attrs):
    out = b"".join(_str(1, i) for i in inputs) + b"".join(_str(2, o) for o in outputs)
    out += _str(3, name) + _str(4, op_type)
    out += b"".join(_len(5, attribute(k, v)) for k, v in attrs.items())
    return out


def value_info(name, shape, elem_type=FLOAT):
    dims = b"".join(_len(1, _int(1, d)) for d in shape)
    tensor_type = _int(1, elem_type) + _len(2, dims)
    return _str(1, name) + _len(2, _len(1, tensor_type))


def model_proto(nodes, initializers, inputs, outputs, opset=13, graph_name="graph", metadata=None):
    graph = b"".join(_len(1, n) for n in nodes) + _str(2, graph_name)
    graph += b"".join(_len(5, t) for t in initializers)
    graph += b"".join(_len(11, v) for v in inputs) + b"".join(_len(12, v) for v in outputs)
    out = _int(1, 7) + _str(2, "webdnn_amd.modelgen") + _len(7, graph)
    out += _len(8, _str(1, "") + _int(2, opset))
    for key, value in (metadata or {}).items():
        out += _len(14, _str(1, key) + _str(2, value))
    return out


# ------------------------------------------------------------------ reader (for the Python graph checker)
def _read_varint(buf, pos):
    result, shift = 0, 0
    while True:
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7


def _fields(buf):
    pos, end = 0, len(buf)
    while pos < end:
        key, pos = _read_varint(buf, pos)
        field, wire = key >> 3, key & 7
        if wire == 0:
            v, pos = _read_varint(buf, pos)
        elif wire == 2:
            n, pos = _read_varint(buf, pos)
            v = buf[pos:pos + n]
            pos += n
        elif wire == 5:
            v = buf[pos:pos + 4]
            pos += 4
        elif wire == 1:
            v = buf[pos:pos + 8]
            pos += 8
        else:
            raise ValueError("wire type %d" % wire)
        yield field, wire, v


def _signed(v):
    return v - (1 << 64) if v >= 1 << 63 else v


def _ints(wire, v):
    if wire == 0:
        return [_signed(v)]
    out, pos = [], 0
    while pos < len(v):
        x, pos = _read_varint(v, pos)
        out.append(_signed(x))
    return out


def parse_model(data):
    """-> dict(opset, nodes=[dict(op_type, name, inputs, outputs, attrs)], initializers={name: array},
    inputs=[(name, shape)], outputs=[(name, shape)])."""
    data = memoryview(data)
    model = {"opset": None, "nodes": [], "initializers": {}, "inputs": [], "outputs": [], "metadata": {}}

    def parse_tensor(buf):
        dims, dt, name, raw = [], None, "", b""
        for f, w, v in _fields(buf):
            if f == 1:
                dims += _ints(w, v)
            elif f == 2:
                dt = v
            elif f == 8:
                name = bytes(v).decode()
            elif f == 9:
                raw = bytes(v)
        np_dt = {FLOAT: np.float32, INT64: np.int64, INT32: np.int32}[dt]
        return name, np.frombuffer(raw, dtype=np_dt).reshape(dims).copy()

    def parse_attr(buf):
        name, value = "", None
        for f, w, v in _fields(buf):
            if f == 1:
                name = bytes(v).decode()
            elif f == 2:
                value = struct.unpack("<f", bytes(v))[0]
            elif f == 3:
                value = _signed(v)
            elif f == 4:
                value = bytes(v).decode()
            elif f == 5:
                value = parse_tensor(v)[1]
            elif f == 8:
                value = (value or []) + _ints(w, v)
        return name, value

    def parse_node(buf):
        n = {"op_type": "", "name": "", "inputs": [], "outputs": [], "attrs": {}}
        for f, w, v in _fields(buf):
            if f == 1:
                n["inputs"].append(bytes(v).decode())
            elif f == 2:
                n["outputs"].append(bytes(v).decode())
            elif f == 3:
                n["name"] = bytes(v).decode()
            elif f == 4:
                n["op_type"] = bytes(v).decode()
            elif f == 5:
                k, val = parse_attr(v)
                n["attrs"][k] = val
        return n

    def parse_value_info(buf):
        name, shape = "", []
        for f, w, v in _fields(buf):
            if f == 1:
                name = bytes(v).decode()
            elif f == 2:
                for f2, _, v2 in _fields(v):            # TypeProto.tensor_type
                    if f2 == 1:
                        for f3, _, v3 in _fields(v2):    # Tensor: elem_type, shape
                            if f3 == 2:
                                for f4, _, v4 in _fields(v3):      # dim
                                    for f5, _, v5 in _fields(v4):  # dim_value
                                        if f5 == 1:
                                            shape.append(v5)
        return name, shape

    for f, w, v in _fields(data):
        if f == 7:
            for gf, gw, gv in _fields(v):
                if gf == 1:
                    model["nodes"].append(parse_node(gv))
                elif gf == 5:
                    name, arr = parse_tensor(gv)
                    model["initializers"][name] = arr
                elif gf == 11:
                    model["inputs"].append(parse_value_info(gv))
                elif gf == 12:
                    model["outputs"].append(parse_value_info(gv))
        elif f == 8 and model["opset"] is None:
            for of, ow, ov in _fields(v):
                if of == 2:
                    model["opset"] = ov
        elif f == 14:
            kv = {}
            for mf, mw, mv in _fields(v):
                kv[mf] = bytes(mv).decode()
            model["metadata"][kv.get(1, "")] = kv.get(2, "")
    model["inputs"] = [(n, s) for n, s in model["inputs"] if n not in model["initializers"]]
    return model


# ------------------------------------------------------------------ graph builders
class GraphBuilder:
    def __init__(self, seed=0):
        self.nodes, self.initializers, self.counter = [], [], 0
        self.seed = seed
        self.flops = 0          # 2*M*N*K of every Gemm / MatMul / Conv
        # What the hip library's default plan saves of that on the matrix cores: its 3x3 stride-1 convs with
        # at least 128 input and output channels run as F(2x2, 3x3), 16 products per 2x2 output block in place
        # of 36 (flops - flops_saved is what the matrix cores execute; the transforms run on the vector units).
        self.flops_saved = 0
        self.conv_gemm_nodes = 0

    def rng(self):
        self.counter += 1
        return np.random.default_rng([self.seed, self.counter])

    def const(self, name, array):
        self.initializers.append(tensor_proto(name, array))
        return name

    def op(self, op_type, inputs, output, **attrs):
        """`output` is one tensor name, or a list of them for a multi-output operator (Split)."""
        outputs = list(output) if isinstance(output, (list, tuple)) else [output]
        self.nodes.append(node(op_type, inputs, outputs, "%s_%d" % (op_type, len(self.nodes)), **attrs))
        return output

    def finish(self, inputs, outputs, opset=13):
        return model_proto(self.nodes, self.initializers, [value_info(n, s) for n, s in inputs],
                           [value_info(n, s) for n, s in outputs], opset)


def gemm_model(m=256, k=512, n=1024, seed=0):
    """Config 1: A[m,k] (input), B[n,k] transB=1, C[n]; uniform[-1,1]."""
    g = GraphBuilder(seed)
    g.const("B", g.rng().uniform(-1, 1, (n, k)).astype(np.float32))
    g.const("C", g.rng().uniform(-1, 1, (n,)).astype(np.float32))
    g.op("Gemm", ["A", "B", "C"], "Y", alpha=1.0, beta=1.0, transB=1)
    g.flops = 2 * m * n * k
    return g.finish([("A", [m, k])], [("Y", [m, n])]), g


def ffn_model(batch=8, seq=512, d=768, hidden=3072, seed=0):
    """Config 2: X -> MatMul W1 -> Add b1 -> Relu -> MatMul W2 -> Add X."""
    g = GraphBuilder(seed)
    g.const("W1", (g.rng().standard_normal((d, hidden)) * 0.02).astype(np.float32))
    g.const("b1", np.zeros(hidden, np.float32))
    g.const("W2", (g.rng().standard_normal((hidden, d)) * 0.02).astype(np.float32))
    g.op("MatMul", ["X", "W1"], "h")
    g.op("Add", ["h", "b1"], "hb")
    g.op("Relu", ["hb"], "hr")
    g.op("MatMul", ["hr", "W2"], "y")
    g.op("Add", ["y", "X"], "out")
    g.flops = 2 * 2 * batch * seq * d * hidden
    return g.finish([("X", [batch, seq, d])], [("out", [batch, seq, d])]), g


def conv_model(batch=32, cin=64, hw=56, cout=64, k=3, seed=0):
    """Config 3: Conv 3x3 pad 1 (He-normal weights, zero bias) -> Relu."""
    g = GraphBuilder(seed)
    g.const("W", (g.rng().standard_normal((cout, cin, k, k)) * np.sqrt(2.0 / (cin * k * k))).astype(np.float32))
    g.const("B", np.zeros(cout, np.float32))
    p = k // 2
    g.op("Conv", ["X", "W", "B"], "c", kernel_shape=[k, k], pads=[p, p, p, p], strides=[1, 1], dilations=[1, 1], group=1)
    g.op("Relu", ["c"], "Y")
    g.flops = 2 * batch * hw * hw * cout * cin * k * k
    return g.finish([("X", [batch, cin, hw, hw])], [("Y", [batch, cout, hw, hw])]), g


def resnet50_model(batch=32, image=224, classes=1000, seed=0, width=64, blocks=(3, 4, 6, 3)):
    """Config 4: ResNet-50 v1 (stride on the first 1x1 of a stage's first block, as in the original
    architecture), He-normal conv weights, BatchNorm folded into the conv bias with gamma=1, beta=0,
    mean=0, var=1 and eps dropped (scale exactly 1, bias exactly 0), FC weights N(0, 0.01).
    Nodes: Conv, Relu, Add, MaxPool, GlobalAveragePool, Flatten, Gemm."""
    g = GraphBuilder(seed)
    x, cin = _resnet_trunk(g, "input", batch, [image, image], width, blocks, init="he")
    x = g.op("GlobalAveragePool", [x], "gap")
    x = g.op("Flatten", [x], "flat", axis=1)
    g.const("fc_w", (g.rng().standard_normal((classes, cin)) * 0.01).astype(np.float32))
    g.const("fc_b", np.zeros(classes, np.float32))
    g.op("Gemm", [x, "fc_w", "fc_b"], "logits", alpha=1.0, beta=1.0, transB=1)
    g.flops += 2 * batch * classes * cin
    g.conv_gemm_nodes += 1
    return g.finish([("input", [batch, 3, image, image])], [("logits", [batch, classes])]), g


def _resnet_trunk(g, x, batch, size, width=64, blocks=(3, 4, 6, 3), init="he"):
    """ResNet-50 v1 trunk up to the last stage (no pooling head).  `size` = [h, w], updated in place.
    Returns (tensor name, channels)."""

    def conv(x, cin, cout, k, stride, pad, relu, name):
        fan_in, fan_out = cin * k * k, cout * k * k
        if init == "he":
            w = g.rng().standard_normal((cout, cin, k, k)) * np.sqrt(2.0 / fan_in)
        else:  # Xavier-uniform
            a = np.sqrt(6.0 / (fan_in + fan_out))
            w = g.rng().uniform(-a, a, (cout, cin, k, k))
        g.const(name + "_w", w.astype(np.float32))
        g.const(name + "_b", np.zeros(cout, np.float32))
        oh = (size[0] + 2 * pad - k) // stride + 1
        ow = (size[1] + 2 * pad - k) // stride + 1
        g.flops += 2 * batch * oh * ow * cout * cin * k * k
        if k == 3 and stride == 1 and cin >= 128 and cout >= 128 and cin % 16 == 0:
            blocks = (batch * ((oh + 1) // 2) * ((ow + 1) // 2) + 15) // 16 * 16
            g.flops_saved += 2 * batch * oh * ow * cout * cin * 9 - 2 * blocks * cout * cin * 16
        g.conv_gemm_nodes += 1
        y = g.op("Conv", [x, name + "_w", name + "_b"], name, kernel_shape=[k, k], pads=[pad] * 4,
                 strides=[stride, stride], dilations=[1, 1], group=1)
        size[0], size[1] = oh, ow
        return g.op("Relu", [y], name + "_relu") if relu else y

    x = conv(x, 3, width, 7, 2, 3, True, "stem")
    x = g.op("MaxPool", [x], "pool", kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[2, 2])
    size[0], size[1] = (size[0] + 2 - 3) // 2 + 1, (size[1] + 2 - 3) // 2 + 1
    cin = width
    for stage, nblocks in enumerate(blocks):
        mid, cout = width * 2 ** stage, width * 4 * 2 ** stage
        for b in range(nblocks):
            stride = 2 if (stage > 0 and b == 0) else 1
            name = "s%db%d" % (stage + 1, b)
            size_in = list(size)
            y = conv(x, cin, mid, 1, stride, 0, True, name + "_c1")
            y = conv(y, mid, mid, 3, 1, 1, True, name + "_c2")
            y = conv(y, mid, cout, 1, 1, 0, False, name + "_c3")
            size_out = list(size)
            if b == 0:
                size[0], size[1] = size_in
                shortcut = conv(x, cin, cout, 1, stride, 0, False, name + "_ds")
                size[0], size[1] = size_out
            else:
                shortcut = x
            x = g.op("Relu", [g.op("Add", [y, shortcut], name + "_add")], name + "_out")
            cin = cout
    return x, cin


def detr_model(image=(800, 1088), d=256, heads=8, ffn=2048, enc_layers=6, dec_layers=6, queries=100,
               classes=92, seed=0, width=64, blocks=(3, 4, 6, 3)):
    """Config 5: DETR-R50-style graph, batch 1.  ResNet-50 trunk -> 1x1 Conv to d -> tokens [T, d] with a
    sinusoidal position encoding -> post-norm transformer (8-head attention as MatMul/Softmax,
    LayerNormalization, FFN) -> class head Gemm [d, classes] and box MLP [d, d, 4] with Sigmoid.
    Xavier-uniform weights, zero biases, learned queries ~N(0,1).  Every MatMul is rank <= 3 (the batch of
    one is dropped), heads are split with Reshape + Transpose, opset 17 (LayerNormalization)."""
    g = GraphBuilder(seed)
    size = [image[0], image[1]]
    x, cin = _resnet_trunk(g, "input", 1, size, width, blocks, init="xavier")
    h, w = size
    tokens = h * w
    hd = d // heads

    def xavier(name, shape):
        a = np.sqrt(6.0 / (shape[0] + shape[1]))
        return g.const(name, g.rng().uniform(-a, a, shape).astype(np.float32))

    def zeros(name, n):
        return g.const(name, np.zeros(n, np.float32))

    def shape(name, dims):
        return g.const(name, np.array(dims, np.int64))

    def linear(xn, rows, din, dout, name, relu=False):
        xavier(name + "_w", (din, dout))
        zeros(name + "_b", dout)
        g.flops += 2 * rows * din * dout
        g.conv_gemm_nodes += 1
        y = g.op("Add", [g.op("MatMul", [xn, name + "_w"], name + "_mm"), name + "_b"], name + "_lin")
        return g.op("Relu", [y], name + "_relu") if relu else y

    def layernorm(xn, name):
        g.const(name + "_g", np.ones(d, np.float32))
        zeros(name + "_beta", d)
        return g.op("LayerNormalization", [xn, name + "_g", name + "_beta"], name, axis=-1, epsilon=1e-5)

    def attention(q_in, k_in, v_in, tq, tk, name):
        q = linear(q_in, tq, d, d, name + "_q")
        k = linear(k_in, tk, d, d, name + "_k")
        v = linear(v_in, tk, d, d, name + "_v")
        shape(name + "_sq", [tq, heads, hd])
        shape(name + "_sk", [tk, heads, hd])
        shape(name + "_so", [tq, d])
        qh = g.op("Transpose", [g.op("Reshape", [q, name + "_sq"], name + "_q3")], name + "_qh", perm=[1, 0, 2])
        kt = g.op("Transpose", [g.op("Reshape", [k, name + "_sk"], name + "_k3")], name + "_kt", perm=[1, 2, 0])
        vh = g.op("Transpose", [g.op("Reshape", [v, name + "_sk"], name + "_v3")], name + "_vh", perm=[1, 0, 2])
        g.const(name + "_scale", np.array(1.0 / np.sqrt(hd), np.float32))
        scores = g.op("MatMul", [qh, kt], name + "_scores")
        attn = g.op("Softmax", [g.op("Mul", [scores, name + "_scale"], name + "_scaled")], name + "_attn", axis=-1)
        ctx = g.op("MatMul", [attn, vh], name + "_ctx")
        g.flops += 2 * 2 * heads * tq * tk * hd
        g.conv_gemm_nodes += 2
        merged = g.op("Reshape", [g.op("Transpose", [ctx], name + "_ctx_t", perm=[1, 0, 2]), name + "_so"], name + "_merged")
        return linear(merged, tq, d, d, name + "_o")

    # 1x1 projection and flattening to tokens
    a = np.sqrt(6.0 / (cin + d))
    g.const("proj_w", g.rng().uniform(-a, a, (d, cin, 1, 1)).astype(np.float32))
    zeros("proj_b", d)
    g.flops += 2 * tokens * d * cin
    g.conv_gemm_nodes += 1
    p = g.op("Conv", [x, "proj_w", "proj_b"], "proj", kernel_shape=[1, 1], pads=[0, 0, 0, 0], strides=[1, 1],
             dilations=[1, 1], group=1)
    shape("tok_shape", [d, tokens])
    src = g.op("Transpose", [g.op("Reshape", [p, "tok_shape"], "proj_flat")], "src0", perm=[1, 0])
    # sinusoidal position encoding over (y, x), d/2 channels each
    half = d // 2
    dim_t = 10000.0 ** (2 * (np.arange(half) // 2) / half)
    ys, xs = np.meshgrid(np.arange(1, h + 1), np.arange(1, w + 1), indexing="ij")
    scale = 2 * np.pi
    py = (ys / (h + 1e-6) * scale)[..., None] / dim_t
    px = (xs / (w + 1e-6) * scale)[..., None] / dim_t
    enc = lambda t: np.stack([np.sin(t[..., 0::2]), np.cos(t[..., 1::2])], axis=-1).reshape(h, w, half)
    g.const("pos", np.concatenate([enc(py), enc(px)], axis=-1).reshape(tokens, d).astype(np.float32))

    for i in range(enc_layers):
        n = "enc%d" % i
        qk = g.op("Add", [src, "pos"], n + "_qk")
        sa = attention(qk, qk, src, tokens, tokens, n + "_sa")
        src = layernorm(g.op("Add", [src, sa], n + "_res1"), n + "_ln1")
        f = linear(linear(src, tokens, d, ffn, n + "_f1", relu=True), tokens, ffn, d, n + "_f2")
        src = layernorm(g.op("Add", [src, f], n + "_res2"), n + "_ln2")
    memory = src
    mem_k = g.op("Add", [memory, "pos"], "mem_k")

    g.const("query_pos", g.rng().standard_normal((queries, d)).astype(np.float32))
    tgt = g.const("tgt0", np.zeros((queries, d), np.float32))
    for i in range(dec_layers):
        n = "dec%d" % i
        qk = g.op("Add", [tgt, "query_pos"], n + "_qk")
        sa = attention(qk, qk, tgt, queries, queries, n + "_sa")
        tgt = layernorm(g.op("Add", [tgt, sa], n + "_res1"), n + "_ln1")
        q = g.op("Add", [tgt, "query_pos"], n + "_q")
        ca = attention(q, mem_k, memory, queries, tokens, n + "_ca")
        tgt = layernorm(g.op("Add", [tgt, ca], n + "_res2"), n + "_ln2")
        f = linear(linear(tgt, queries, d, ffn, n + "_f1", relu=True), queries, ffn, d, n + "_f2")
        tgt = layernorm(g.op("Add", [tgt, f], n + "_res3"), n + "_ln3")
    hs = layernorm(tgt, "dec_norm")

    xavier("class_w", (d, classes))
    zeros("class_b", classes)
    g.flops += 2 * queries * d * classes
    g.op("Gemm", [hs, "class_w", "class_b"], "logits", alpha=1.0, beta=1.0)
    b1 = linear(hs, queries, d, d, "box1", relu=True)
    b2 = linear(b1, queries, d, d, "box2", relu=True)
    b3 = linear(b2, queries, d, 4, "box3")
    g.op("Sigmoid", [b3], "boxes")
    g.conv_gemm_nodes += 1
    data = g.finish([("input", [1, 3, image[0], image[1]])], [("logits", [queries, classes]), ("boxes", [queries, 4])],
                    opset=17)
    return data, g


def glue_model(opset=11, seed=0):
    """Shape arithmetic and layout glue as ONNX exporters emit around attention blocks:
    Shape -> Gather -> Unsqueeze -> Concat -> Reshape on the metadata side, and
    Split / Concat / Slice / Cast / Squeeze / Unsqueeze on the data.  `opset` below 13 puts
    axes/split in attributes, 13 and above passes them as input tensors."""
    g = GraphBuilder(seed)
    as_input = opset >= 13
    i64 = lambda *v: np.array(v, np.int64)

    def unsqueeze(x, axes, out):
        if as_input:
            return g.op("Unsqueeze", [x, g.const(out + "_axes", i64(*axes))], out)
        return g.op("Unsqueeze", [x], out, axes=list(axes))

    def squeeze(x, axes, out):
        if as_input:
            return g.op("Squeeze", [x, g.const(out + "_axes", i64(*axes))], out)
        return g.op("Squeeze", [x], out, axes=list(axes))

    # metadata side: [batch, -1] computed from the input's shape
    g.op("Shape", ["X"], "shape")
    g.op("Gather", ["shape", g.const("zero", np.array(0, np.int64))], "batch", axis=0)
    unsqueeze("batch", [0], "batch1")
    g.op("Constant", [], "minus1", value=i64(-1))
    g.op("Concat", ["batch1", "minus1"], "flat_shape", axis=0)
    g.op("Reshape", ["X", "flat_shape"], "flat")                       # [2, 120]
    # data side
    if as_input:
        g.op("Split", ["flat", g.const("parts", i64(40, 30, 50))], ["a", "b", "c"], axis=1)
    else:
        g.op("Split", ["flat"], ["a", "b", "c"], axis=1, split=[40, 30, 50])
    g.op("Concat", ["c", "a", "b"], "cat", axis=-1)                    # [2, 120], bands rotated
    g.op("Slice", ["cat", g.const("st", i64(1)), g.const("en", i64(-1)), g.const("ax", i64(1)),
                   g.const("sp", i64(2))], "sl")                       # [2, 59]
    g.op("Mul", ["sl", g.const("hundred", np.array(100.0, np.float32))], "scaled")
    g.op("Cast", ["scaled"], "ints", to=INT32)
    g.op("Cast", ["ints"], "floats", to=FLOAT)
    unsqueeze("floats", [0, 3], "u")                                   # [1, 2, 59, 1]
    squeeze("u", [3], "s")                                             # [1, 2, 59]
    g.op("Slice", ["s", g.const("st2", i64(-1, 58)), g.const("en2", i64(-100, -100)),
                   g.const("ax2", i64(1, 2)), g.const("sp2", i64(-1, -3))], "rev")   # [1, 2, 20]
    g.op("Add", ["rev", g.const("bias", g.rng().standard_normal(20).astype(np.float32))], "Y")
    return g.finish([("X", [2, 6, 4, 5])], [("Y", [1, 2, 20]), ("ints", [2, 59])], opset), g


# ------------------------------------------------------------------ model surgery for optimized-model directories
def _reencode(field, wire, v):
    if wire == 0:
        return _tag(field, 0) + _varint(v)
    if wire == 2:
        return _len(field, bytes(v))
    return _tag(field, wire) + bytes(v)


def strip_initializers(model_bytes):
    """-> (the model without graph.initializer entries, {name: array} of what was removed)."""
    tensors = parse_model(model_bytes)["initializers"]
    out = b""
    for f, w, v in _fields(memoryview(model_bytes)):
        if f == 7 and w == 2:
            graph = b"".join(_reencode(gf, gw, gv) for gf, gw, gv in _fields(v) if gf != 5)
            out += _len(7, graph)
        else:
            out += _reencode(f, w, v)
    return out, tensors


def add_metadata(model_bytes, metadata):
    """Appends ModelProto.metadata_props entries (key/value strings)."""
    return bytes(model_bytes) + b"".join(_len(14, _str(1, k) + _str(2, v)) for k, v in metadata.items())
