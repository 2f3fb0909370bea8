"use strict";
// Unit tests of the Node.js host (no GPU, no test framework: plain assertions, one JSON
// summary line at the end).  The expectations for CPUTensor, the array helpers and the Relu
// operator are the ones the reference pins in test/unit/cpuTensor.test.ts:5-38,
// test/unit/math.test.ts:29-52 and test/unit/cpuOperator.test.ts:6-20; the registry rules are
// written from core/operatorTable.ts:21-69 and the load() fallbacks from index.ts:42-149.
const assert = require("assert");
const path = require("path");
const fs = require("fs");
const os = require("os");

const JS = path.join(__dirname, "..", "..", "webdnn_amd", "js");
const { CPUTensorImpl } = require(path.join(JS, "backend", "cpu", "cpuTensorImpl"));
const { WebDNNCPUContextImpl } = require(path.join(JS, "backend", "cpu", "cpuContextImpl"));
const { WebDNNHipContextImpl } = require(path.join(JS, "backend", "hip", "hipContextImpl"));
const table = require(path.join(JS, "core", "operatorTable"));
const onnx = require(path.join(JS, "core", "onnxProto"));
const util = require(path.join(JS, "util"));
const opUtil = require(path.join(JS, "operators", "operatorUtil"));
const { fuseForHip, findTensorReleaseTiming, modelTransform } = require(path.join(JS, "core", "modelTransform"));
const Logging = require(path.join(JS, "logging"));
const oracle = require(path.join(__dirname, "..", "..", "oracle", "js", "cpuOperators"));
const fakeNative = require("./fake_native");

const tests = [];
const test = (name, fn) => tests.push([name, fn]);

// ---- CPUTensorImpl (reference vectors) -------------------------------------------------
test("CPUTensor allocates zero-filled data", () => {
  const t = new CPUTensorImpl([2, 3], "float32");
  assert(t.data instanceof Float32Array);
  assert.strictEqual(t.data.length, 6);
  assert.strictEqual(t.length, 6);
  assert.strictEqual(t.ndim, 2);
  assert.deepStrictEqual(Array.from(t.dims), [2, 3]);
  assert.deepStrictEqual(Array.from(t.strides), [3, 1]);
});
test("CPUTensor wraps an external buffer; getValue/setValue; int32", () => {
  const buf = new Float32Array([1, 2, 3, 4, 5, 6]);
  const t = new CPUTensorImpl([2, 3], "float32", buf);
  assert.strictEqual(t.data, buf);
  assert.strictEqual(t.useExternalBuffer, true);
  assert.strictEqual(t.getValue([0, 0]), 1);
  assert.strictEqual(t.getValue([1, 2]), 6);
  t.setValue(99, [1, 1]);
  assert.strictEqual(t.getValue([1, 1]), 99);
  assert.throws(() => t.getValue([1]));
  const i = new CPUTensorImpl([2], "int32");
  assert(i.data instanceof Int32Array);
  assert.strictEqual(i.dataType, "int32");
  const s = new CPUTensorImpl([], "float32");
  assert.strictEqual(s.length, 1);
  assert.deepStrictEqual(s.strides, []);
});
test("array helpers", () => {
  assert.strictEqual(util.arrayProd([2, 3, 4]), 24);
  assert.strictEqual(util.arraySum([2, 3, 4]), 9);
  assert.strictEqual(util.arrayEqual([1, 2], [1, 2]), true);
  assert.strictEqual(util.arrayEqual([1, 2], [1, 3]), false);
  assert.deepStrictEqual(util.arange(3), [0, 1, 2]);
  assert.deepStrictEqual(util.arange(2, 5), [2, 3, 4]);
  assert.deepStrictEqual(util.arange(3, 0, -1), [3, 2, 1]);
  assert.strictEqual(util.clipToInt32(2 ** 40), 2147483647);
  assert.strictEqual(util.clipToInt32(-(2 ** 40)), -2147483648);
  assert.strictEqual(util.clipToInt32(BigInt("9223372036854775807")), 2147483647);
});
test("Relu entry: the reference's vector", async () => {
  const ctx = new WebDNNCPUContextImpl();
  await ctx.initialize();
  const entry = oracle.getOpEntries().find((e) => e.opType === "Relu");
  assert(entry);
  const relu = entry.factory();
  const input = new CPUTensorImpl([5], "float32", new Float32Array([-2, -0.5, 0, 1, 3]));
  const [output] = await relu.run(ctx, [input]);
  assert.deepStrictEqual(Array.from(output.data), [0, 0, 0, 1, 3]);
  assert.deepStrictEqual(Array.from(output.dims), [5]);
});

// ---- broadcasting ---------------------------------------------------------------------
test("broadcastUni / broadcastMulti", () => {
  assert.deepStrictEqual(opUtil.broadcastUni([4, 5], [5]), [0, 1]);
  assert.deepStrictEqual(opUtil.broadcastUni([4, 5], [4, 1]), [1, 0]);
  assert.deepStrictEqual(opUtil.broadcastUni([4, 5], []), [0, 0]);
  assert.throws(() => opUtil.broadcastUni([4, 5], [3]), /Unidirectional/);
  assert.throws(() => opUtil.broadcastUni([5], [1, 5]), /Unidirectional/);
  const r = opUtil.broadcastMulti([[2, 3, 10, 12], [1, 3, 1, 12]]);
  assert.deepStrictEqual(r.dims, [2, 3, 10, 12]);
  assert.deepStrictEqual(r.allStrides, [[360, 120, 12, 1], [0, 12, 0, 1]]);
  assert.throws(() => opUtil.broadcastMulti([[2, 3], [4]]), /Multidirectional/);
});

// ---- operator registry -----------------------------------------------------------------
function entry(opType, backend, opsetMin, opsetMax, tag) {
  return { opType, backend, opsetMin, opsetMax, factory: () => ({ backend, tag }) };
}
test("registry: first backend in order that has an entry in the opset window", () => {
  table.clearOperators();
  table.registerOperators([
    entry("Foo", "cpu", 1, undefined, "cpu-any"),
    entry("Foo", "hip", 7, 13, "hip-7-12"),
    entry("Foo", "hip", 13, undefined, "hip-13+"),
  ]);
  assert.strictEqual(table.instantiateOperator("Foo", 9, ["hip", "cpu"], [["cpu"]]).tag, "hip-7-12");
  assert.strictEqual(table.instantiateOperator("Foo", 13, ["hip", "cpu"], [["cpu"]]).tag, "hip-13+"); // max is exclusive
  assert.strictEqual(table.instantiateOperator("Foo", 6, ["hip", "cpu"], [["cpu"]]).tag, "cpu-any");  // below hip's min
  assert.strictEqual(table.instantiateOperator("Foo", 9, ["cpu"], [["cpu"]]).tag, "cpu-any");
  assert.strictEqual(table.instantiateOperator("Bar", 9, ["hip", "cpu"], [["cpu"]]), null);
});
test("registry: layout operators run where input 0 lives, last backend in order wins; Shape on cpu", () => {
  table.clearOperators();
  const both = (op) => [entry(op, "cpu", 1, undefined, "cpu"), entry(op, "hip", 1, undefined, "hip")];
  table.registerOperators([].concat(...["Reshape", "Transpose", "Flatten", "Squeeze", "Unsqueeze", "Pad", "Shape", "Relu"].map(both)));
  for (const op of ["Reshape", "Transpose", "Flatten", "Squeeze", "Unsqueeze", "Pad"]) {
    assert.strictEqual(table.instantiateOperator(op, 13, ["hip", "cpu"], [["cpu"]]).tag, "cpu", op);
    assert.strictEqual(table.instantiateOperator(op, 13, ["hip", "cpu"], [["hip"]]).tag, "hip", op);
    // on both: the scan has no early exit, so the last backend of the order wins
    assert.strictEqual(table.instantiateOperator(op, 13, ["hip", "cpu"], [["hip", "cpu"]]).tag, "cpu", op);
  }
  assert.strictEqual(table.instantiateOperator("Shape", 13, ["hip", "cpu"], [["hip"]]).tag, "cpu");
  assert.strictEqual(table.instantiateOperator("Relu", 13, ["hip", "cpu"], [["cpu"]]).tag, "hip");
  table.clearOperators();
});

// ---- ONNX wire format --------------------------------------------------------------------
test("onnx: hand-assembled bytes decode field by field", () => {
  // ModelProto{ ir_version(1)=6, graph(7)=GraphProto{ node(1)=NodeProto{input "x", output "y",
  // name "n0", op_type "Relu", attribute{name "k", i=-3, type INT} }, name(2)="g" },
  // opset_import(8)={version(2)=9} }
  const neg3 = [0xfd, 0xff, 0xff, 0xff, 0xff, 0xff, 0xff, 0xff, 0xff, 0x01];
  const attr = [0x0a, 0x01, 0x6b, 0x18, ...neg3, 0xa0, 0x01, 0x02];
  const node = [0x0a, 0x01, 0x78, 0x12, 0x01, 0x79, 0x1a, 0x02, 0x6e, 0x30, 0x22, 0x04, 0x52, 0x65, 0x6c, 0x75,
    0x2a, attr.length, ...attr];
  const graph = [0x0a, node.length, ...node, 0x12, 0x01, 0x67];
  const bytes = Uint8Array.from([0x08, 0x06, 0x3a, graph.length, ...graph, 0x42, 0x02, 0x10, 0x09]);
  const m = onnx.decodeModel(bytes);
  assert.strictEqual(m.irVersion, 6);
  assert.strictEqual(m.opsetImport[0].version, 9);
  assert.strictEqual(m.graph.name, "g");
  const n = m.graph.node[0];
  assert.deepStrictEqual([n.input, n.output, n.name, n.opType], [["x"], ["y"], "n0", "Relu"]);
  assert.strictEqual(n.attribute[0].name, "k");
  assert.strictEqual(n.attribute[0].i, -3);
  assert.strictEqual(n.attribute[0].type, onnx.AttributeType.INT);
  assert.strictEqual(opUtil.getAttrInt(n.attribute, "k", 0), -3);
  assert.strictEqual(opUtil.getAttrInt(n.attribute, "absent", 7), 7);
  assert.throws(() => opUtil.getAttrFloat(n.attribute, "k", 0), /not float/);
  assert.throws(() => onnx.decodeModel(bytes.subarray(0, 10)), /truncated/);
});
test("onnx: write/read round trip incl. int64 extremes, packed lists, raw and typed tensor data", () => {
  const raw = new Uint8Array(new Float32Array([1.5, -2, 3.25]).buffer);
  const raw64 = new Uint8Array(new BigInt64Array([BigInt(5), BigInt(-1), BigInt("9223372036854775807")]).buffer);
  const model = {
    irVersion: 7,
    opsetImport: [{ domain: "", version: 13 }],
    metadataProps: [{ key: "WebDNN2.TensorMoveOptions", value: "{}" }],
    graph: {
      name: "g",
      node: [{
        input: ["a", "b"], output: ["c"], name: "n", opType: "Conv",
        attribute: [
          { name: "pads", ints: [1, 0, -1, 2147483648 * 4], floats: [], strings: [], type: 7 },
          { name: "alpha", f: 0.5, ints: [], floats: [], strings: [], type: 1 },
          { name: "auto_pad", s: Buffer.from("SAME_UPPER"), ints: [], floats: [], strings: [], type: 3 },
        ],
      }],
      initializer: [
        { dims: [3], dataType: 1, name: "w", rawData: raw, floatData: [], int32Data: [], int64Data: [] },
        { dims: [3], dataType: 7, name: "s", rawData: raw64, floatData: [], int32Data: [], int64Data: [] },
        { dims: [2], dataType: 7, name: "t", int64Data: [-7, 8], floatData: [], int32Data: [] },
        { dims: [2], dataType: 1, name: "u", floatData: [0.25, -0.5], int32Data: [], int64Data: [] },
      ],
      input: [{ name: "a", type: { tensorType: { elemType: 1, shape: { dim: [{ dimValue: 2 }, { dimValue: 3 }] } } } }],
      output: [{ name: "c", type: { tensorType: { elemType: 1, shape: { dim: [{ dimValue: 2 }] } } } }],
      valueInfo: [],
    },
  };
  const back = onnx.decodeModel(onnx.encodeModel(model));
  const a = back.graph.node[0].attribute;
  assert.deepStrictEqual(opUtil.getAttrInts(a, "pads", []), [1, 0, -1, 2147483647]);   // clipped like util.ts:73-81
  assert.strictEqual(opUtil.getAttrFloat(a, "alpha", 1), 0.5);
  assert.strictEqual(opUtil.getAttrString(a, "auto_pad", "NOTSET"), "SAME_UPPER");
  const [w, s, t, u] = back.graph.initializer.map(opUtil.tensorProtoToArray);
  assert.deepStrictEqual(Array.from(w.data), [1.5, -2, 3.25]);
  assert.deepStrictEqual([s.dataType, Array.from(s.data)], ["int32", [5, -1, 2147483647]]);
  assert.deepStrictEqual(Array.from(t.data), [-7, 8]);
  assert.deepStrictEqual(Array.from(u.data), [0.25, -0.5]);
  assert.strictEqual(back.metadataProps[0].key, "WebDNN2.TensorMoveOptions");
  assert.deepStrictEqual(back.graph.input[0].type.tensorType.shape.dim.map((d) => d.dimValue), [2, 3]);
  assert.throws(() => opUtil.tensorProtoToArray({ dims: [1], dataType: 11, rawData: raw }), /Unsupported/);
});

// ---- graph passes ---------------------------------------------------------------------------
function mkNode(opType, input, output, name) {
  return { opType, input, output, name, attribute: [] };
}
function mkModel(nodes, inputs, outputs, initializers) {
  return {
    graph: {
      node: nodes,
      input: inputs.map((name) => ({ name })),
      output: outputs.map((name) => ({ name })),
      initializer: (initializers || []).map(([name, dims]) => ({ name, dims })),
    },
  };
}
test("modelTransform renames duplicate and unnamed nodes", () => {
  Logging.captureToMemory(true);
  const m = mkModel([mkNode("Relu", ["x"], ["a"], "n"), mkNode("Relu", ["a"], ["b"], "n"), mkNode("Relu", ["b"], ["c"], ""), mkNode("Relu", ["c"], ["d"], "")],
    ["x"], ["d"]);
  modelTransform(m, ["cpu"]);
  assert.deepStrictEqual(m.graph.node.map((n) => n.name), ["n", "n_", "unnamed", "unnamed_"]);
  assert.strictEqual(Logging.takeRecords().filter((r) => r.level === "WARN").length, 2);
  Logging.captureToMemory(false);
});
test("findTensorReleaseTiming: last reader frees; inputs, outputs and initializers never", () => {
  const m = mkModel([mkNode("A", ["x", "w"], ["t1"], "a"), mkNode("B", ["t1"], ["t2"], "b"), mkNode("C", ["t1", "t2"], ["y"], "c")],
    ["x"], ["y"]);
  const timing = findTensorReleaseTiming(m, new Set(["w"]));
  assert.deepStrictEqual(Array.from(timing.entries()), [["c", ["t1", "t2"]]]);
});
test("fusion: Conv+Add+Relu, Conv+Relu, MatMul+bias+Relu, MatMul+residual; shared tensors stay", () => {
  const m = mkModel([
    mkNode("Conv", ["x", "w1", "b1"], ["c1"], "conv1"), mkNode("Relu", ["c1"], ["r1"], "relu1"),
    mkNode("Conv", ["r1", "w2"], ["c2"], "conv2"), mkNode("Add", ["x", "c2"], ["s"], "add"), mkNode("Relu", ["s"], ["r2"], "relu2"),
    mkNode("MatMul", ["r2", "w3"], ["m1"], "mm1"), mkNode("Add", ["m1", "bias"], ["m1b"], "addb"), mkNode("Relu", ["m1b"], ["m1r"], "relu3"),
    mkNode("MatMul", ["m1r", "w4"], ["m2"], "mm2"), mkNode("Add", ["m2", "r2"], ["out"], "addr"),
    mkNode("Conv", ["out", "w5"], ["c3"], "conv3"), mkNode("Relu", ["c3"], ["r3"], "relu4"), mkNode("Add", ["r3", "c3"], ["y"], "add2"),
  ], ["x"], ["y"], [["w1", [1]], ["b1", [4]], ["w2", [1]], ["w3", [4, 4]], ["bias", [4]], ["w4", [4, 4]], ["w5", [1]]]);
  assert.strictEqual(fuseForHip(m), 4);
  const got = m.graph.node.map((n) => [n.opType, n.name, n.input.join(","), n.output[0]]);
  assert.deepStrictEqual(got, [
    ["WebDNNHipFusedConv", "relu1", "x,w1,b1", "r1"],
    ["WebDNNHipFusedConv", "relu2", "r1,w2,x", "r2"],
    ["WebDNNHipFusedMatMul", "relu3", "r2,w3,bias", "m1r"],
    ["WebDNNHipFusedMatMul", "addr", "m1r,w4,r2", "out"],
    ["Conv", "conv3", "out,w5", "c3"], ["Relu", "relu4", "c3", "r3"], ["Add", "add2", "r3,c3", "y"],
  ]);
  const attrs = (n) => Object.assign({}, ...n.attribute.map((a) => ({ [a.name]: a.s ? Buffer.from(a.s).toString() : a.i })));
  assert.deepStrictEqual(attrs(m.graph.node[0]), { has_bias: 1, has_residual: 0, activation: "Relu" });
  assert.deepStrictEqual(attrs(m.graph.node[1]), { has_bias: 0, has_residual: 1, activation: "Relu" });
  assert.deepStrictEqual(attrs(m.graph.node[2]), { has_bias: 1, has_residual: 0, activation: "Relu" });
  assert.deepStrictEqual(attrs(m.graph.node[3]), { has_bias: 0, has_residual: 1, activation: "" });
  // a graph output in the middle of a chain blocks the fusion
  const m2 = mkModel([mkNode("Conv", ["x", "w"], ["c"], "conv"), mkNode("Relu", ["c"], ["y"], "relu")], ["x"], ["y", "c"], [["w", [1]]]);
  assert.strictEqual(fuseForHip(m2), 0);
});

// ---- hip tensors over the fake native -----------------------------------------------------------
test("fusion: attention block -- Transposes, scale and head merge ride on the MatMuls; bias then residual", () => {
  const f32init = (name, dims, values) => ({ name, dims, dataType: 1, floatData: values });
  const nd = (opType, input, output, attrs) => ({
    opType, input, output, name: output[0], attribute: (attrs || []),
  });
  const perm = (p) => [{ name: "perm", type: 7, ints: p, floats: [], strings: [] }];
  const model = {
    graph: {
      node: [
        nd("Transpose", ["q3"], ["qh"], perm([1, 0, 2])),
        nd("Transpose", ["k3"], ["kt"], perm([1, 2, 0])),
        nd("Transpose", ["v3"], ["vh"], perm([1, 0, 2])),
        nd("MatMul", ["qh", "kt"], ["scores"]),
        nd("Mul", ["scores", "scale"], ["scaled"]),
        nd("Softmax", ["scaled"], ["attn"]),
        nd("MatMul", ["attn", "vh"], ["ctx"]),
        nd("Transpose", ["ctx"], ["ctx_t"], perm([1, 0, 2])),
        nd("Reshape", ["ctx_t", "shape"], ["merged"]),
        nd("MatMul", ["merged", "w"], ["o_mm"]),
        nd("Add", ["o_mm", "b"], ["o_lin"]),
        nd("Add", ["src", "o_lin"], ["res"]),
        nd("Transpose", ["res"], ["res_t"], perm([1, 0])), // rank 2: stays a node
        nd("MatMul", ["res_t", "w2"], ["out"]),
      ],
      initializer: [f32init("scale", [], [0.125]), f32init("b", [4], [0, 0, 0, 0]), f32init("w", [4, 4], new Array(16).fill(1)),
        f32init("w2", [4, 4], new Array(16).fill(1))],
      input: [], output: [{ name: "out" }],
    },
  };
  const unfused = JSON.parse(JSON.stringify(model));
  assert.strictEqual(fuseForHip(model), 4);
  const ops = model.graph.node.map((n) => n.opType);
  assert.deepStrictEqual(ops, ["WebDNNHipAttention", "Reshape", "WebDNNHipFusedMatMul", "Transpose", "MatMul"]);
  const attr = (node, name) => node.attribute.find((a) => a.name === name);
  const [att, , proj] = model.graph.node;
  assert.deepStrictEqual(att.input, ["q3", "k3", "v3"]);
  assert.deepStrictEqual(attr(att, "perm_q").ints, [1, 0, 2]);
  assert.deepStrictEqual(attr(att, "perm_k").ints, [1, 2, 0]);
  assert.deepStrictEqual(attr(att, "perm_v").ints, [1, 0, 2]);
  assert.deepStrictEqual(attr(att, "perm_y").ints, [1, 0, 2]);
  assert.strictEqual(attr(att, "alpha").f, 0.125);
  assert.strictEqual(attr(att, "softmax_axis").i, -1);
  assert.deepStrictEqual(att.output, ["ctx_t"]);
  assert.deepStrictEqual(proj.input, ["merged", "w", "b", "src"]);
  assert.strictEqual(attr(proj, "has_bias").i, 1);
  assert.strictEqual(attr(proj, "has_residual").i, 1);
  assert.deepStrictEqual(proj.output, ["res"]);
  // probabilities that something else reads too (or that leave the graph) keep the three nodes
  const watched = JSON.parse(JSON.stringify(unfused));
  watched.graph.output.push({ name: "attn" });
  assert.strictEqual(fuseForHip(watched), 3);
  assert.deepStrictEqual(watched.graph.node.slice(0, 3).map((n) => n.opType), ["WebDNNHipFusedMatMul", "Softmax", "WebDNNHipFusedMatMul"]);
  const [scores, , ctx] = watched.graph.node;
  assert.deepStrictEqual(scores.input, ["q3", "k3"]);
  assert.deepStrictEqual(attr(scores, "perm_a").ints, [1, 0, 2]);
  assert.deepStrictEqual(attr(scores, "perm_b").ints, [1, 2, 0]);
  assert.strictEqual(attr(scores, "alpha").f, 0.125);
  assert.deepStrictEqual(ctx.input, ["attn", "v3"]);
  assert.deepStrictEqual(attr(ctx, "perm_y").ints, [1, 0, 2]);
  // a Softmax over another axis is no attention
  const other = JSON.parse(JSON.stringify(unfused));
  other.graph.node[5].attribute = [{ name: "axis", type: 2, i: 1, floats: [], ints: [], strings: [] }];
  assert.strictEqual(fuseForHip(other), 3);
  assert.ok(other.graph.node.some((n) => n.opType === "Softmax"));
});

test("fusion: LayerNormalization followed by an Add of an already known tensor becomes one two-output node", () => {
  const { fuseLayerNormAdd } = require("../../webdnn_amd/js/core/modelTransform");
  const nd = (opType, input, output) => ({ opType, input, output, name: output[0], attribute: [] });
  const init = (name) => ({ name, dims: [4], dataType: 1, floatData: [0, 0, 0, 0] });
  const graph = {
    node: [
      nd("LayerNormalization", ["x", "g", "b"], ["n1"]),
      nd("Relu", ["n1"], ["r"]),
      nd("Add", ["n1", "pos"], ["n1p"]),          // pos: initializer -> fused
      nd("Add", ["n1", "pos"], ["again"]),        // a second Add of the same result stays
      nd("LayerNormalization", ["n1p", "g", "b"], ["n2"]),
      nd("Add", ["late", "n2"], ["n2l"]),         // `late` is produced after n2 -> stays
      nd("Relu", ["r"], ["late"]),
      nd("LayerNormalization", ["again", "g", "b"], ["n3"]),
      nd("Add", ["r", "n3"], ["out"]),            // r: an earlier node's output -> fused
    ],
    initializer: [init("g"), init("b"), init("pos")], input: [{ name: "x" }], output: [{ name: "out" }, { name: "n2l" }],
  };
  assert.strictEqual(fuseLayerNormAdd(graph), 2);
  assert.deepStrictEqual(graph.node.map((n) => [n.opType, n.input.join(), n.output.join()]), [
    ["WebDNNHipLayerNormAdd", "x,g,b,pos", "n1,n1p"],
    ["Relu", "n1", "r"],
    ["Add", "n1,pos", "again"],
    ["LayerNormalization", "n1p,g,b", "n2"],
    ["Add", "late,n2", "n2l"],
    ["Relu", "r", "late"],
    ["WebDNNHipLayerNormAdd", "again,g,b,r", "n3,out"],
  ]);
});

test("fusion: neighbouring linear layers that do not read each other become one group node", () => {
  const { groupLinears } = require("../../webdnn_amd/js/core/modelTransform");
  const nd = (opType, input, output, attribute) => ({ opType, input, output, name: output[0], attribute: attribute || [] });
  const fusedAttrs = (bias, act, extra) => [
    { name: "has_bias", i: bias, type: 2, floats: [], ints: [], strings: [] },
    { name: "has_residual", i: 0, type: 2, floats: [], ints: [], strings: [] },
    { name: "activation", s: Buffer.from(act), type: 3, floats: [], ints: [], strings: [] },
  ].concat(extra || []);
  const graph = {
    node: [
      nd("WebDNNHipFusedMatMul", ["x", "wq", "bq"], ["q"], fusedAttrs(1, "")),
      nd("WebDNNHipFusedMatMul", ["x", "wk", "bk"], ["k"], fusedAttrs(1, "")),
      nd("MatMul", ["y", "wv"], ["v"]),
      nd("MatMul", ["q", "wo"], ["o"]),                                               // reads q: starts a new run
      nd("WebDNNHipFusedMatMul", ["y", "w1", "b1"], ["h"], fusedAttrs(1, "Relu")),    // another activation: alone
      nd("Relu", ["o"], ["r"]),
      nd("MatMul", ["r", "w2"], ["a"]),
      nd("WebDNNHipFusedMatMul", ["r", "w3"], ["b"], fusedAttrs(0, "", [{ name: "alpha", f: 0.5, type: 1, floats: [], ints: [], strings: [] }])),
      nd("MatMul", ["r", "w4"], ["c"]),
    ],
    initializer: [], input: [], output: [],
  };
  assert.strictEqual(groupLinears(graph), 1);
  assert.deepStrictEqual(graph.node.map((n) => [n.opType, n.input.join(), n.output.join()]), [
    ["WebDNNHipLinearGroup", "x,wq,bq,x,wk,bk,y,wv", "q,k,v"],
    ["MatMul", "q,wo", "o"],
    ["WebDNNHipFusedMatMul", "y,w1,b1", "h"],
    ["Relu", "o", "r"],
    ["MatMul", "r,w2", "a"],
    ["WebDNNHipFusedMatMul", "r,w3", "b"],
    ["MatMul", "r,w4", "c"],
  ]);
  assert.deepStrictEqual(graph.node[0].attribute.find((a) => a.name === "arity").ints, [3, 3, 2]);
});

test("HipTensor: alias shares one reference-counted buffer; data round trip; use after dispose throws", async () => {
  const cpu = new WebDNNCPUContextImpl();
  const ctx = new WebDNNHipContextImpl(cpu, { native: fakeNative, contractionTile: 3, splitK: 2 });
  await ctx.initialize();
  assert.deepStrictEqual(fakeNative.__options(), { contraction_tile: 3, split_k: 2 });
  const live0 = fakeNative.__liveBuffers();
  const t = ctx.emptyTensor([2, 3], "float32");
  await t.setData(new Float32Array([1, 2, 3, 4, 5, 6]));
  const a = t.alias([3, 2]), b = a.alias([6]);
  assert.strictEqual(a.handle, t.handle);
  assert.deepStrictEqual(b.dims, [6]);
  t.dispose();
  a.dispose();
  assert.strictEqual(fakeNative.__liveBuffers(), live0 + 1);
  assert.deepStrictEqual(Array.from(await b.getData()), [1, 2, 3, 4, 5, 6]);
  b.dispose();
  b.dispose(); // idempotent
  assert.strictEqual(fakeNative.__liveBuffers(), live0);
  assert.throws(() => b.handle, /already disposed/);
  await assert.rejects(() => ctx.emptyTensor([2], "float32").setData(new Float32Array(3)), /length mismatch/);
  assert.throws(() => ctx.emptyTensor([2], "bool"), /not supported/);
  const moved = await ctx.moveTensor(new CPUTensorImpl([2], "int32", new Int32Array([7, -8])), {});
  assert.strictEqual(moved.backend, "hip");
  assert.deepStrictEqual(Array.from(await (await cpu.moveTensor(moved)).getData()), [7, -8]);
  assert.throws(() => ctx.assertsHipTensor(new CPUTensorImpl([1])), /hip is expected/);
});

// ---- load() ----------------------------------------------------------------------------------------
function writeReluModel(dir) {
  const model = {
    irVersion: 7, opsetImport: [{ domain: "", version: 13 }], metadataProps: [],
    graph: {
      name: "g", node: [{ input: ["x"], output: ["y"], name: "r", opType: "Relu", attribute: [] }], initializer: [],
      input: [{ name: "x", type: { tensorType: { elemType: 1, shape: { dim: [{ dimValue: 5 }] } } } }],
      output: [{ name: "y", type: { tensorType: { elemType: 1, shape: { dim: [{ dimValue: 5 }] } } } }],
      valueInfo: [],
    },
  };
  fs.writeFileSync(path.join(dir, "model.onnx"), onnx.encodeModel(model));
}
test("load(): unknown backend throws, empty order has no backend, hip failure falls back to cpu", async () => {
  const WebDNN = require(path.join(JS, "index"));
  const dir = fs.mkdtempSync(path.join(os.tmpdir(), "webdnn_unit_"));
  writeReluModel(dir);
  await assert.rejects(() => WebDNN.load(dir, { backendOrder: ["webgl", "cpu"] }), /Unknown backend webgl/);
  await assert.rejects(() => WebDNN.load(dir, { backendOrder: [] }), /No backend available/);
  // a native whose init() throws, as the addon does on a machine without a GPU
  const dead = Object.assign({}, fakeNative, { init() { throw new Error("wdh_init failed (-1): no HIP device"); } });
  WebDNN.resetDefaultContexts();
  table.clearOperators();
  table.registerOperators(oracle.getOpEntries());
  const runner = await WebDNN.load(dir, { backendOrder: ["hip", "cpu"], backendOptions: { hip: { native: dead } } });
  assert.strictEqual(runner.backendName, "cpu");
  assert.deepStrictEqual(runner.backendOrder, ["cpu"]);
  const [y] = await runner.run([new WebDNN.CPUTensor([5], "float32", new Float32Array([-2, -0.5, 0, 1, 3]))]);
  assert.deepStrictEqual(Array.from(y.data), [0, 0, 0, 1, 3]);
  assert.deepStrictEqual(runner.lastRunStats.nodesByBackend, { cpu: 1 });
  assert.deepStrictEqual(runner.getInputNames(), ["x"]);
  assert.deepStrictEqual(runner.getOutputNames(), ["y"]);
  await assert.rejects(() => runner.run([]), /length of inputs mismatch/);
  // strict: the same failure is an error instead of a fallback
  WebDNN.resetDefaultContexts();
  await assert.rejects(() => WebDNN.load(dir, { backendOrder: ["hip", "cpu"], backendOptions: { hip: { native: dead, strict: true } } }),
    /no HIP device/);
  // a working (fake) hip backend: order becomes [hip, cpu], Relu runs on hip
  WebDNN.resetDefaultContexts();
  const r2 = await WebDNN.load(dir, { backendOrder: ["hip", "cpu"], backendOptions: { hip: { native: fakeNative } } });
  assert.deepStrictEqual(r2.backendOrder, ["hip", "cpu"]);
  const [y2] = await r2.run([new WebDNN.CPUTensor([5], "float32", new Float32Array([-2, -0.5, 0, 1, 3]))]);
  assert.deepStrictEqual(Array.from(y2.data), [0, 0, 0, 1, 3]);
  assert.deepStrictEqual(r2.lastRunStats.nodesByBackend, { hip: 1 });
  fs.rmdirSync(dir, { recursive: true });
});

test("runner: an operator that throws after allocating leaves no device buffer behind", async () => {
  const WebDNN = require(path.join(JS, "index"));
  const dir = fs.mkdtempSync(path.join(os.tmpdir(), "webdnn_unit_"));
  writeReluModel(dir);
  WebDNN.resetDefaultContexts();
  table.clearOperators();
  const runner = await WebDNN.load(dir, { backendOrder: ["hip", "cpu"], backendOptions: { hip: { native: fakeNative, strict: true } } });
  // the Relu entry becomes one that allocates its output and two temporaries, then fails
  // (the first matching entry wins, so the registry is rebuilt around it)
  table.clearOperators();
  table.registerOperators([{
    opType: "Relu", backend: "hip", opsetMin: 1,
    factory: () => ({
      backend: "hip",
      initialize() {},
      getTensorBackendRequirement(nIn) { return new Array(nIn).fill("hip"); },
      async run(context, inputs) {
        context.emptyTensor(inputs[0].dims, "float32");
        const tmp = context.emptyTensor([16], "float32");
        tmp.dispose();
        context.emptyTensor([3], "int32");
        throw new Error("kernel refused");
      },
    }),
  }]);
  const live0 = fakeNative.__liveBuffers();
  const x = new WebDNN.CPUTensor([5], "float32", new Float32Array([-2, -0.5, 0, 1, 3]));
  await assert.rejects(() => runner.run([x]), /kernel refused/);
  assert.strictEqual(fakeNative.__liveBuffers(), live0);
  assert.strictEqual(runner.backendContexts.hip.tracked, null);
  fs.rmdirSync(dir, { recursive: true });
});

test("runner: graph replays read runner-owned input buffers, never the caller's device tensors", async () => {
  const WebDNN = require(path.join(JS, "index"));
  const dir = fs.mkdtempSync(path.join(os.tmpdir(), "webdnn_unit_"));
  writeReluModel(dir);
  WebDNN.resetDefaultContexts();
  table.clearOperators();
  const runner = await WebDNN.load(dir, { backendOrder: ["hip", "cpu"], backendOptions: { hip: { native: fakeNative, strict: true } } });
  const hip = runner.backendContexts.hip;
  const A = await hip.moveTensor(new WebDNN.CPUTensor([5], "float32", new Float32Array([-2, -1, 0, 1, 2])), {});
  const B = await hip.moveTensor(new WebDNN.CPUTensor([5], "float32", new Float32Array([5, -6, 7, -8, 9])), {});
  const want = { A: [0, 0, 0, 1, 2], B: [5, 0, 7, 0, 9] };
  const order = ["A", "A", "B", "A", "B", "B", "A"]; // eager, capture, replays
  for (const which of order) {
    const [y] = await runner.run([which === "A" ? A : B], { graph: true });
    assert.deepStrictEqual(Array.from(y.data), want[which], `run with ${which}`);
  }
  assert.ok(runner.graphState && runner.graphState.inputs[0] !== A && runner.graphState.inputs[0] !== B);
  // the caller's tensors are untouched and may be disposed while the graph lives on
  assert.deepStrictEqual(Array.from(await A.getData()), [-2, -1, 0, 1, 2]);
  assert.deepStrictEqual(Array.from(await B.getData()), [5, -6, 7, -8, 9]);
  A.dispose();
  const [y] = await runner.run([B], { graph: true });
  assert.deepStrictEqual(Array.from(y.data), want.B);
  // other shapes: the graph is dropped and the next run warms up eagerly before a new capture
  assert.strictEqual(runner.graphWarm, true);
  B.dispose();
  runner.disposeGraph();
  fs.rmdirSync(dir, { recursive: true });
});

test("runner: loading another model frees the device copies of the old initializers", async () => {
  const WebDNN = require(path.join(JS, "index"));
  const dir = fs.mkdtempSync(path.join(os.tmpdir(), "webdnn_unit_"));
  const model = {
    irVersion: 7, opsetImport: [{ domain: "", version: 13 }], metadataProps: [],
    graph: {
      name: "g", node: [{ input: ["x", "w"], output: ["y"], name: "a", opType: "Add", attribute: [] }],
      initializer: [{ name: "w", dims: [5], dataType: 1, floatData: [1, 1, 1, 1, 1] }],
      input: [{ name: "x", type: { tensorType: { elemType: 1, shape: { dim: [{ dimValue: 5 }] } } } }],
      output: [{ name: "y", type: { tensorType: { elemType: 1, shape: { dim: [{ dimValue: 5 }] } } } }],
      valueInfo: [],
    },
  };
  fs.writeFileSync(path.join(dir, "model.onnx"), onnx.encodeModel(model));
  WebDNN.resetDefaultContexts();
  table.clearOperators();
  const live0 = fakeNative.__liveBuffers();
  const runner = await WebDNN.load(dir, { backendOrder: ["hip", "cpu"], backendOptions: { hip: { native: fakeNative, strict: true } } });
  const x = new WebDNN.CPUTensor([5], "float32", new Float32Array([1, 2, 3, 4, 5]));
  const [y] = await runner.run([x]);
  assert.deepStrictEqual(Array.from(y.data), [2, 3, 4, 5, 6]);
  assert.strictEqual(fakeNative.__liveBuffers(), live0 + 1); // the weight's device copy
  await runner.loadModel(dir, "model.onnx");
  assert.strictEqual(fakeNative.__liveBuffers(), live0);
  const [y2] = await runner.run([x]);
  assert.deepStrictEqual(Array.from(y2.data), [2, 3, 4, 5, 6]);
  fs.rmdirSync(dir, { recursive: true });
});

(async () => {
  let passed = 0, failed = 0;
  for (const [name, fn] of tests) {
    try {
      await fn();
      passed++;
    } catch (e) {
      failed++;
      console.log(`FAIL ${name}\n${e && e.stack ? e.stack : e}`);
    }
  }
  console.log(JSON.stringify({ passed, failed, total: tests.length }));
  process.exit(failed ? 1 : 0);
})();
