"use strict";
// softmax(alpha * Q K) V as one node: what the hip fusion pass makes of
//   [Transpose ->] MatMul [* scalar] -> Softmax(last axis) -> MatMul [<- Transpose] [-> Transpose(1,0,2)].
// The reference runs these as separate nodes (cpu matmul.ts:11-111, softmax.ts:13-59); this
// operator yields the same tensor.  When the operands are heads lying side by side in
// [tokens, heads, d] projections (d = 32, 64 or 128 contiguous, at most 1024 keys) the whole
// chain is one kernel launch; any other layout runs the steps one by one, exactly as the
// unfused nodes would, errors included.
const { OperatorImpl } = require("../../../operatorImpl");
const { getAttrFloat, getAttrInt, getAttrInts } = require("../../../operatorUtil");
const { HipMatMul, operandView } = require("./matmul");

const MAX_KEYS = 1024;

class HipAttention extends OperatorImpl {
  constructor() {
    super("hip");
  }

  initialize(attribute) {
    super.initialize(attribute);
    this.alpha = getAttrFloat(attribute, "alpha", 1.0);
    this.softmaxAxis = getAttrInt(attribute, "softmax_axis", -1);
    this.permQ = getAttrInts(attribute, "perm_q", []);
    this.permK = getAttrInts(attribute, "perm_k", []);
    this.permV = getAttrInts(attribute, "perm_v", []);
    this.permY = getAttrInts(attribute, "perm_y", []);
    // the separate steps, for layouts the kernel does not take
    this.scores = new HipMatMul(true);
    this.scores.initialize([]);
    this.scores.alpha = this.alpha;
    this.scores.permA = this.permQ;
    this.scores.permB = this.permK;
    this.context = new HipMatMul(true);
    this.context.initialize([]);
    this.context.permB = this.permV;
    this.context.permY = this.permY;
  }

  async run(context, inputs) {
    context.assertsHipTensorArray(inputs);
    const [q, k, v] = inputs;
    for (const t of inputs) if (t.dataType !== "float32") throw new Error("only float32 is supported");
    const plan = this.oneLaunchPlan(q, k, v);
    if (plan) {
      const { batch, tq, tk, d } = plan;
      const merged = this.permY.length === 3;
      const output = context.emptyTensor(merged ? [tq, batch, d] : [batch, tq, d], "float32");
      context.native.attention(q.handle, k.handle, v.handle, output.handle, batch, tq, tk, d,
        plan.q[0], plan.q[1], plan.k[0], plan.k[2], plan.v[0], plan.v[1],
        merged ? d : tq * d, merged ? batch * d : d, this.alpha);
      return [output];
    }
    return this.stepByStep(context, q, k, v);
  }

  // Strides of the three operands as [batch, row, column] views if the kernel can take them, else null.
  oneLaunchPlan(q, k, v) {
    const view = (t, perm) => {
      if (!perm.length) return t.ndim === 3 ? { dims: t.dims, strides: t.strides } : null;
      if (perm.length !== 3 || t.ndim !== 3) return null;
      return { dims: perm.map((p) => t.dims[p]), strides: perm.map((p) => t.strides[p]) };
    };
    const vq = view(q, this.permQ), vk = view(k, this.permK), vv = view(v, this.permV);
    if (!vq || !vk || !vv) return null;
    if (this.permY.length && this.permY.join() !== "1,0,2") return null;
    const axis = this.softmaxAxis < 0 ? this.softmaxAxis + 3 : this.softmaxAxis;
    if (axis !== 2) return null;
    const [batch, tq, d] = vq.dims, tk = vk.dims[2];
    if (vk.dims[0] !== batch || vv.dims[0] !== batch) return null; // a broadcast batch takes the general MatMul
    if (vk.dims[1] !== d || vv.dims[1] !== tk || vv.dims[2] !== d) return null; // (the steps report the mismatch)
    if (d !== 32 && d !== 64 && d !== 128) return null;
    if (tk < 1 || tk > MAX_KEYS || batch < 1 || tq < 1) return null;
    // the head dimension contiguous in all three, 16-byte steps for Q and K
    if (vq.strides[2] !== 1 || vk.strides[1] !== 1 || vv.strides[2] !== 1) return null;
    if ([vq.strides[0], vq.strides[1], vk.strides[0], vk.strides[2]].some((s) => s % 4 !== 0)) return null;
    return { batch, tq, tk, d, q: vq.strides, k: vk.strides, v: vv.strides };
  }

  async stepByStep(context, q, k, v) {
    const viewQ = operandView(context, q, this.permQ), viewK = operandView(context, k, this.permK);
    let scores;
    try {
      scores = this.scores.product(context, q, k, viewQ, viewK, null, null);
    } finally {
      if (viewQ.temp) viewQ.temp.dispose();
      if (viewK.temp) viewK.temp.dispose();
    }
    let probs;
    try {
      let axis = this.softmaxAxis;
      if (axis < 0) axis += scores.ndim;
      if (axis !== scores.ndim - 1) throw new Error("Softmax: currently only reducing final axis is supported");
      const len = scores.dims[axis];
      probs = context.emptyTensor(scores.dims, "float32");
      context.native.softmax(scores.handle, probs.handle, len ? scores.length / len : 0, len);
    } finally {
      scores.dispose();
    }
    const viewP = operandView(context, probs, []), viewV = operandView(context, v, this.permV);
    try {
      return [this.context.product(context, probs, v, viewP, viewV, null, null)];
    } finally {
      probs.dispose();
      if (viewV.temp) viewV.temp.dispose();
    }
  }
}

function getOpEntries() {
  // produced by the hip fusion pass
  return [{ opType: "WebDNNHipAttention", backend: "hip", opsetMin: 1, factory: () => new HipAttention() }];
}
module.exports = { getOpEntries };
