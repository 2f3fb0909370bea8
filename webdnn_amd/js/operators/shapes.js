"use strict";
// Shape arithmetic of the operators, as plain functions of dims and attributes.
//
// Everything here is derived from the ONNX operator definitions (Conv, MatMul, Gemm, Transpose,
// Squeeze, Unsqueeze, Split, Flatten, and the two broadcasting rules) and written around three
// small tools: a dense-stride rule, "view a shape as a larger one" (stretching extent-1 axes
// with stride 0), and per-axis sliding-window arithmetic.  The operator classes in
// operators/base/ are adapters that read attributes and hand the results on under the property
// names the backends' kernels expect; those names follow the reference's operator classes
// (src/descriptor_runner/operators/base/*.ts), whose results these functions must reproduce.

// Row-major element strides: the last axis is contiguous.
function denseStrides(dims) {
  const strides = new Array(dims.length);
  let run = 1;
  for (let axis = dims.length - 1; axis >= 0; axis--) {
    strides[axis] = run;
    run *= dims[axis];
  }
  return strides;
}

function elementCount(dims) {
  let n = 1;
  for (const d of dims) n *= d;
  return n;
}

// dims with extent-1 axes added on the left until it has `rank` axes.
function leftPad(dims, rank) {
  const out = Array.from(dims);
  if (out.length > rank) return null;
  return new Array(rank - out.length).fill(1).concat(out);
}

// Element strides with which a tensor of shape `dims` is read as if it had shape `target`
// (same or higher rank): axes it lacks and axes of extent 1 repeat (stride 0); any other
// mismatch is what `complain()` reports.
function stretchedStrides(dims, target, complain) {
  const padded = leftPad(dims, target.length);
  if (!padded) throw complain();
  const strides = denseStrides(padded);
  padded.forEach((extent, axis) => {
    if (extent === target[axis]) return;
    if (extent !== 1) throw complain();
    strides[axis] = 0;
  });
  return strides;
}

// Unidirectional broadcast (Gemm's C, a MatMul bias): strides of B read in A's shape.
function broadcastOnto(dimsA, dimsB) {
  return stretchedStrides(dimsB, Array.from(dimsA), () => new Error(`Unidirectional broadcast error: ${dimsA}, ${dimsB}`));
}

// Multidirectional (numpy) broadcast: the common shape and every operand's strides in it.
function broadcastTogether(allDims) {
  const rank = allDims.reduce((r, d) => Math.max(r, d.length), 0);
  const dims = new Array(rank).fill(1);
  for (const d of allDims) leftPad(d, rank).forEach((extent, axis) => { if (extent > dims[axis]) dims[axis] = extent; });
  const complain = () => new Error(`Multidirectional broadcasting error: ${allDims.map((d) => `[${d}]`)}`);
  return { dims, allStrides: allDims.map((d) => stretchedStrides(d, dims, complain)) };
}

// One spatial axis of a sliding window (Conv, pooling): how many window positions fit.
function windowPositions(extent, padBegin, padEnd, dilation, kernel, stride) {
  const reach = dilation * (kernel - 1) + 1; // input span of one window
  return Math.floor((extent + padBegin + padEnd - reach) / stride) + 1;
}

// 2-D convolution geometry.  attrs: {dilations, group, kernelShape, pads, strides}, empty lists = defaults.
function convGeometry(dimsX, dimsW, attrs) {
  const orDefault = (list, fallback) => (list && list.length ? list : fallback);
  const g = {
    batch: dimsX[0],
    dilations: orDefault(attrs.dilations, [1, 1]),
    group: attrs.group,
    kernelShape: orDefault(attrs.kernelShape, dimsW.slice(2, 4)),
    pads: orDefault(attrs.pads, [0, 0, 0, 0]),
    strides: orDefault(attrs.strides, [1, 1]),
    inShape: dimsX.slice(2, 4),
    chIn: dimsX[1],
    chOut: dimsW[0],
  };
  g.outShape = g.inShape.map((extent, axis) =>
    windowPositions(extent, g.pads[axis], g.pads[axis + 2], g.dilations[axis], g.kernelShape[axis], g.strides[axis]));
  g.chInPerGroup = g.chIn / g.group;
  g.chOutPerGroup = g.chOut / g.group;
  return g;
}

// A rank-2 Gemm operand seen as [outer, inner] of the product; `swapped`: stored as [inner, outer].
function gemmOperand(dims, swapped) {
  return swapped ? { outer: dims[1], inner: dims[0], strides: [1, dims[1]] } : { outer: dims[0], inner: dims[1], strides: [dims[1], 1] };
}

function gemmPlan(dimsA, dimsB, transA, transB) {
  if (dimsA.length !== 2 || dimsB.length !== 2) throw new Error("Gemm: inputs must be 2-D");
  const a = gemmOperand(dimsA, !!transA); // rows x k
  const b = gemmOperand(dimsB, !transB); //  columns x k when seen from the result
  if (a.inner !== b.inner) throw new Error("Gemm: inner dimensions differ");
  return { m: a.outer, n: b.outer, k: a.inner, strideA: a.strides, strideB: [b.strides[1], b.strides[0]] };
}

// numpy matmul: the last two axes multiply, the axes before them broadcast; a rank-1 operand is
// a row (left) or a column (right) whose added axis is dropped from the result again.
function matmulPlan(dimsA, dimsB) {
  if (dimsA.length === 0 || dimsB.length === 0) throw new Error("MatMul: scalar input");
  const matA = dimsA.length === 1 ? [1, dimsA[0]] : Array.from(dimsA);
  const matB = dimsB.length === 1 ? [dimsB[0], 1] : Array.from(dimsB);
  const rank = Math.max(matA.length, matB.length);
  const fullA = leftPad(matA, rank), fullB = leftPad(matB, rank);
  const [rows, innerProductLength] = fullA.slice(rank - 2);
  const [innerB, cols] = fullB.slice(rank - 2);
  if (innerProductLength !== innerB) throw new Error("MatMul: inner dimensions differ");
  // batch axes: the larger extent wins; an operand whose extent is 1 there is re-read (stride 0).
  // (An extent that is neither equal nor 1 is not diagnosed here; the kernels' bounds checks are.)
  const stridesA = denseStrides(fullA), stridesB = denseStrides(fullB);
  const resultDims = [];
  for (let axis = 0; axis < rank - 2; axis++) {
    if (fullA[axis] === 1) stridesA[axis] = 0;
    if (fullB[axis] === 1) stridesB[axis] = 0;
    resultDims.push(Math.max(fullA[axis], fullB[axis]));
  }
  resultDims.push(rows, cols);
  const resultDimsAfterSqueeze = resultDims.filter((_, axis) =>
    !(dimsA.length === 1 && axis === rank - 2) && !(dimsB.length === 1 && axis === rank - 1));
  return {
    resultLength: elementCount(resultDims), resultDims, resultStrides: denseStrides(resultDims),
    resultDimsAfterSqueeze, stridesA, stridesB, innerProductLength,
  };
}

// Transpose as a strided view: output axis i walks input axis perm[i].  No perm = reversed axes.
function permutedView(dims, strides, perm) {
  const order = perm && perm.length ? perm : dims.map((_, axis) => dims.length - 1 - axis);
  if (order.length !== dims.length) throw new Error("Transpose: perm length differs from rank");
  return { outShape: order.map((axis) => dims[axis]), inStrides: order.map((axis) => strides[axis]) };
}

function normalizeAxis(axis, rank) {
  return axis < 0 ? axis + rank : axis;
}

// Squeeze: the listed axes go; with no list, every axis of extent 1 goes.
function withoutAxes(dims, axes) {
  if (!axes.length) return dims.filter((extent) => extent !== 1);
  const gone = new Set(axes.map((a) => normalizeAxis(a, dims.length)));
  return dims.filter((_, axis) => !gone.has(axis));
}

// Unsqueeze: axes of extent 1 appear at the listed positions of the RESULT (negative positions
// count from its end); the input's extents fill the other positions in order.
function withAxes(dims, axes) {
  const rank = dims.length + axes.length;
  const ones = new Set(axes.map((a) => normalizeAxis(a, rank)));
  const rest = Array.from(dims);
  const out = [];
  for (let axis = 0; axis < rank; axis++) out.push(ones.has(axis) ? 1 : rest.shift());
  if (rest.length || out.includes(undefined)) throw new Error("Unsqueeze: axes are out of range or repeated");
  return out;
}

// Split: consecutive bands of one axis.  lengths = [] -> equal parts of floor(extent / nOutputs).
function splitBands(dims, axisAttr, nOutputs, lengths) {
  const axis = normalizeAxis(axisAttr, dims.length);
  if (!(axis >= 0 && axis < dims.length)) throw new Error(`Split: axis ${axis} out of range`);
  const extent = dims[axis];
  const parts = [];
  let offset = 0;
  for (let i = 0; i < nOutputs; i++) {
    const dim = lengths.length ? lengths[i] : Math.floor(extent / nOutputs);
    if (!(dim >= 0)) throw new Error("Split: fewer part lengths than outputs");
    parts.push({ dim, offset, outShape: dims.map((d, a) => (a === axis ? dim : d)) });
    offset += dim;
  }
  if (offset > extent) throw new Error("Split: parts exceed the axis");
  return { axis, parts };
}

// Flatten to 2-D at axis 1 (the only form the reference supports).
function flattened(dims) {
  return [dims[0], elementCount(dims.slice(1))];
}

module.exports = {
  denseStrides, elementCount, leftPad, stretchedStrides, broadcastOnto, broadcastTogether, windowPositions,
  convGeometry, gemmPlan, matmulPlan, permutedView, withoutAxes, withAxes, splitBands, flattened,
};
