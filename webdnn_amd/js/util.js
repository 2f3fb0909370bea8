"use strict";
// Small helpers.  Reference: src/descriptor_runner/util.ts:1-92.

function nonnull(value) {
  if (value === null || value === undefined) {
    throw new Error("value is null");
  }
  return value;
}

function arraySum(vec) {
  let x = 0;
  for (let i = 0; i < vec.length; i++) x += vec[i];
  return x;
}

function arrayProd(vec) {
  let x = 1;
  for (let i = 0; i < vec.length; i++) x *= vec[i];
  return x;
}

function arrayEqual(a, b) {
  if (a.length !== b.length) return false;
  for (let i = 0; i < a.length; i++) if (a[i] !== b[i]) return false;
  return true;
}

function arange(start, stop, step) {
  if (stop === undefined) {
    stop = start;
    start = 0;
  }
  if (step === undefined) step = 1;
  const out = [];
  if (step > 0) for (let v = start; v < stop; v += step) out.push(v);
  else for (let v = start; v > stop; v += step) out.push(v);
  return out;
}

const INT32_MAX = 2147483647;
const INT32_MIN = -2147483648;

// ONNX int64 values are kept as int32 on every backend; out-of-range values
// saturate (util.ts:73-81, used for "slice to the end" sentinels like 2^63-1).
function clipToInt32(v) {
  if (typeof v === "bigint") {
    if (v > BigInt(INT32_MAX)) return INT32_MAX;
    if (v < BigInt(INT32_MIN)) return INT32_MIN;
    return Number(v);
  }
  if (v > INT32_MAX) return INT32_MAX;
  if (v < INT32_MIN) return INT32_MIN;
  return v;
}

module.exports = { nonnull, arraySum, arrayProd, arrayEqual, arange, clipToInt32, INT32_MAX, INT32_MIN };
