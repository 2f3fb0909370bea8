"use strict";
// Test helper: node load_tensors.js FILE[,FILE...]  -> one JSON line
//   {"ok": true, "tensors": {name: {dims, dataType, bits: [uint32...]}}, "progress": [..]}
// or {"ok": false, "error": message}.  Values travel as their 32-bit patterns so that the
// comparison on the Python side is exact.
const path = require("path");
const JS = path.join(__dirname, "..", "..", "webdnn_amd", "js");
const { TensorLoaderImpl } = require(path.join(JS, "core", "tensorLoaderImpl"));
const { WebDNNCPUContextImpl } = require(path.join(JS, "backend", "cpu", "cpuContextImpl"));

(async () => {
  const cpu = new WebDNNCPUContextImpl();
  await cpu.initialize();
  const progress = [];
  try {
    const tensors = await new TensorLoaderImpl(process.argv[2].split(","), cpu).loadAll((n) => progress.push(n));
    const out = {};
    for (const [name, t] of tensors.entries()) {
      out[name] = { dims: t.dims, dataType: t.dataType, bits: Array.from(new Uint32Array(t.data.buffer, t.data.byteOffset, t.data.length)) };
    }
    console.log(JSON.stringify({ ok: true, tensors: out, progress }));
  } catch (e) {
    console.log(JSON.stringify({ ok: false, error: e.message }));
  }
})();
