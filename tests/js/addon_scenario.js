"use strict";
/* Runs the JavaScript `hip` backend (torchlette_amd/addon/hip_backend.js) over the
 * inputs a pytest run wrote into a directory, and writes what it computed back there.
 * Usage: node addon_scenario.js <dir>.  <dir>/manifest.json lists the cases; every
 * array is a raw little-endian file.  One process runs every case. */
const fs = require("fs");
const path = require("path");
const H = require(path.join(__dirname, "..", "..", "torchlette_amd", "addon", "hip_backend.js"));

const dir = process.argv[2];
const manifest = JSON.parse(fs.readFileSync(path.join(dir, "manifest.json"), "utf8"));
const TYPES = { f32: Float32Array, u32: Uint32Array, u16: Uint16Array, i32: Int32Array };

function load(name, type) {
  const buf = fs.readFileSync(path.join(dir, name));
  const ab = buf.buffer.slice(buf.byteOffset, buf.byteOffset + buf.byteLength);
  return new TYPES[type](ab);
}
function save(name, typed) {
  fs.writeFileSync(path.join(dir, name), Buffer.from(typed.buffer, typed.byteOffset, typed.byteLength));
}
/* activations arrive as f32 files; an f16 tensor is made by the backend's own codec */
function tensor(be, name, shape, dtype) {
  return be.ops.tensorFromArray(load(name, "f32"), shape, dtype);
}
function weightOf(be, c) {
  const fmt = H.resolveWeightFormat(c.format, c.element);
  const scales = load(c.scales, c.format === "int8-row" ? "f32" : "u16");
  return be.createQuantizedWeight(load(c.packed, "u32"), scales, c.n, c.k, fmt);
}

const D = require(path.join(__dirname, "..", "..", "torchlette_amd", "addon", "hip_matmul_dispatch.js"));

const results = { cases: {}, errors: {} };
const be = H.getBackend(0);
results.device = be.deviceInfo();

for (const c of manifest.cases) {
  const r = {};
  if (c.kind === "linear") {
    const w = weightOf(be, c);
    const x = tensor(be, c.x, [c.m, c.k], c.xdtype);
    const bias = c.bias ? tensor(be, c.bias, [c.n], "f32") : null;
    const g0 = H.getQuantGemvDispatchCount(), m0 = H.getQuantGemmDispatchCount();
    const y = be.linear(x, w, bias, c.act, c.fused);
    r.gemv = H.getQuantGemvDispatchCount() - g0;
    r.gemm = H.getQuantGemmDispatchCount() - m0;
    r.shape = y.shape;
    r.dtype = y.dtype;
    save(c.out, be.readSync(y));
  } else if (c.kind === "quantize") {
    const q = H.quantizeLinearWeight(load(c.weight, "f32"), c.n, c.k, c.g);
    save(c.out_packed, q.packed);
    save(c.out_scales, q.scales);
    const w = be.createQuantizedWeight(q.packed, q.scales, c.n, c.k, H.resolveWeightFormat(c.g === 64 ? "int8-64" : "int8-128", "f32"));
    const d0 = H.getDequantI8DispatchCount();
    save(c.out_dequant, be.readSync(be.dequantizeToF32(w)));
    r.dequant = H.getDequantI8DispatchCount() - d0;
    // and on the device, from the f32 weight uploaded as it is
    const wdev = be.ops.tensorFromArray(load(c.weight, "f32"), [c.n, c.k], "f32");
    const qd = be.quantizeLinearWeightOnDevice(wdev, c.g, "f32");
    save(c.out_dequant_device, be.readSync(be.dequantizeToF32(qd)));
  } else if (c.kind === "rmsnorm_linear" || c.kind === "gated_linear") {
    const w = weightOf(be, c);
    const x = tensor(be, c.x, [c.m, c.k], c.xdtype);
    let y, apart;
    if (c.kind === "rmsnorm_linear") {
      const nw = tensor(be, c.norm_weight, [c.k], "f32");
      const normed = be.ops.fusedRMSNormForward(x, nw, { numRows: c.m, featureDim: c.k, eps: c.eps });
      save(c.out_norm, be.readSync(normed));
      y = be.linearAfterRMSNorm(x, nw, c.eps, w);
      apart = be.linear(normed, w, null, "none", true);
    } else {
      const up = tensor(be, c.up, [c.m, c.k], c.xdtype);
      const prod = be.ops.mul(be.ops.silu(x), up);   // the model's two ops
      save(c.out_prod, be.readSync(prod));
      y = be.linearAfterGatedMul(x, up, "silu", w);
      apart = be.linear(prod, w, null, "none", true);
    }
    save(c.out, be.readSync(y));
    save(c.out_apart, be.readSync(apart));
  } else if (c.kind === "grouped") {
    const x = tensor(be, c.x, [c.m, c.k], "f16");
    const ws = c.weights.map((wc) => weightOf(be, Object.assign({ k: c.k, format: c.format, element: "f16" }, wc)));
    const outs = be.linearGrouped(x, ws);
    outs.forEach((o, i) => save(c.weights[i].out, be.readSync(o)));
    if (c.out_noalloc) {
      const out = be.ops.zeros([c.m, c.weights[0].n], "f16");
      save(c.out_noalloc, be.readSync(be.linearInto(out, x, ws[0], null, "none")));
      // an output or a bias shorter than the shapes say is refused before anything is launched
      r.into_errors = r.into_errors || [];
      try {
        be.linearInto(be.ops.zeros([Math.max(1, (x.size / ws[0].shape[1]) * ws[0].shape[0] - 1)], out.dtype), x, ws[0], null, "none");
        r.into_errors.push(null);
      } catch (e) {
        r.into_errors.push(e.message);
      }
      try {
        be.linearInto(out, x, ws[0], be.ops.zeros([ws[0].shape[0] - 1], "f32"), "none");
        r.into_errors.push(null);
      } catch (e) {
        r.into_errors.push(e.message);
      }
    }
  } else if (c.kind === "mlp") {
    // the MLP block of a decode step as one call into the addon
    const x = tensor(be, c.x, [c.m, c.k], "f16");
    const [gate, up, down] = c.weights.map((wc) => weightOf(be, Object.assign({ format: c.format, element: "f16" }, wc)));
    const g0 = H.getQuantGemvDispatchCount();
    const y = be.mlpDecode(x, gate, up, down, c.act);
    r.dispatches = H.getQuantGemvDispatchCount() - g0;
    r.shape = y.shape;
    r.dtype = y.dtype;
    save(c.out, be.readSync(y));
    r.status = be.sequenceStatus();
  } else if (c.kind === "side_door") {
    // the fused path's call for matmul -> bias -> unary (-> cast): executor.ts:2959-3049
    const w = weightOf(be, c);
    const x = tensor(be, c.x, [c.m, c.k], c.xdtype);
    const bias = tensor(be, c.bias, [c.n], "f32");
    const epilogue = { ops: [{ kind: "bias", inputIndex: 0 }, { kind: "unary", op: c.act }, { kind: "cast", toDtype: c.out_dtype }],
                       additionalInputCount: 1, outputDtype: c.out_dtype };
    const g0 = H.getQuantGemvDispatchCount() + H.getQuantGemmDispatchCount();
    const y1 = D.dispatchMatmul(x, be.ops.transpose(w), false, false, undefined, { epilogue, epilogueInputs: [bias] });
    r.launches = H.getQuantGemvDispatchCount() + H.getQuantGemmDispatchCount() - g0;
    const y2 = D.dispatchMatmul(x, w, false, true, undefined, { epilogue, epilogueInputs: [bias] });
    const donated = be.ops.zeros([c.m, c.n], "f32");   // larger than needed for f16: reused
    const y3 = D.dispatchMatmul(x, be.ops.transpose(w), false, false, donated, { epilogue, epilogueInputs: [bias] });
    r.donated_reused = y3.ptr === donated.ptr;
    const y4 = D.dispatchMatmulDirect(x, w, { m: c.m, n: c.n, k: c.k, outShape: [c.m, c.n], dtypeA: c.xdtype,
      outputDtype: c.out_dtype, epilogueConfig: epilogue, epilogueBuffers: [bias], packing: w.format.packing, scales: w.scales });
    r.dtype = y1.dtype;
    r.plan = D.planBareMatmul(x, be.ops.transpose(w));
    [y1, y2, y3, y4].forEach((y, i) => save(c.out + i, be.readSync(y)));
    // matmul -> bias -> unary -> add residual: a binary step with an [M,N] input
    const residual = tensor(be, c.residual, [c.m, c.n], "f32");
    const chain = { ops: [{ kind: "bias", inputIndex: 0 }, { kind: "unary", op: c.act }, { kind: "binary", op: "add", inputIndex: 1 }],
                    additionalInputCount: 2, outputDtype: c.out_dtype };
    save(c.out + "_residual", be.readSync(D.dispatchMatmul(x, be.ops.transpose(w), false, false, undefined,
      { epilogue: chain, epilogueInputs: [bias, residual] })));
    try {   // an [N] tensor where the [M,N] one belongs must be refused, not read out of bounds
      D.dispatchMatmul(x, be.ops.transpose(w), false, false, undefined,
        { epilogue: { ops: [{ kind: "binary", op: "mul", inputIndex: 0 }], additionalInputCount: 1, outputDtype: "f32" }, epilogueInputs: [bias] });
      r.binary_error = null;
    } catch (e) {
      r.binary_error = e.message;
    }
    try {
      D.dispatchMatmul(x, be.ops.transpose(w), false, false, undefined,
        { epilogue: { ops: [{ kind: "binary", op: "div", inputIndex: 0 }], additionalInputCount: 1, outputDtype: "f32" }, epilogueInputs: [residual] });
      r.binary_op_error = null;
    } catch (e) {
      r.binary_op_error = e.message;
    }
  } else if (c.kind === "topk") {
    const logits = tensor(be, c.logits, [c.length], "f32");
    be.ops.readTopK(logits, c.k).then((t) => {
      save(c.out_values, t.values);
      save(c.out_indices, t.indices);
    });
    const packed = be.ops.deviceTopK(logits, c.k);
    save(c.out_packed, be.readSync(packed));
  }
  results.cases[c.name] = r;
}

/* the error channel: every failure is a thrown Error carrying the library's message */
function expectThrow(name, fn) {
  try {
    fn();
    results.errors[name] = null;
  } catch (e) {
    results.errors[name] = { message: e.message, code: e.code || null };
  }
}
{
  const c = manifest.cases.find((v) => v.kind === "linear");
  const w = weightOf(be, c);
  const bad = be.ops.zeros([1, c.k + 32], "f32");
  expectThrow("dimension_mismatch", () => be.linear(bad, w));
  expectThrow("dense_matmul", () => be.ops.matmul(bad, be.ops.zeros([c.k + 32, 8], "f32")));
  expectThrow("quantize_bad_k", () => H.quantizeLinearWeight(new Float32Array(6), 2, 3, 64));
  expectThrow("bad_config", () => {
    const x = be.ops.zeros([1, c.k], c.xdtype);
    be.linear(x, w, null, "none", true, new Int32Array([2, 256, 256, 64, 2, 2, 0, 0]));  // a prefill tile for M = 1
  });
  expectThrow("unknown_format", () => H.resolveWeightFormat("int3-7"));
  // tuning cache: seed, export, clear, import
  const x = be.ops.zeros([1, c.k], c.xdtype);
  const cfg = be.candidates(w, c.xdtype, 1, c.element === "f16" && c.xdtype === "f16" ? "f16" : "f32")[0];
  const ydt = c.element === "f16" && c.xdtype === "f16" ? "f16" : "f32";
  be.seedPerShapeMatmulChoice(w, c.xdtype, 1, ydt, cfg);
  const text = H.exportTuningCache();
  H.clearTuningCache();
  const cleared = H.exportTuningCache();
  H.importTuningCache(text);
  results.tuning = {
    seeded: Array.from(cfg), exported_entries: Object.keys(JSON.parse(text).entries).length,
    text_has_key: text.length > cleared.length,
    selected_after_import: Array.from(be.selectedConfig(w, c.xdtype, 1, ydt)),
  };
  H.setAutotuneEnabled(true);
  results.autotune_enabled = H.isAutotuneEnabled();
  const a0 = H.getAutotuneRunCount();
  H.clearTuningCache();
  be.linear(x, w);
  results.autotune_runs = H.getAutotuneRunCount() - a0;
  H.setAutotuneEnabled(false);
}
/* the Backend contract (src/backend/types.ts:340-696): every required op is there (the list is
 * the mock backend's, src/backend/mock/index.ts:150-176), `read` is a Promise of numbers, and
 * the ops outside this path are declared delegates to a cpu backend */
const pending = [];
{
  const conf = {};
  conf.required = H.REQUIRED_OPS.slice();
  conf.missing = H.REQUIRED_OPS.filter((n) => typeof be.ops[n] !== "function");
  conf.name = be.name;
  const a = be.ops.tensorFromArray([1, 2, 3, 4, 5, 6], [2, 3], "f32");
  const b = be.ops.tensorFromArray([6, 5, 4, 3, 2, 1], [2, 3], "f32");
  const p = be.ops.read(a);
  conf.read_is_promise = p instanceof Promise;
  pending.push(p.then((v) => {
    conf.read_value = v;
    conf.read_is_array = Array.isArray(v);
  }));
  expectThrow("delegated_without_cpu", () => be.ops.sub(a, b));
  // a stand-in for getBackend("cpu"): tensors are {shape, toArray()}, as BackendTensor requires
  const cpuTensor = (shape, data) => ({ shape, toArray: () => data });
  be.setCpuDelegate({ name: "cpu", ops: {
    tensorFromArray: (values, shape) => cpuTensor(shape, Array.from(values)),
    sub: (x, y) => cpuTensor(x.shape, x.toArray().map((v, i) => v - y.toArray()[i])),
    sum: (x) => cpuTensor([], [x.toArray().reduce((s, v) => s + v, 0)]),
  } });
  const d = be.ops.sub(a, b);
  conf.sub = Array.from(be.readSync(d));
  conf.sub_shape = d.shape;
  conf.sum = Array.from(be.readSync(be.ops.sum(a)));
  expectThrow("delegated_unknown_to_cpu", () => be.ops.gather(a, 0, b));
  // a strided view is materialised through the host
  const at = be.ops.transpose(a);
  conf.transposed_contiguous = at.isContiguous;
  conf.transposed = Array.from(be.readSync(be.ops.contiguous(at)));
  conf.transposed_to_array = at.toArray();
  be.setCpuDelegate(null);
  results.conformance = conf;
}
be.synchronize();
Promise.all(pending).then(() => setImmediate(() => {
  fs.writeFileSync(path.join(dir, "results.json"), JSON.stringify(results));
}));
