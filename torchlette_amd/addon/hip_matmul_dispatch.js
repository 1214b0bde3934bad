"use strict";
/* The fused side door of the `hip` backend: the four functions the graph layer loads
 * by backend name for `matmul -> bias -> activation` chains
 * (src/graph/node-factory.ts:186-217 loads dispatchMatmul, dispatchMatmulDirect,
 * deferredDestroyBuffer and planBareMatmul from the webgpu backend;
 * src/executor/executor.ts:2959-3049 calls them with an EpilogueConfig).
 *
 * The reference keeps a matmul with a packed B operand OUT of this path
 * (src/compiler/graph-compiler.ts:150-152) because its tiled kernel cannot read packed
 * words.  Here the packed operand is the case served: the chain goes to the GEMV /
 * prefill kernels' epilogue in one launch. */
const H = require("./hip_backend.js");
const tl = H.native;

const DT = { f32: 0, f16: 1 };
const UNARY = { relu: 1, silu: 2, gelu: 3, gelu_tanh: 3, gelu_erf: 4, sigmoid: 5, tanh: 6 };
const EPI_BIAS = 1, EPI_UNARY = 2, EPI_BINARY = 3, EPI_CAST_F16 = 4;
const BINARY = { add: 0, sub: 1, mul: 2 };

/** EpilogueConfig.ops (matmul/types.ts:13-24) -> the addon's op list.  `binary` takes an
 *  [M,N] input (add, sub, mul: matmul-skeleton.ts:934-955); a `cast` to f16 in the middle of
 *  the chain rounds the value there, one that closes the chain must name the output dtype. */
function lowerEpilogue(epilogue, epilogueInputs, outputDtype, m, n) {
  const ops = [];
  const list = (epilogue && epilogue.ops) || [];
  list.forEach((op, i) => {
    if (op.kind === "none") return;
    if (op.kind === "bias") {
      const t = epilogueInputs[op.inputIndex];
      if (!t) throw new Error(`hip dispatchMatmul: epilogue input ${op.inputIndex} missing`);
      if (!(t.dtype in DT)) throw new Error(`hip dispatchMatmul: bias dtype ${t.dtype}`);
      const biasCount = t.size !== undefined ? t.size : t.nbytes / (t.dtype === "f16" ? 2 : 4);
      if (biasCount !== n) throw new Error(`hip dispatchMatmul: a bias epilogue input must hold N = ${n} elements`);
      ops.push([EPI_BIAS, 0, t.ptr, DT[t.dtype], 1]);
    } else if (op.kind === "unary") {
      if (!(op.op in UNARY)) throw new Error(`hip dispatchMatmul: unary epilogue op ${op.op} is not built`);
      ops.push([EPI_UNARY, UNARY[op.op], null, 0, 0]);
    } else if (op.kind === "binary") {
      const t = epilogueInputs[op.inputIndex];
      if (!t) throw new Error(`hip dispatchMatmul: epilogue input ${op.inputIndex} missing`);
      if (!(t.dtype in DT)) throw new Error(`hip dispatchMatmul: binary epilogue input dtype ${t.dtype}`);
      if (!(op.op in BINARY)) throw new Error(`Unsupported binary epilogue: ${op.op}`);
      // the kernels index it by output element: anything but M*N elements would be read out of bounds
      const count = t.size !== undefined ? t.size : t.nbytes / (t.dtype === "f16" ? 2 : 4);
      if (count !== m * n || !t.isContiguous)
        throw new Error(`hip dispatchMatmul: a binary epilogue input must be a contiguous [M,N] = [${m},${n}] tensor`);
      ops.push([EPI_BINARY, BINARY[op.op], t.ptr, DT[t.dtype], m]);
    } else if (op.kind === "cast") {
      if (i === list.length - 1) {
        if (op.toDtype !== outputDtype) throw new Error("hip dispatchMatmul: the cast that closes the chain must name the output dtype");
      } else if (op.toDtype === "f16") {
        ops.push([EPI_CAST_F16, 0, null, 0, 0]);
      }  // a cast to f32 in the chain changes nothing: the chain computes in f32
    } else {
      throw new Error(`hip dispatchMatmul: epilogue op kind ${op.kind} is not built`);
    }
  });
  if (ops.length > 4) throw new Error("hip dispatchMatmul: at most 4 epilogue ops");
  return ops;
}

/** dispatchMatmul(a, b, transA, transB, donatedBuffer, epilogueOpts) (webgpu/dispatch.ts:859-957)
 *  for a packed B: either the transposed [K,N] view of the weight, or the [N,K] weight
 *  itself with transB. */
function dispatchMatmul(a, b, transA, transB, donatedBuffer, epilogueOpts) {
  if (!(b.format && b.format.packing)) throw new Error("hip backend: dense matmul is outside the quantized-weight linear path");
  if (transA) throw new Error("hip dispatchMatmul: transposed A is not part of the linear path");
  const be = H.getBackend();
  const wargs = be._weightArgs(b, !transB);
  const n = wargs[2], k = wargs[3];
  if (!a.shape.length || a.shape[a.shape.length - 1] !== k) throw new Error("matmul dimension mismatch");
  if (!a.isContiguous) throw new Error("matmulQuantizedB: strided activations");
  const promoted = a.dtype === "f16" && b.format.elementType === "f16" ? "f16" : "f32";
  const outputDtype = (epilogueOpts && epilogueOpts.epilogue && epilogueOpts.epilogue.outputDtype) || promoted;
  const m = k ? a.size / k : 0;
  const ops = epilogueOpts ? lowerEpilogue(epilogueOpts.epilogue, epilogueOpts.epilogueInputs || [], outputDtype, m, n) : [];
  const outShape = a.shape.slice(0, -1).concat([n]);
  const need = outShape.reduce((p, c) => p * c, 1) * (outputDtype === "f16" ? 2 : 4);
  let out;
  if (donatedBuffer && donatedBuffer.nbytes >= need) {
    out = new H.HipTensor(be, outShape, outputDtype, donatedBuffer.ptr, need, false, donatedBuffer);
  } else {
    out = be._alloc(outShape, outputDtype);
  }
  tl.matmulQuantizedOps.apply(null, wargs.concat([a.ptr, DT[a.dtype], m, out.ptr, DT[outputDtype], ops]));
  return out;
}

/** dispatchMatmulDirect(bufA, bufB, config) (webgpu/dispatch.ts:968-1040): geometry was
 *  resolved on the first execution and cached by the caller; the packed operand's
 *  description travels in `config.packing` / `config.scales` (two fields the lowered
 *  plan gains for a packed B). */
function dispatchMatmulDirect(bufA, bufB, config) {
  const p = config.packing;
  if (!p) throw new Error("hip dispatchMatmulDirect: config.packing is required");
  const be = H.getBackend();
  const FMT = { "int8-grouped": 0, "int8-row": 1, "int4-grouped": 2 };
  const ops = lowerEpilogue(config.epilogueConfig, config.epilogueBuffers || [], config.outputDtype, config.m, config.n);
  const out = be._alloc(config.outShape, config.outputDtype);
  tl.matmulQuantizedOps(FMT[p.scheme], p.groupSize, config.n, config.k, bufB.ptr, config.scales.ptr, bufA.ptr,
    DT[config.dtypeA], config.m, out.ptr, DT[config.outputDtype], ops);
  return out;
}

/** planBareMatmul (webgpu/dispatch.ts:814-857): a packed operand has no generated plan;
 *  the caller then keeps the matmul a sequential action, which is dispatchMatmul above. */
function planBareMatmul(a, b) {
  if (b.format && b.format.packing) return "quantized-operand";
  return "dense-matmul-not-built";
}

/** Buffers are freed in stream order, so there is nothing to defer. */
function deferredDestroyBuffer(t) {
  if (t && t.destroy) t.destroy();
}

module.exports = { dispatchMatmul, dispatchMatmulDirect, planBareMatmul, deferredDestroyBuffer };
