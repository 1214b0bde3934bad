"use strict";
/* The `hip` backend object in JavaScript: what `src/backend/hip/index.ts` would hold in
 * the reference tree, written as CommonJS so that the Node this image ships runs it as
 * it is.  It serves the backend op interface of the quantized-weight linear path
 * (src/backend/types.ts:340-696) over the N-API addon beside it:
 *
 *   ops.tensorFromArray / zeros / read             webgpu/ops/creation.ts:51-87, `read`
 *   ops.transpose / permute / reshape / contiguous views; format + scales travel with
 *                                                  the view (webgpu/ops/views.ts:925-934)
 *   ops.matmul                                     matmul-ops.ts:42-59 -> matmulQuantizedB
 *                                                  (matmul-ops.ts:113-182)
 *   ops.add / mul / relu / silu / sigmoid / tanh / gelu / cast
 *   ops.fusedRMSNormForward                        types.ts:635-640
 *   readTopK / deviceTopK                          types.ts:632-634, 669-678
 *   createQuantizedWeight                          runtime/engine.ts:2041-2149
 *   quantizeLinearWeight, f32ToF16Bits, f16BitsToF32   backend/quantize.ts
 *   resolveWeightFormat                            types.ts:55-67 (+ "int4-32", "int8-row")
 *   linear                                         frontend/torchlette.ts:878-894
 *   setAutotuneEnabled, exportTuningCache, ...     matmul/dispatch.ts:99-141, autotune.ts:309-329
 *
 *   ops.sub / div / sqrt / expand / gather / scatterAdd / sum / max / mean / where /
 *   stridedScatterCopy / stridedScatterAdd / contiguous (of a strided view)
 *                                                  the rest of the required BackendOps
 *                                                  (types.ts:340-679; the smallest conforming
 *                                                  backend is mock/index.ts:150-176): OUTSIDE
 *                                                  this path, declared host-copy delegates to
 *                                                  the cpu backend given to setCpuDelegate()
 *
 * There is no CPU fallback for the path itself: without a gfx950 device `getBackend()`
 * throws, and the delegated ops throw with the op's name until a cpu backend is set. */
const path = require("path");
const tl = require(path.join(__dirname, "tlhip_napi.node"));

const FMT = { "int8-grouped": 0, "int8-row": 1, "int4-grouped": 2 };
const DT = { f32: 0, f16: 1, i32: 2 };
const BYTES = { f32: 4, f16: 2, u32: 4, i32: 4 };
const UNARY = { none: 0, relu: 1, silu: 2, gelu: 3, gelu_tanh: 3, gelu_erf: 4, sigmoid: 5, tanh: 6 };
const PRO_RMSNORM = 1, PRO_GATED_MUL = 2;
/* BackendOps that every backend must have (types.ts:340-679; mock/index.ts:150-176) and that
 * are not part of the quantized-weight linear path. */
const DELEGATED_OPS = ["sub", "div", "sqrt", "expand", "gather", "scatterAdd", "sum", "max", "mean", "where",
                       "stridedScatterCopy", "stridedScatterAdd"];
/* ... and the whole required set, for conformance checks. */
const REQUIRED_OPS = ["tensorFromArray", "add", "sub", "div", "mul", "matmul", "sqrt", "relu", "expand", "reshape", "transpose",
                      "permute", "contiguous", "gather", "scatterAdd", "sum", "max", "mean", "where", "stridedScatterCopy",
                      "stridedScatterAdd", "read"];

function sizeOf(shape) {
  return shape.reduce((p, c) => p * c, 1);
}
function stridesFor(shape) {
  const s = new Array(shape.length);
  let acc = 1;
  for (let i = shape.length - 1; i >= 0; i--) {
    s[i] = acc;
    acc *= shape[i];
  }
  return s;
}

/** resolveWeightFormat (types.ts:57-67) with the two formats this backend adds. */
function resolveWeightFormat(name, elementType) {
  elementType = elementType || "f16";
  if (name === "int8-64" || name === "int8-128")
    return { elementType, packing: { scheme: "int8-grouped", groupSize: name === "int8-64" ? 64 : 128, scalesDtype: "f16" } };
  if (name === "int4-32") return { elementType, packing: { scheme: "int4-grouped", groupSize: 32, scalesDtype: "f16" } };
  if (name === "int8-row") return { elementType, packing: { scheme: "int8-row", groupSize: 0, scalesDtype: "f32" } };
  throw new Error(`resolveWeightFormat: unknown weight format ${name}`);
}

/* f16 <-> f32 for host arrays: the codec of quantize.ts:22-60. */
function toF16Bits(values) {
  const out = new Uint16Array(values.length);
  for (let i = 0; i < values.length; i++) out[i] = tl.f32ToF16Bits(values[i]);
  return out;
}
function fromF16Bits(bits) {
  const out = new Float32Array(bits.length);
  for (let i = 0; i < bits.length; i++) out[i] = tl.f16BitsToF32(bits[i]);
  return out;
}

class HipTensor {
  constructor(backend, shape, dtype, ptr, nbytes, owns, base) {
    this.backend = backend;
    this.shape = shape.slice();
    this.strides = stridesFor(shape);
    this.dtype = dtype;
    this.ptr = ptr;
    this.nbytes = nbytes;
    this.ownsBuffer = owns;
    this.isContiguous = true;
    this.format = undefined;
    this.scales = undefined;
    this._base = base || null;
  }
  get size() {
    return sizeOf(this.shape);
  }
  /** BackendTensor.toArray: a host copy as plain numbers. */
  toArray() {
    return Array.from(this.backend.readSync(this));
  }
  destroy() {
    if (this.ownsBuffer && this.ptr) {
      tl.free(this.ptr);
      this.ptr = 0n;
    }
  }
}

class HipBackend {
  constructor(deviceIndex) {
    tl.init(deviceIndex || 0);
    this.name = "hip";
    this.fusedPrologueMaxRows = 2;  // see linearAfterRMSNorm
    const self = this;
    this.ops = {
      tensorFromArray(values, shape, dtype) {
        dtype = dtype || "f32";
        if (!(dtype in BYTES)) throw new Error(`hip backend: unsupported dtype ${dtype}`);
        let host;
        if (dtype === "f32") host = values instanceof Float32Array ? values : Float32Array.from(values);
        else if (dtype === "f16") host = values instanceof Uint16Array ? values : toF16Bits(values);
        else if (dtype === "u32") host = values instanceof Uint32Array ? values : Uint32Array.from(values);
        else host = values instanceof Int32Array ? values : Int32Array.from(values);
        if (host.length !== sizeOf(shape)) throw new Error("tensorFromArray: data length does not match shape");
        const t = self._alloc(shape, dtype);
        tl.memcpyH2D(t.ptr, host);
        return t;
      },
      zeros(shape, dtype) {
        const t = self._alloc(shape, dtype || "f32");
        if (t.nbytes) tl.memset(t.ptr, 0, t.nbytes);
        return t;
      },
      /** read(a): Promise<number[]> (types.ts:666): the one op that waits.  f16 tensors come
       *  back as f32 values, as the reference's read does. */
      read(a) {
        return new Promise((resolve, reject) => {
          try {
            resolve(Array.from(self.readSync(a)));
          } catch (e) {
            reject(e);
          }
        });
      },
      permute(a, dims) {
        const v = new HipTensor(self, dims.map((d) => a.shape[d]), a.dtype, a.ptr, a.nbytes, false, a._base || a);
        v.strides = dims.map((d) => a.strides[d]);
        v.isContiguous = v.strides.every((s, i) => s === stridesFor(v.shape)[i]);
        v.format = a.format;  // views.ts:925-934: the format and its scales follow the view
        v.scales = a.scales;
        return v;
      },
      transpose(a, options) {
        const r = a.shape.length;
        let d0 = options && options.dim0 !== undefined ? options.dim0 : r - 2;
        let d1 = options && options.dim1 !== undefined ? options.dim1 : r - 1;
        if (d0 < 0) d0 += r;
        if (d1 < 0) d1 += r;
        const dims = a.shape.map((_, i) => i);
        dims[d0] = d1;
        dims[d1] = d0;
        return self.ops.permute(a, dims);
      },
      reshape(a, shape) {
        if (!a.isContiguous) throw new Error("hip backend reshape: contiguous tensors only");
        if (sizeOf(shape) !== a.size) throw new Error("reshape: element count mismatch");
        const v = new HipTensor(self, shape, a.dtype, a.ptr, a.nbytes, false, a._base || a);
        v.format = a.format;
        v.scales = a.scales;
        return v;
      },
      /** A strided view is materialised through a host copy (outside the path: the
       *  Linear's transposed weight view is consumed by matmul as a view, never copied). */
      contiguous(a) {
        if (a.isContiguous) return a;
        if (a.format && a.format.packing) throw new Error("hip backend contiguous: a packed weight view is not materialised");
        return self.ops.tensorFromArray(self.readSync(a), a.shape, a.dtype === "f16" ? "f16" : a.dtype);
      },
      /** matmul-ops.ts:42-59: a packed B operand goes to matmulQuantizedB. */
      matmul(a, b) {
        if (b.format && b.format.packing) return self._matmulQuantizedB(a, b, null, "none");
        throw new Error("hip backend: dense matmul is outside the quantized-weight linear path");
      },
      /** Only the Linear bias case: b is [N] broadcast over a's rows. */
      add(a, b) {
        const n = a.shape[a.shape.length - 1];
        if (b.size !== n || !(a.dtype in DT) || !(b.dtype in DT) || !a.isContiguous)
          throw new Error("hip backend add: only a[...,N] + bias[N]");
        const out = self._alloc(a.shape, a.dtype);
        tl.biasAdd(a.ptr, DT[a.dtype], b.ptr, DT[b.dtype], out.ptr, n ? a.size / n : 0, n);
        return out;
      },
      mul(a, b) {
        return self.ops.gatedMul(a, b, "none");
      },
      gatedMul(gate, up, activation) {
        if (gate.dtype !== up.dtype || gate.size !== up.size || !gate.isContiguous || !up.isContiguous)
          throw new Error("hip backend mul: two contiguous f32/f16 tensors of one shape");
        const out = self._alloc(gate.shape, gate.dtype);
        tl.gatedMul(UNARY[activation === "gelu" ? "gelu_tanh" : activation || "silu"], gate.ptr, up.ptr, DT[gate.dtype], out.ptr, gate.size);
        return out;
      },
      relu: (a) => self._unary("relu", a),
      silu: (a) => self._unary("silu", a),
      sigmoid: (a) => self._unary("sigmoid", a),
      tanh: (a) => self._unary("tanh", a),
      /** CPU backend default is the tanh form (src/backend/cpu/numeric.ts:626-630). */
      gelu: (a, options) => self._unary(!options || (options.approximate || "tanh") === "tanh" ? "gelu_tanh" : "gelu_erf", a),
      cast(a, dtype) {
        if (a.dtype === dtype) return a;
        if (!(a.dtype in DT) || !(dtype in DT) || !a.isContiguous) throw new Error("hip backend cast: f32 <-> f16 only");
        const out = self._alloc(a.shape, dtype);
        tl.cast(a.ptr, DT[a.dtype], out.ptr, DT[dtype], a.size);
        return out;
      },
      /** types.ts:635-640: x [N,D], weight f32 [D], config {numRows, featureDim, eps}. */
      fusedRMSNormForward(x, weight, config) {
        if (weight.dtype !== "f32" || !x.isContiguous) throw new Error("hip backend rmsnorm: contiguous x, f32 weight");
        if (x.size !== config.numRows * config.featureDim || weight.size !== config.featureDim)
          throw new Error("fusedRMSNormForward: shape mismatch");
        const out = self._alloc(x.shape, x.dtype);
        tl.rmsnorm(x.ptr, DT[x.dtype], weight.ptr, out.ptr, DT[x.dtype], config.numRows, config.featureDim, config.eps);
        return out;
      },
      /** types.ts:669-678: the k largest of a[offset .. offset+length), only 2k numbers read back. */
      async readTopK(a, k, opts) {
        const offset = (opts && opts.offset) || 0;
        const length = opts && opts.length !== undefined ? opts.length : a.size - offset;
        if (a.dtype !== "f32") throw new Error("readTopK: f32 logits");
        const vals = self._alloc([k], "f32");
        const idx = self._alloc([k], "i32");
        tl.topk(a.ptr, offset, length, k, vals.ptr, idx.ptr, DT.i32);
        const values = new Float32Array(k);
        const indices = new Int32Array(k);
        tl.memcpyD2H(values, vals.ptr);
        tl.memcpyD2H(indices, idx.ptr);
        vals.destroy();
        idx.destroy();
        return { values, indices };
      },
      /** types.ts:632-634: [2k] f32 on the device, values then indices (as f32). */
      deviceTopK(logits, config) {
        const k = typeof config === "number" ? config : config.k;
        const out = self._alloc([2 * k], "f32");
        tl.topk(logits.ptr, 0, logits.size, k, out.ptr, out.ptr + BigInt(4 * k), DT.f32);
        return out;
      },
    };
    /* The required BackendOps that are not on the quantized-weight linear path: declared
     * host-copy delegates.  Each downloads its tensor arguments, runs the cpu backend's op
     * of the same name and uploads the result. */
    for (const name of DELEGATED_OPS) {
      if (!(name in this.ops)) this.ops[name] = (...args) => self._viaHost(name, args);
    }
    this._cpu = null;
  }

  /** The cpu backend (`getBackend("cpu")` of a torchlette checkout) the delegated ops run on. */
  setCpuDelegate(cpuBackend) {
    this._cpu = cpuBackend;
  }

  _viaHost(name, args) {
    const cpu = this._cpu;
    if (!cpu || !cpu.ops || typeof cpu.ops[name] !== "function")
      throw new Error(`hip backend: ${name} is outside the quantized-weight linear path; it runs on the cpu backend ` +
                      "through a host copy once setCpuDelegate(cpuBackend) has been called");
    let dtype = "f32";
    const onCpu = [];
    const lower = (v) => {
      if (v instanceof HipTensor) {
        if (v.dtype === "f16") dtype = "f16";
        // the cpu backend holds every dtype as f32 values (src/backend/cpu/numeric.ts:29-117)
        const t = cpu.ops.tensorFromArray(Array.from(this.readSync(v)), v.shape.slice());
        onCpu.push(t);
        return t;
      }
      return Array.isArray(v) && v.some((e) => e instanceof HipTensor) ? v.map(lower) : v;
    };
    const out = cpu.ops[name].apply(cpu.ops, args.map(lower));
    const up = this.ops.tensorFromArray(out.toArray(), out.shape.slice(), dtype);
    for (const t of onCpu.concat([out])) if (t.destroy) t.destroy();
    return up;
  }

  /** Synchronous host copy of a tensor as a typed array (f16 -> f32 values); a strided
   *  view is gathered on the host from its base buffer. */
  readSync(a) {
    const TYPES = { f32: Float32Array, u32: Uint32Array, i32: Int32Array };
    const fetch = (ptr, n, dtype) => {
      if (dtype === "f16") {
        const bits = new Uint16Array(n);
        if (n) tl.memcpyD2H(bits, ptr);
        return fromF16Bits(bits);
      }
      const out = new TYPES[dtype](n);
      if (n) tl.memcpyD2H(out, ptr);
      return out;
    };
    if (a.isContiguous) return fetch(a.ptr, a.size, a.dtype);
    const base = fetch(a.ptr, a.nbytes / BYTES[a.dtype], a.dtype);
    const out = new base.constructor(a.size);
    const idx = new Array(a.shape.length).fill(0);
    for (let i = 0; i < out.length; i++) {
      let off = 0;
      for (let d = 0; d < idx.length; d++) off += idx[d] * a.strides[d];
      out[i] = base[off];
      for (let d = idx.length - 1; d >= 0 && ++idx[d] === a.shape[d]; d--) idx[d] = 0;
    }
    return out;
  }

  _alloc(shape, dtype) {
    const nbytes = sizeOf(shape) * BYTES[dtype];
    const ptr = tl.malloc(Math.max(nbytes, 16));
    return new HipTensor(this, shape, dtype, ptr, nbytes, true, null);
  }

  _unary(name, a) {
    if (!(a.dtype in DT) || !a.isContiguous) throw new Error(`hip backend ${name}: contiguous f32/f16 only`);
    const out = this._alloc(a.shape, a.dtype);
    tl.unary(UNARY[name], a.ptr, DT[a.dtype], out.ptr, a.size);
    return out;
  }

  synchronize() {
    tl.synchronize();
  }
  deviceInfo() {
    return tl.deviceInfo();
  }

  /** RuntimeEngine.createQuantizedWeight (engine.ts:2041-2149): upload packed words and
   *  scales, then present the logical [N,K] tensor with `format` and `scales` attached. */
  createQuantizedWeight(packed, scalesBits, n, k, format) {
    const packing = format.packing;
    if (!packing) throw new Error("createQuantizedWeight: format.packing is required");
    const perWord = packing.scheme === "int4-grouped" ? 8 : 4;
    if (k % perWord !== 0) throw new Error(`createQuantizedWeight: K=${k} must be divisible by ${perWord}`);
    const wordsPerRow = k / perWord;
    if (packed.length !== n * wordsPerRow)
      throw new Error(`createQuantizedWeight: packed length ${packed.length} != ${n * wordsPerRow}`);
    let scalesT;
    if (packing.scheme === "int8-row") {
      if (scalesBits.length !== n) throw new Error(`createQuantizedWeight: scales length ${scalesBits.length} != ${n}`);
      scalesT = this.ops.tensorFromArray(scalesBits, [n], "f32");
    } else {
      const groupsPerRow = k / packing.groupSize;
      if (scalesBits.length !== n * groupsPerRow)
        throw new Error(`createQuantizedWeight: scales length ${scalesBits.length} != ${n * groupsPerRow}`);
      // two f16 per u32 word, the same bytes as the u16 array (engine.ts:2077-2087)
      const scaleWords = Math.ceil(scalesBits.length / 2);
      const scalesU32 = new Uint32Array(scaleWords);
      new Uint16Array(scalesU32.buffer).set(scalesBits);
      scalesT = this.ops.tensorFromArray(scalesU32, [scaleWords], "u32");
    }
    const packedT = this.ops.tensorFromArray(packed, [n, wordsPerRow], "u32");
    // the buffer is unchanged; the metadata above the matmul seam is the logical view
    packedT.shape = [n, k];
    packedT.strides = [k, 1];
    packedT.dtype = format.elementType;
    packedT.format = format;
    packedT.scales = scalesT;
    return packedT;
  }

  /** tlhip_qweight_t fields of a packed operand, given as the logical [N,K] tensor or
   *  its transposed [K,N] view. */
  _weightArgs(w, transposed) {
    const packing = w.format && w.format.packing;
    if (!packing || !w.scales) throw new Error("matmulQuantizedB: missing packing/scales on B operand");
    const r = w.shape.length;
    const n = transposed ? w.shape[r - 1] : w.shape[r - 2];
    const k = transposed ? w.shape[r - 2] : w.shape[r - 1];
    const wantStrides = transposed ? [1, k] : [k, 1];
    if (w.strides[r - 2] !== wantStrides[0] || w.strides[r - 1] !== wantStrides[1])
      throw new Error("matmulQuantizedB: the packed operand must be the weight or its transposed view");
    return [FMT[packing.scheme], packing.groupSize, n, k, w.ptr, w.scales.ptr];
  }

  /** matmul-ops.ts:113-182.  B is the transposed [K,N] view of the logical [N,K]
   *  weight; A is [..., M, K] and its leading dimensions fold into M. */
  _matmulQuantizedB(a, b, bias, activation, config) {
    const wargs = this._weightArgs(b, true);
    const n = wargs[2], k = wargs[3];
    if (!(a.dtype in DT)) throw new Error(`matmulQuantizedB: unsupported activation dtype ${a.dtype}`);
    if (!a.shape.length || a.shape[a.shape.length - 1] !== k) throw new Error("matmul dimension mismatch");
    if (!a.isContiguous) throw new Error("matmulQuantizedB: strided activations");
    const m = k ? a.size / k : 0;
    // f16 out only when activations and the weight's element type are both f16 (gemv.ts:27-29)
    const outDtype = a.dtype === "f16" && b.format.elementType === "f16" ? "f16" : "f32";
    const out = this._alloc(a.shape.slice(0, -1).concat([n]), outDtype);
    const args = wargs.concat([a.ptr, DT[a.dtype], m, out.ptr, DT[outDtype], bias ? bias.ptr : null,
                               bias ? DT[bias.dtype] : 0, UNARY[activation || "none"]]);
    if (config) args.push(config);
    tl.matmulQuantized.apply(null, args);
    return out;
  }

  /** api.linear (torchlette.ts:878-894): transpose view, matmul, add, then the model's
   *  activation.  fused = false issues the ops one by one as a plain Backend receives
   *  them; fused = true hands bias and activation to the kernel's epilogue. */
  linear(input, weight, bias, activation, fused, config) {
    const wT = this.ops.transpose(weight);
    const act = activation === "gelu" ? "gelu_tanh" : activation || "none";
    if (fused) return this._matmulQuantizedB(input, wT, bias || null, act, config);
    let y = config ? this._matmulQuantizedB(input, wT, null, "none", config) : this.ops.matmul(input, wT);
    if (bias) {
      const y2 = this.ops.add(y, bias);
      y.destroy();
      y = y2;
    }
    if (act !== "none") {
      const y2 = this._unary(act, y);
      y.destroy();
      y = y2;
    }
    return y;
  }

  /** Up to four decode Linears on the same f16 activations (1..16 rows; one row with a
   *  prologue) in one launch (q/k/v, gate/up). */
  linearGrouped(input, weights, biases, activation, prologue) {
    if (weights.length < 1 || weights.length > 4) throw new Error("linearGrouped: a group holds 1..4 weights");
    if (input.dtype !== "f16") throw new Error("linearGrouped: f16 activations");
    const rows = input.size / this._weightArgs(weights[0], false)[3];
    if (!(rows >= 1 && rows <= 16) || (prologue && rows !== 1)) throw new Error("linearGrouped: 1..16 activation rows (one row with a prologue)");
    const outDtype = weights.every((w) => w.format.elementType === "f16") ? "f16" : "f32";
    const act = UNARY[activation === "gelu" ? "gelu_tanh" : activation || "none"];
    const outs = [];
    const probs = weights.map((w, i) => {
      const wa = this._weightArgs(w, false);
      if (input.size !== rows * wa[3]) throw new Error("linearGrouped: the weights of a group share K");
      const out = this._alloc(input.shape.slice(0, -1).concat([wa[2]]), outDtype);
      outs.push(out);
      const b = biases && biases[i];
      return wa.concat([input.ptr, out.ptr, b ? b.ptr : null, b ? DT[b.dtype] : 0, act]);
    });
    if (prologue) tl.gemvGrouped(probs, DT[input.dtype], DT[outDtype], prologue.kind, prologue.operand, prologue.unary, prologue.eps);
    else if (rows === 1) tl.gemvGrouped(probs, DT[input.dtype], DT[outDtype]);
    else tl.gemvGroupedRows(probs, DT[input.dtype], rows, DT[outDtype]);
    return outs;
  }

  _linearWithPrologue(input, prologue, weight, bias, activation) {
    const wa = this._weightArgs(weight, false);
    const n = wa[2], k = wa[3];
    if (!input.isContiguous || input.shape[input.shape.length - 1] !== k) throw new Error("linear: activations must be contiguous [..., K]");
    const m = k ? input.size / k : 0;
    if (m > this.fusedPrologueMaxRows) return null;
    const outDtype = input.dtype === "f16" && weight.format.elementType === "f16" ? "f16" : "f32";
    const out = this._alloc(input.shape.slice(0, -1).concat([n]), outDtype);
    const act = UNARY[activation === "gelu" ? "gelu_tanh" : activation || "none"];
    const ok = tl.gemvPrologue.apply(null, wa.concat([input.ptr, DT[input.dtype], m, out.ptr, DT[outDtype],
      bias ? bias.ptr : null, bias ? DT[bias.dtype] : 0, act, prologue.kind, prologue.operand, prologue.unary, prologue.eps]));
    if (!ok) {
      out.destroy();
      return null;
    }
    return out;
  }

  /** linear(rmsnorm(input, normWeight, eps), weight, bias): the norm runs inside the GEMV's
   *  activation staging for one or two rows (where that measures faster), else apart. */
  linearAfterRMSNorm(input, normWeight, eps, weight, bias, activation) {
    if (normWeight.dtype !== "f32" || normWeight.size !== input.shape[input.shape.length - 1])
      throw new Error("linearAfterRMSNorm: norm weight must be f32 [K]");
    const fused = this._linearWithPrologue(input, { kind: PRO_RMSNORM, operand: normWeight.ptr, unary: 0, eps }, weight, bias, activation);
    if (fused) return fused;
    const d = normWeight.size;
    const normed = this.ops.fusedRMSNormForward(input, normWeight, { numRows: input.size / d, featureDim: d, eps });
    const out = this.linear(normed, weight, bias, activation, true);
    normed.destroy();
    return out;
  }

  /** linear(mul(gateActivation(gate), up), weight, bias): the MLP's down projection. */
  linearAfterGatedMul(gate, up, gateActivation, weight, bias, activation) {
    if (gate.dtype !== up.dtype || gate.size !== up.size || !up.isContiguous) throw new Error("linearAfterGatedMul: gate and up must share shape and dtype");
    const un = UNARY[gateActivation === "gelu" ? "gelu_tanh" : gateActivation];
    const fused = this._linearWithPrologue(gate, { kind: PRO_GATED_MUL, operand: up.ptr, unary: un, eps: 0 }, weight, bias, activation);
    if (fused) return fused;
    const x = this.ops.gatedMul(gate, up, gateActivation);
    const out = this.linear(x, weight, bias, activation, true);
    x.destroy();
    return out;
  }

  /** down(mul(gateActivation(gate(input)), up(input))) of a decode step's MLP block
   *  (packages/qwen3-browser/src/model.ts:357-361) from ONE call into the addon instead
   *  of three (the library issues the launches, whichever form is faster): f16
   *  activations, 1..16 rows. */
  mlpDecode(input, gate, up, down, gateActivation) {
    const ga = this._weightArgs(gate, false), ua = this._weightArgs(up, false), da = this._weightArgs(down, false);
    const k = ga[3], ff = ga[2];
    if (input.dtype !== "f16" || !input.isContiguous || input.shape[input.shape.length - 1] !== k)
      throw new Error("mlpDecode: activations must be contiguous f16 [..., K]");
    const m = input.size / k;
    if (!Number.isInteger(m) || m < 1 || m > 16) throw new Error("mlpDecode: 1..16 activation rows");
    if (ua[2] !== ff || ua[3] !== k || da[3] !== ff) throw new Error("mlpDecode: gate and up are [F,K], down is [N,F]");
    const outDtype = down.format.elementType === "f16" ? "f16" : "f32";
    const h = this._alloc([m, ff], "f16");
    const out = this._alloc(input.shape.slice(0, -1).concat([da[2]]), outDtype);
    try {
      tl.mlpDecode(ga, ua, da, UNARY[gateActivation === "gelu" ? "gelu_tanh" : gateActivation || "silu"], input.ptr, DT.f16, m, h.ptr, out.ptr, DT[outDtype]);
    } catch (e) {
      out.destroy();
      throw e;
    } finally {
      h.destroy();  // hipFree waits for the launch
    }
    return out;
  }

  /** Waits for the stream; 0, or throws if a sequence launch (mlpDecode) gave up a wait. */
  sequenceStatus() {
    return tl.sequenceStatus();
  }

  linearGroupedAfterRMSNorm(input, normWeight, eps, weights, biases, activation) {
    return this.linearGrouped(input, weights, biases, activation, { kind: PRO_RMSNORM, operand: normWeight.ptr, unary: 0, eps });
  }

  /** linear(input, weight, bias, activation) for M <= 16 through the entry point that allocates no
   *  device memory (tlhip_gemv_noalloc; `out` is the caller's): for code under graph capture. */
  linearInto(out, input, weight, bias, activation) {
    const wa = this._weightArgs(weight, false);
    const n = wa[2], k = wa[3];
    const m = input.size / k;
    // `out` and `bias` are the caller's buffers and the kernel sees only pointers: anything
    // shorter than the shapes say would be read or written past its end, so refuse it here
    if (!Number.isInteger(m) || m < 1 || m > 16) throw new Error("linearInto: 1..16 activation rows");
    if (!(input.dtype in DT) || !input.isContiguous) throw new Error("linearInto: activations must be contiguous f32 or f16");
    if (!(out.dtype in DT) || !out.isContiguous || out.nbytes < m * n * (out.dtype === "f16" ? 2 : 4))
      throw new Error(`linearInto: out must be a contiguous tensor of at least [${m},${n}] ${out.dtype} elements`);
    if (bias && (!(bias.dtype in DT) || !bias.isContiguous || bias.size !== n)) throw new Error(`linearInto: bias must hold N = ${n} elements`);
    const act = UNARY[activation === "gelu" ? "gelu_tanh" : activation || "none"];
    tl.gemvNoalloc.apply(null, wa.concat([input.ptr, DT[input.dtype], m, out.ptr, DT[out.dtype], bias ? bias.ptr : null,
                                          bias ? DT[bias.dtype] : 0, act]));
    return out;
  }

  /** Explicit dequantisation to f32 [N,K] (dispatchDequantizeInt8Grouped, dispatch.ts:949-1037). */
  dequantizeToF32(w) {
    const wa = this._weightArgs(w, false);
    const out = this._alloc([wa[2], wa[3]], "f32");
    tl.dequant.apply(null, wa.concat([out.ptr]));
    return out;
  }

  /** quantizeLinearWeight for an f32 [N,K] weight already on the device; same bits. */
  quantizeLinearWeightOnDevice(weight, groupSize, elementType) {
    groupSize = groupSize || 64;
    if (weight.dtype !== "f32" || weight.shape.length !== 2 || !weight.isContiguous) throw new Error("quantizeLinearWeightOnDevice: contiguous f32 [N,K]");
    const n = weight.shape[0], k = weight.shape[1];
    const packedT = this._alloc([n, k / 4], "u32");
    const scalesT = this._alloc([Math.ceil((n * k) / groupSize / 2)], "u32");
    tl.quantizeInt8GroupedDevice(weight.ptr, n, k, groupSize, packedT.ptr, scalesT.ptr);
    const format = resolveWeightFormat(groupSize === 64 ? "int8-64" : "int8-128", elementType || "f16");
    if (groupSize !== 64 && groupSize !== 128) format.packing.groupSize = groupSize;
    packedT.shape = [n, k];
    packedT.strides = [k, 1];
    packedT.dtype = format.elementType;
    packedT.format = format;
    packedT.scales = scalesT;
    return packedT;
  }

  /** Backend.pretuneMatmulShapes (types.ts:688). */
  async pretuneMatmulShapes(shapes) {
    tl.pretuneMatmulShapes([].concat.apply([], shapes));
  }
  autotune(input, weight) {
    const wa = this._weightArgs(weight, false);
    const m = input.size / wa[3];
    const outDtype = input.dtype === "f16" && weight.format.elementType === "f16" ? "f16" : "f32";
    const out = this._alloc([m, wa[2]], outDtype);
    const us = tl.autotune.apply(null, wa.concat([input.ptr, DT[input.dtype], m, out.ptr, DT[outDtype]]));
    out.destroy();
    return us;
  }
  selectedConfig(weight, xDtype, m, yDtype) {
    return tl.selectedConfig.apply(null, this._weightArgs(weight, false).concat([DT[xDtype], m, DT[yDtype]]));
  }
  candidates(weight, xDtype, m, yDtype) {
    return tl.candidates.apply(null, this._weightArgs(weight, false).concat([DT[xDtype], m, DT[yDtype]]));
  }
  seedPerShapeMatmulChoice(weight, xDtype, m, yDtype, config) {
    tl.tuneCacheSeed.apply(null, this._weightArgs(weight, false).concat([DT[xDtype], m, DT[yDtype], config]));
  }
}

let backend = null;
function getBackend(deviceIndex) {
  if (!backend) backend = new HipBackend(deviceIndex || 0);
  return backend;
}

/** quantizeLinearWeight (quantize.ts:77-131): host in, host out. */
function quantizeLinearWeight(weight, n, k, groupSize) {
  const w = weight instanceof Float32Array ? weight : Float32Array.from(weight);
  const q = tl.quantizeInt8Grouped(w, n, k, groupSize === undefined ? 64 : groupSize);
  return { packed: q.packed, scales: q.scales, n, k, groupSize: groupSize === undefined ? 64 : groupSize };
}

module.exports = {
  getBackend,
  HipBackend,
  HipTensor,
  resolveWeightFormat,
  quantizeLinearWeight,
  f32ToF16Bits: tl.f32ToF16Bits,
  f16BitsToF32: tl.f16BitsToF32,
  setAutotuneEnabled: (on) => tl.setAutotuneEnabled(!!on),
  isAutotuneEnabled: () => tl.isAutotuneEnabled(),
  exportTuningCache: () => tl.tuneCacheExport(),
  importTuningCache: (text) => tl.tuneCacheImport(text),
  clearTuningCache: () => tl.tuneCacheClear(),
  getQuantGemvDispatchCount: () => tl.counter("quant_gemv_dispatches"),
  getQuantGemmDispatchCount: () => tl.counter("quant_gemm_dispatches"),
  getDequantI8DispatchCount: () => tl.counter("dequant_dispatches"),
  getAutotuneRunCount: () => tl.counter("autotune_runs"),
  resetMatmulState() {
    tl.tuneCacheClear();
    tl.countersReset();
  },
  REQUIRED_OPS,
  DELEGATED_OPS,
  native: tl,
};
