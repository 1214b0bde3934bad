/* Node N-API addon over the C ABI of libtlhip.so (include/tlhip.h): the thin native
 * layer a TypeScript / JavaScript `hip` backend calls for device memory, copies,
 * streams and kernel launches, where the reference's WebGPU backend calls
 * GPUDevice / GPUQueue (src/backend/webgpu/gpu-context.ts, ops/creation.ts:51-87).
 *
 * Conventions
 *   - device pointers, graphs: BigInt (0n = null);  sizes and shapes: Number
 *   - host data: TypedArray / ArrayBuffer views, copied synchronously (the JS
 *     buffer may be collected or reused as soon as the call returns)
 *   - errors: every failing tlhip_* call throws Error(tlhip_last_error()), the
 *     reference's only error channel (webgpu/ops/matmul-ops.ts:121-126); the
 *     numeric code is on the error's `code` property as "TLHIP_<n>"
 *   - all work goes to the library stream (stream argument NULL)
 *
 * Plain C against node_api.h; built by the Makefile beside it. */
#define NAPI_VERSION 6
#include <node_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tlhip.h"

#define MAX_ARGS 20

static napi_value throw_last(napi_env env, int rc) {
  char code[32];
  snprintf(code, sizeof code, "TLHIP_%d", rc);
  napi_throw_error(env, code, tlhip_last_error());
  return NULL;
}
static napi_value throw_type(napi_env env, const char* msg) {
  napi_throw_type_error(env, NULL, msg);
  return NULL;
}
#define CHECK(rc_expr)                     \
  do {                                     \
    int rc_ = (rc_expr);                   \
    if (rc_ != 0) return throw_last(env, rc_); \
  } while (0)

/* Fetches exactly `n` arguments into a[]. */
#define ARGS(n)                                                               \
  napi_value a[MAX_ARGS];                                                     \
  size_t argc = MAX_ARGS;                                                     \
  if (napi_get_cb_info(env, info, &argc, a, NULL, NULL) != napi_ok) return NULL; \
  if ((n) > 0 && argc < (size_t)(n)) return throw_type(env, "tlhip: too few arguments")

static int get_ptr(napi_env env, napi_value v, void** out) {
  napi_valuetype t;
  *out = NULL;
  if (napi_typeof(env, v, &t) != napi_ok) return 0;
  if (t == napi_null || t == napi_undefined) return 1;
  if (t == napi_bigint) {
    uint64_t p = 0;
    bool lossless = false;
    if (napi_get_value_bigint_uint64(env, v, &p, &lossless) != napi_ok || !lossless) return 0;
    *out = (void*)(uintptr_t)p;
    return 1;
  }
  return 0;
}
static int get_i64(napi_env env, napi_value v, int64_t* out) {
  napi_valuetype t;
  if (napi_typeof(env, v, &t) != napi_ok || t != napi_number) return 0;
  return napi_get_value_int64(env, v, out) == napi_ok;
}
static int get_i32(napi_env env, napi_value v, int32_t* out) {
  int64_t x;
  if (!get_i64(env, v, &x)) return 0;
  *out = (int32_t)x;
  return 1;
}
static int get_f64(napi_env env, napi_value v, double* out) {
  napi_valuetype t;
  if (napi_typeof(env, v, &t) != napi_ok || t != napi_number) return 0;
  return napi_get_value_double(env, v, out) == napi_ok;
}
#define PTR(i, name)  void* name; if (!get_ptr(env, a[i], &name)) return throw_type(env, "tlhip: argument " #i " (" #name ") must be a BigInt device pointer")
#define I64(i, name)  int64_t name; if (!get_i64(env, a[i], &name)) return throw_type(env, "tlhip: argument " #i " (" #name ") must be a number")
#define I32(i, name)  int32_t name; if (!get_i32(env, a[i], &name)) return throw_type(env, "tlhip: argument " #i " (" #name ") must be a number")
#define F64(i, name)  double name; if (!get_f64(env, a[i], &name)) return throw_type(env, "tlhip: argument " #i " (" #name ") must be a number")

/* Bytes behind a TypedArray / DataView / ArrayBuffer argument. */
static int get_bytes(napi_env env, napi_value v, void** data, size_t* nbytes) {
  bool is = false;
  if (napi_is_typedarray(env, v, &is) == napi_ok && is) {
    napi_typedarray_type t;
    size_t len, off;
    napi_value ab;
    if (napi_get_typedarray_info(env, v, &t, &len, data, &ab, &off) != napi_ok) return 0;
    static const size_t elt[] = {1, 1, 1, 2, 2, 4, 4, 4, 8, 8, 8};
    *nbytes = len * elt[t];
    return 1;
  }
  if (napi_is_arraybuffer(env, v, &is) == napi_ok && is) return napi_get_arraybuffer_info(env, v, data, nbytes) == napi_ok;
  if (napi_is_dataview(env, v, &is) == napi_ok && is) {
    napi_value ab;
    size_t off;
    return napi_get_dataview_info(env, v, nbytes, data, &ab, &off) == napi_ok;
  }
  return 0;
}

static napi_value make_ptr(napi_env env, const void* p) {
  napi_value v;
  napi_create_bigint_uint64(env, (uint64_t)(uintptr_t)p, &v);
  return v;
}
static napi_value make_num(napi_env env, double x) {
  napi_value v;
  napi_create_double(env, x, &v);
  return v;
}
static napi_value undefined(napi_env env) {
  napi_value v;
  napi_get_undefined(env, &v);
  return v;
}
static void set_num(napi_env env, napi_value obj, const char* key, double x) {
  napi_set_named_property(env, obj, key, make_num(env, x));
}

/* (format, groupSize, n, k, packedPtr, scalesPtr) starting at a[i]. */
static int get_weight(napi_env env, napi_value* a, tlhip_qweight_t* w) {
  int32_t f, g;
  int64_t n, k;
  void *packed, *scales;
  if (!get_i32(env, a[0], &f) || !get_i32(env, a[1], &g) || !get_i64(env, a[2], &n) || !get_i64(env, a[3], &k) ||
      !get_ptr(env, a[4], &packed) || !get_ptr(env, a[5], &scales))
    return 0;
  w->format = f;
  w->group_size = g;
  w->n = n;
  w->k = k;
  w->packed = packed;
  w->scales = scales;
  return 1;
}
#define WEIGHT(i, name) tlhip_qweight_t name; if (!get_weight(env, a + (i), &name)) return throw_type(env, "tlhip: bad weight arguments (format, groupSize, n, k, packed, scales)")

/* (biasPtr | null, biasDtype, unary) -> epilogue [bias][unary]. */
static void make_epilogue(void* bias, int32_t bias_dtype, int32_t unary, tlhip_epilogue_t* ep) {
  memset(ep, 0, sizeof *ep);
  if (bias) {
    ep->ops[ep->n_ops].kind = TLHIP_EPI_BIAS;
    ep->ops[ep->n_ops].input = bias;
    ep->ops[ep->n_ops].input_dtype = bias_dtype;
    ep->ops[ep->n_ops].rows = 1;
    ep->n_ops++;
  }
  if (unary) {
    ep->ops[ep->n_ops].kind = TLHIP_EPI_UNARY;
    ep->ops[ep->n_ops].unary = unary;
    ep->n_ops++;
  }
}

/* ------------------------------------------------------------------ runtime */
static napi_value Init(napi_env env, napi_callback_info info) {
  ARGS(0);
  int32_t dev = 0;
  if (argc >= 1) get_i32(env, a[0], &dev);
  CHECK(tlhip_init(dev));
  return undefined(env);
}
static napi_value Shutdown(napi_env env, napi_callback_info info) {
  (void)info;
  CHECK(tlhip_shutdown());
  return undefined(env);
}
static napi_value DeviceInfo(napi_env env, napi_callback_info info) {
  (void)info;
  tlhip_device_info_t d;
  CHECK(tlhip_device_info(&d));
  napi_value o, s;
  napi_create_object(env, &o);
  napi_create_string_utf8(env, d.name, NAPI_AUTO_LENGTH, &s);
  napi_set_named_property(env, o, "name", s);
  napi_create_string_utf8(env, d.arch, NAPI_AUTO_LENGTH, &s);
  napi_set_named_property(env, o, "arch", s);
  set_num(env, o, "computeUnits", d.compute_units);
  set_num(env, o, "wavefrontSize", d.wavefront_size);
  set_num(env, o, "ldsBytesPerBlock", d.lds_bytes_per_block);
  set_num(env, o, "clockKhz", d.clock_khz);
  set_num(env, o, "memoryClockKhz", d.memory_clock_khz);
  set_num(env, o, "memoryBusBits", d.memory_bus_bits);
  set_num(env, o, "totalMemoryBytes", (double)d.total_memory_bytes);
  set_num(env, o, "l2Bytes", (double)d.l2_bytes);
  return o;
}
static napi_value Malloc(napi_env env, napi_callback_info info) {
  ARGS(1);
  I64(0, bytes);
  if (bytes < 0) return throw_type(env, "tlhip: negative size");
  void* p = NULL;
  CHECK(tlhip_malloc((size_t)bytes, &p));
  return make_ptr(env, p);
}
static napi_value Free(napi_env env, napi_callback_info info) {
  ARGS(1);
  PTR(0, p);
  CHECK(tlhip_free(p));
  return undefined(env);
}
static napi_value Memset(napi_env env, napi_callback_info info) {
  ARGS(3);
  PTR(0, p);
  I32(1, value);
  I64(2, bytes);
  CHECK(tlhip_memset(p, value, (size_t)bytes, NULL));
  return undefined(env);
}
/* memcpyH2D(dst, hostView [, dstByteOffset]) */
static napi_value MemcpyH2D(napi_env env, napi_callback_info info) {
  ARGS(2);
  PTR(0, dst);
  void* data;
  size_t nbytes;
  if (!get_bytes(env, a[1], &data, &nbytes)) return throw_type(env, "tlhip: memcpyH2D needs a TypedArray or ArrayBuffer");
  int64_t off = 0;
  if (argc >= 3) get_i64(env, a[2], &off);
  if (nbytes == 0) return undefined(env);
  CHECK(tlhip_memcpy_h2d((char*)dst + off, data, nbytes, NULL));
  CHECK(tlhip_stream_synchronize(NULL));
  return undefined(env);
}
/* memcpyD2H(hostView, src [, srcByteOffset]): waits for the stream's earlier work. */
static napi_value MemcpyD2H(napi_env env, napi_callback_info info) {
  ARGS(2);
  void* data;
  size_t nbytes;
  if (!get_bytes(env, a[0], &data, &nbytes)) return throw_type(env, "tlhip: memcpyD2H needs a TypedArray or ArrayBuffer");
  PTR(1, src);
  int64_t off = 0;
  if (argc >= 3) get_i64(env, a[2], &off);
  if (nbytes == 0) return undefined(env);
  CHECK(tlhip_memcpy_d2h(data, (const char*)src + off, nbytes, NULL));
  CHECK(tlhip_stream_synchronize(NULL));
  return undefined(env);
}
static napi_value MemcpyD2D(napi_env env, napi_callback_info info) {
  ARGS(3);
  PTR(0, dst);
  PTR(1, src);
  I64(2, bytes);
  CHECK(tlhip_memcpy_d2d(dst, src, (size_t)bytes, NULL));
  return undefined(env);
}
static napi_value Synchronize(napi_env env, napi_callback_info info) {
  (void)info;
  CHECK(tlhip_stream_synchronize(NULL));
  return undefined(env);
}
static napi_value GraphBeginCapture(napi_env env, napi_callback_info info) {
  (void)info;
  CHECK(tlhip_graph_begin_capture(NULL));
  return undefined(env);
}
static napi_value GraphEndCapture(napi_env env, napi_callback_info info) {
  (void)info;
  tlhip_graph_t g = NULL;
  CHECK(tlhip_graph_end_capture(NULL, &g));
  return make_ptr(env, g);
}
static napi_value GraphLaunch(napi_env env, napi_callback_info info) {
  ARGS(1);
  PTR(0, g);
  CHECK(tlhip_graph_launch(g, NULL));
  return undefined(env);
}
static napi_value GraphDestroy(napi_env env, napi_callback_info info) {
  ARGS(1);
  PTR(0, g);
  CHECK(tlhip_graph_destroy(g));
  return undefined(env);
}

/* ------------------------------------------------------- weight preparation */
static napi_value F32ToF16Bits(napi_env env, napi_callback_info info) {
  ARGS(1);
  F64(0, x);
  return make_num(env, tlhip_f32_to_f16_bits((float)x));
}
static napi_value F16BitsToF32(napi_env env, napi_callback_info info) {
  ARGS(1);
  I32(0, bits);
  return make_num(env, tlhip_f16_bits_to_f32((uint16_t)bits));
}
/* quantizeInt8Grouped(Float32Array weight, n, k, groupSize) -> {packed: Uint32Array, scales: Uint16Array} */
static napi_value QuantizeInt8Grouped(napi_env env, napi_callback_info info) {
  ARGS(4);
  void* data;
  size_t nbytes;
  if (!get_bytes(env, a[0], &data, &nbytes)) return throw_type(env, "tlhip: quantizeInt8Grouped needs a Float32Array");
  I64(1, n);
  I64(2, k);
  I64(3, g);
  if (n < 0 || k < 0 || (uint64_t)n * (uint64_t)k * 4 != nbytes)
    return throw_type(env, "tlhip: quantizeInt8Grouped: weight length is not n*k");
  const size_t nwords = (size_t)n * (size_t)k / 4, nscales = g > 0 ? (size_t)n * (size_t)k / (size_t)g : 0;
  napi_value ab_p, ab_s, packed, scales, o;
  void *pp, *ps;
  napi_create_arraybuffer(env, nwords * 4, &pp, &ab_p);
  napi_create_arraybuffer(env, nscales * 2, &ps, &ab_s);
  uint64_t none = 0; /* an empty ArrayBuffer has no storage; the library still wants a pointer */
  CHECK(tlhip_quantize_int8_grouped((const float*)data, n, k, g, pp ? (uint32_t*)pp : (uint32_t*)&none,
                                    ps ? (uint16_t*)ps : (uint16_t*)&none));
  napi_create_typedarray(env, napi_uint32_array, nwords, ab_p, 0, &packed);
  napi_create_typedarray(env, napi_uint16_array, nscales, ab_s, 0, &scales);
  napi_create_object(env, &o);
  napi_set_named_property(env, o, "packed", packed);
  napi_set_named_property(env, o, "scales", scales);
  return o;
}
/* quantizeInt8GroupedDevice(weightPtr, n, k, groupSize, packedPtr, scalesPtr) */
static napi_value QuantizeInt8GroupedDevice(napi_env env, napi_callback_info info) {
  ARGS(6);
  PTR(0, w);
  I64(1, n);
  I64(2, k);
  I64(3, g);
  PTR(4, packed);
  PTR(5, scales);
  CHECK(tlhip_quantize_int8_grouped_device((const float*)w, n, k, g, (uint32_t*)packed, (uint16_t*)scales, NULL));
  return undefined(env);
}

/* ------------------------------------------------------------------ compute */
/* dequant(format, groupSize, n, k, packed, scales, outPtr) */
static napi_value Dequant(napi_env env, napi_callback_info info) {
  ARGS(7);
  WEIGHT(0, w);
  PTR(6, out);
  CHECK(tlhip_dequant(&w, (float*)out, NULL));
  return undefined(env);
}
/* matmulQuantized(format, groupSize, n, k, packed, scales, xPtr, xDtype, m, yPtr, yDtype,
 *                 biasPtr | null, biasDtype, unary [, config: Int32Array(8)]) */
static napi_value MatmulQuantized(napi_env env, napi_callback_info info) {
  ARGS(14);
  WEIGHT(0, w);
  PTR(6, x);
  I32(7, xd);
  I64(8, m);
  PTR(9, y);
  I32(10, yd);
  PTR(11, bias);
  I32(12, bd);
  I32(13, un);
  tlhip_epilogue_t ep;
  make_epilogue(bias, bd, un, &ep);
  if (argc >= 15) {
    void* cdata;
    size_t cbytes;
    if (!get_bytes(env, a[14], &cdata, &cbytes) || cbytes != sizeof(tlhip_kernel_config_t))
      return throw_type(env, "tlhip: config must be an Int32Array of 8");
    CHECK(tlhip_matmul_quantized_config(&w, x, xd, m, y, yd, 1.0f, ep.n_ops ? &ep : NULL,
                                        (const tlhip_kernel_config_t*)cdata, NULL));
  } else {
    CHECK(tlhip_matmul_quantized(&w, x, xd, m, y, yd, 1.0f, ep.n_ops ? &ep : NULL, NULL));
  }
  return undefined(env);
}
/* matmulQuantizedOps(format, groupSize, n, k, packed, scales, xPtr, xDtype, m, yPtr, yDtype,
 *                    [[kind, unary, inputPtr | null, inputDtype, inputRows], ...])
 * An epilogue chain of up to TLHIP_MAX_EPILOGUE_OPS steps in the caller's order: the
 * EpilogueConfig.ops of the fused path (src/backend/webgpu/matmul/types.ts:13-24). */
static napi_value MatmulQuantizedOps(napi_env env, napi_callback_info info) {
  ARGS(12);
  WEIGHT(0, w);
  PTR(6, x);
  I32(7, xd);
  I64(8, m);
  PTR(9, y);
  I32(10, yd);
  bool is_array = false;
  uint32_t count = 0;
  if (napi_is_array(env, a[11], &is_array) != napi_ok || !is_array) return throw_type(env, "tlhip: ops must be an array");
  napi_get_array_length(env, a[11], &count);
  if (count > TLHIP_MAX_EPILOGUE_OPS) return throw_type(env, "tlhip: too many epilogue ops");
  tlhip_epilogue_t ep;
  memset(&ep, 0, sizeof ep);
  for (uint32_t i = 0; i < count; ++i) {
    napi_value row, f[5];
    uint32_t len = 0;
    napi_get_element(env, a[11], i, &row);
    if (napi_is_array(env, row, &is_array) != napi_ok || !is_array) return throw_type(env, "tlhip: an op is [kind, unary, input, inputDtype, inputRows]");
    napi_get_array_length(env, row, &len);
    if (len != 5) return throw_type(env, "tlhip: an op is [kind, unary, input, inputDtype, inputRows]");
    for (uint32_t j = 0; j < 5; ++j) napi_get_element(env, row, j, &f[j]);
    int32_t kind, unary, idt, rows;
    void* input;
    if (!get_i32(env, f[0], &kind) || !get_i32(env, f[1], &unary) || !get_ptr(env, f[2], &input) || !get_i32(env, f[3], &idt) ||
        !get_i32(env, f[4], &rows))
      return throw_type(env, "tlhip: an op is [kind, unary, input, inputDtype, inputRows]");
    ep.ops[i].kind = kind;
    ep.ops[i].unary = unary;
    ep.ops[i].input = input;
    ep.ops[i].input_dtype = idt;
    ep.ops[i].rows = rows;
  }
  ep.n_ops = (int32_t)count;
  CHECK(tlhip_matmul_quantized(&w, x, xd, m, y, yd, 1.0f, count ? &ep : NULL, NULL));
  return undefined(env);
}
/* gemvPrologue(format, groupSize, n, k, packed, scales, xPtr, xDtype, m, yPtr, yDtype,
 *              biasPtr | null, biasDtype, unary, kind, operandPtr, proUnary, eps)
 * -> true, or false when no fused kernel covers the request (run the steps apart). */
static napi_value GemvPrologue(napi_env env, napi_callback_info info) {
  ARGS(18);
  WEIGHT(0, w);
  PTR(6, x);
  I32(7, xd);
  I64(8, m);
  PTR(9, y);
  I32(10, yd);
  PTR(11, bias);
  I32(12, bd);
  I32(13, un);
  I32(14, kind);
  PTR(15, operand);
  I32(16, pro_unary);
  F64(17, eps);
  tlhip_epilogue_t ep;
  make_epilogue(bias, bd, un, &ep);
  tlhip_prologue_t pro;
  memset(&pro, 0, sizeof pro);
  pro.kind = kind;
  pro.unary = pro_unary;
  pro.eps = (float)eps;
  pro.operand = operand;
  const int rc = tlhip_gemv_prologue(&w, &pro, x, xd, m, y, yd, 1.0f, ep.n_ops ? &ep : NULL, NULL);
  napi_value b;
  if (rc == TLHIP_ERR_UNSUPPORTED) {
    napi_get_boolean(env, false, &b);
    return b;
  }
  CHECK(rc);
  napi_get_boolean(env, true, &b);
  return b;
}
/* A JavaScript array of problems [format, groupSize, n, k, packed, scales, xPtr, yPtr, biasPtr|null,
 * biasDtype, unary] -> tlhip_gemv_problem_t[count]; NULL (with a pending exception) on a bad one. */
static const char* parse_problems(napi_env env, napi_value arr, tlhip_gemv_problem_t* probs, tlhip_epilogue_t* eps,
                                  uint32_t* count_out) {
  uint32_t count = 0;
  bool is_array = false;
  if (napi_is_array(env, arr, &is_array) != napi_ok || !is_array) return "tlhip: gemvGrouped needs an array of problems";
  napi_get_array_length(env, arr, &count);
  if (count > 4) return "tlhip: a group holds at most 4 problems";
  for (uint32_t i = 0; i < count; ++i) {
    napi_value row, f[11];
    uint32_t len = 0;
    napi_get_element(env, arr, i, &row);
    if (napi_is_array(env, row, &is_array) != napi_ok || !is_array) return "tlhip: a problem is an array of 11";
    napi_get_array_length(env, row, &len);
    if (len != 11) return "tlhip: a problem is an array of 11";
    for (uint32_t j = 0; j < 11; ++j) napi_get_element(env, row, j, &f[j]);
    if (!get_weight(env, f, &probs[i].w)) return "tlhip: bad weight in problem";
    void *x, *y, *bias;
    int32_t bd, un;
    if (!get_ptr(env, f[6], &x) || !get_ptr(env, f[7], &y) || !get_ptr(env, f[8], &bias) || !get_i32(env, f[9], &bd) ||
        !get_i32(env, f[10], &un))
      return "tlhip: bad problem fields";
    make_epilogue(bias, bd, un, &eps[i]);
    probs[i].x = x;
    probs[i].y = y;
    probs[i].epilogue = eps[i].n_ops ? &eps[i] : NULL;
  }
  *count_out = count;
  return NULL;
}
/* gemvGrouped([ [format, groupSize, n, k, packed, scales, xPtr, yPtr, biasPtr|null, biasDtype, unary], ... ],
 *             xDtype, yDtype [, kind, operandPtr, proUnary, eps]) */
static napi_value GemvGrouped(napi_env env, napi_callback_info info) {
  ARGS(3);
  I32(1, xd);
  I32(2, yd);
  tlhip_gemv_problem_t probs[4];
  tlhip_epilogue_t eps[4];
  uint32_t count = 0;
  const char* bad = parse_problems(env, a[0], probs, eps, &count);
  if (bad) return throw_type(env, bad);
  if (argc >= 7) {
    I32(3, kind);
    PTR(4, operand);
    I32(5, pro_unary);
    F64(6, eps_value);
    tlhip_prologue_t pro;
    memset(&pro, 0, sizeof pro);
    pro.kind = kind;
    pro.unary = pro_unary;
    pro.eps = (float)eps_value;
    pro.operand = operand;
    CHECK(tlhip_gemv_grouped_prologue(probs, (int)count, &pro, xd, yd, 1.0f, NULL));
  } else {
    CHECK(tlhip_gemv_grouped(probs, (int)count, xd, yd, 1.0f, NULL));
  }
  return undefined(env);
}
/* gemvGroupedRows(problems as for gemvGrouped, xDtype, m, yDtype): m <= 16 rows on shared activations */
static napi_value GemvGroupedRows(napi_env env, napi_callback_info info) {
  ARGS(4);
  I32(1, xd);
  I64(2, m);
  I32(3, yd);
  tlhip_gemv_problem_t probs[4];
  tlhip_epilogue_t eps[4];
  uint32_t count = 0;
  const char* bad = parse_problems(env, a[0], probs, eps, &count);
  if (bad) return throw_type(env, bad);
  CHECK(tlhip_gemv_grouped_rows(probs, (int)count, xd, m, yd, 1.0f, NULL));
  return undefined(env);
}
/* gemvNoalloc(format, groupSize, n, k, packed, scales, xPtr, xDtype, m, yPtr, yDtype, biasPtr | null, biasDtype, unary):
 * tlhip_gemv without any allocation (for callers under graph capture) */
static napi_value GemvNoalloc(napi_env env, napi_callback_info info) {
  ARGS(14);
  WEIGHT(0, w);
  PTR(6, x);
  I32(7, xd);
  I64(8, m);
  PTR(9, y);
  I32(10, yd);
  PTR(11, bias);
  I32(12, bd);
  I32(13, un);
  tlhip_epilogue_t ep;
  make_epilogue(bias, bd, un, &ep);
  CHECK(tlhip_gemv_noalloc(&w, x, xd, m, y, yd, 1.0f, ep.n_ops ? &ep : NULL, NULL));
  return undefined(env);
}
/* [format, groupSize, n, k, packed, scales] as one array argument. */
static int get_weight_array(napi_env env, napi_value arr, tlhip_qweight_t* w) {
  bool is_array = false;
  uint32_t len = 0;
  napi_value f[6];
  if (napi_is_array(env, arr, &is_array) != napi_ok || !is_array) return 0;
  napi_get_array_length(env, arr, &len);
  if (len != 6) return 0;
  for (uint32_t j = 0; j < 6; ++j) napi_get_element(env, arr, j, &f[j]);
  return get_weight(env, f, w);
}
/* mlpDecode(gate, up, down (each [format, groupSize, n, k, packed, scales]), unary, xPtr, xDtype, m, hPtr, yPtr, yDtype):
 * y = (unary(x gate^T) * (x up^T)) down^T in one launch; h is the caller's f16 [m, gate.n] */
static napi_value MlpDecode(napi_env env, napi_callback_info info) {
  ARGS(10);
  tlhip_qweight_t gate, up, down;
  if (!get_weight_array(env, a[0], &gate) || !get_weight_array(env, a[1], &up) || !get_weight_array(env, a[2], &down))
    return throw_type(env, "tlhip: mlpDecode takes three weights as [format, groupSize, n, k, packed, scales]");
  I32(3, un);
  PTR(4, x);
  I32(5, xd);
  I64(6, m);
  PTR(7, h);
  PTR(8, y);
  I32(9, yd);
  CHECK(tlhip_mlp_decode(&gate, &up, &down, un, x, xd, m, h, y, yd, NULL, NULL));
  return undefined(env);
}
/* sequenceStatus(): waits for the library stream; throws if a sequence launch gave up a wait */
static napi_value SequenceStatus(napi_env env, napi_callback_info info) {
  (void)info;
  int error = 0;
  CHECK(tlhip_sequence_status(NULL, &error));
  return make_num(env, (double)error);
}
/* biasAdd(inPtr, dtype, biasPtr, biasDtype, outPtr, m, n) */
static napi_value BiasAdd(napi_env env, napi_callback_info info) {
  ARGS(7);
  PTR(0, in);
  I32(1, dt);
  PTR(2, bias);
  I32(3, bd);
  PTR(4, out);
  I64(5, m);
  I64(6, n);
  CHECK(tlhip_bias_add(in, dt, bias, bd, out, m, n, NULL));
  return undefined(env);
}
/* unary(op, inPtr, dtype, outPtr, count) */
static napi_value Unary(napi_env env, napi_callback_info info) {
  ARGS(5);
  I32(0, op);
  PTR(1, in);
  I32(2, dt);
  PTR(3, out);
  I64(4, count);
  CHECK(tlhip_unary(op, in, dt, out, count, NULL));
  return undefined(env);
}
/* cast(inPtr, inDtype, outPtr, outDtype, count) */
static napi_value Cast(napi_env env, napi_callback_info info) {
  ARGS(5);
  PTR(0, in);
  I32(1, idt);
  PTR(2, out);
  I32(3, odt);
  I64(4, count);
  CHECK(tlhip_cast(in, idt, out, odt, count, NULL));
  return undefined(env);
}
/* rmsnorm(xPtr, xDtype, weightPtr, yPtr, yDtype, rows, d, eps) */
static napi_value RmsNorm(napi_env env, napi_callback_info info) {
  ARGS(8);
  PTR(0, x);
  I32(1, xd);
  PTR(2, w);
  PTR(3, y);
  I32(4, yd);
  I64(5, rows);
  I64(6, d);
  F64(7, eps);
  CHECK(tlhip_rmsnorm(x, xd, (const float*)w, y, yd, rows, d, (float)eps, NULL));
  return undefined(env);
}
/* gatedMul(unary, gatePtr, upPtr, dtype, outPtr, count) */
static napi_value GatedMul(napi_env env, napi_callback_info info) {
  ARGS(6);
  I32(0, op);
  PTR(1, gate);
  PTR(2, up);
  I32(3, dt);
  PTR(4, out);
  I64(5, count);
  CHECK(tlhip_gated_mul(op, gate, up, dt, out, count, NULL));
  return undefined(env);
}
/* topk(logitsPtr, offset, length, k, valuesPtr, indicesPtr, indexDtype) */
static napi_value TopK(napi_env env, napi_callback_info info) {
  ARGS(7);
  PTR(0, logits);
  I64(1, offset);
  I64(2, length);
  I32(3, k);
  PTR(4, values);
  PTR(5, indices);
  I32(6, idt);
  CHECK(tlhip_topk((const float*)logits, offset, length, k, (float*)values, indices, idt, NULL));
  return undefined(env);
}

/* ------------------------------------------------------------ kernel choice */
static napi_value config_to_js(napi_env env, const tlhip_kernel_config_t* c) {
  napi_value ab, arr;
  void* data;
  napi_create_arraybuffer(env, sizeof *c, &data, &ab);
  memcpy(data, c, sizeof *c);
  napi_create_typedarray(env, napi_int32_array, 8, ab, 0, &arr);
  return arr;
}
/* selectedConfig(format, groupSize, n, k, packed, scales, xDtype, m, yDtype) -> Int32Array(8) */
static napi_value SelectedConfig(napi_env env, napi_callback_info info) {
  ARGS(9);
  WEIGHT(0, w);
  I32(6, xd);
  I64(7, m);
  I32(8, yd);
  tlhip_kernel_config_t c;
  CHECK(tlhip_selected_config(&w, xd, m, yd, &c));
  return config_to_js(env, &c);
}
/* candidates(format, groupSize, n, k, packed, scales, xDtype, m, yDtype) -> [Int32Array(8), ...] */
static napi_value Candidates(napi_env env, napi_callback_info info) {
  ARGS(9);
  WEIGHT(0, w);
  I32(6, xd);
  I64(7, m);
  I32(8, yd);
  int count = 0;
  CHECK(tlhip_candidate_count(&w, xd, m, yd, &count));
  napi_value arr;
  napi_create_array_with_length(env, (size_t)count, &arr);
  for (int i = 0; i < count; ++i) {
    tlhip_kernel_config_t c;
    CHECK(tlhip_candidate_get(&w, xd, m, yd, i, &c));
    napi_set_element(env, arr, (uint32_t)i, config_to_js(env, &c));
  }
  return arr;
}
/* autotune(format, groupSize, n, k, packed, scales, xPtr, xDtype, m, yPtr, yDtype) -> best us */
static napi_value Autotune(napi_env env, napi_callback_info info) {
  ARGS(11);
  WEIGHT(0, w);
  PTR(6, x);
  I32(7, xd);
  I64(8, m);
  PTR(9, y);
  I32(10, yd);
  double us = 0;
  CHECK(tlhip_autotune(&w, x, xd, m, y, yd, &us));
  return make_num(env, us);
}
/* tuneCacheSeed(format, groupSize, n, k, packed, scales, xDtype, m, yDtype, config: Int32Array(8)) */
static napi_value TuneCacheSeed(napi_env env, napi_callback_info info) {
  ARGS(10);
  WEIGHT(0, w);
  I32(6, xd);
  I64(7, m);
  I32(8, yd);
  void* cdata;
  size_t cbytes;
  if (!get_bytes(env, a[9], &cdata, &cbytes) || cbytes != sizeof(tlhip_kernel_config_t))
    return throw_type(env, "tlhip: config must be an Int32Array of 8");
  CHECK(tlhip_tune_cache_seed(&w, xd, m, yd, (const tlhip_kernel_config_t*)cdata));
  return undefined(env);
}
static napi_value SetAutotuneEnabled(napi_env env, napi_callback_info info) {
  ARGS(1);
  bool on = false;
  napi_coerce_to_bool(env, a[0], &a[0]);
  napi_get_value_bool(env, a[0], &on);
  CHECK(tlhip_set_autotune_enabled(on ? 1 : 0));
  return undefined(env);
}
static napi_value IsAutotuneEnabled(napi_env env, napi_callback_info info) {
  (void)info;
  napi_value b;
  napi_get_boolean(env, tlhip_is_autotune_enabled() != 0, &b);
  return b;
}
/* pretuneMatmulShapes(flat [m, n, k, m, n, k, ...]) */
static napi_value PretuneMatmulShapes(napi_env env, napi_callback_info info) {
  ARGS(1);
  uint32_t len = 0;
  bool is_array = false;
  if (napi_is_array(env, a[0], &is_array) != napi_ok || !is_array) return throw_type(env, "tlhip: pretuneMatmulShapes needs a flat array");
  napi_get_array_length(env, a[0], &len);
  if (len % 3 != 0) return throw_type(env, "tlhip: pretuneMatmulShapes: [m, n, k] triples");
  int64_t* mnk = (int64_t*)malloc(sizeof(int64_t) * (len ? len : 1));
  for (uint32_t i = 0; i < len; ++i) {
    napi_value e;
    napi_get_element(env, a[0], i, &e);
    if (!get_i64(env, e, &mnk[i])) {
      free(mnk);
      return throw_type(env, "tlhip: pretuneMatmulShapes: numbers only");
    }
  }
  const int rc = tlhip_pretune_matmul_shapes(mnk, (int)(len / 3));
  free(mnk);
  CHECK(rc);
  return undefined(env);
}
static napi_value TuneCacheExport(napi_env env, napi_callback_info info) {
  (void)info;
  size_t need = 0;
  CHECK(tlhip_tune_cache_export(NULL, 0, &need));
  char* buf = (char*)malloc(need + 1);
  const int rc = tlhip_tune_cache_export(buf, need + 1, &need);
  if (rc) {
    free(buf);
    return throw_last(env, rc);
  }
  napi_value s;
  napi_create_string_utf8(env, buf, NAPI_AUTO_LENGTH, &s);
  free(buf);
  return s;
}
static napi_value TuneCacheImport(napi_env env, napi_callback_info info) {
  ARGS(1);
  size_t len = 0;
  if (napi_get_value_string_utf8(env, a[0], NULL, 0, &len) != napi_ok) return throw_type(env, "tlhip: tuneCacheImport needs a string");
  char* buf = (char*)malloc(len + 1);
  napi_get_value_string_utf8(env, a[0], buf, len + 1, &len);
  const int rc = tlhip_tune_cache_import(buf);
  free(buf);
  CHECK(rc);
  return undefined(env);
}
static napi_value TuneCacheClear(napi_env env, napi_callback_info info) {
  (void)info;
  CHECK(tlhip_tune_cache_clear());
  return undefined(env);
}
static napi_value Counter(napi_env env, napi_callback_info info) {
  ARGS(1);
  char name[64];
  size_t len = 0;
  if (napi_get_value_string_utf8(env, a[0], name, sizeof name, &len) != napi_ok) return throw_type(env, "tlhip: counter needs a name");
  return make_num(env, (double)tlhip_counter(name));
}
static napi_value CountersReset(napi_env env, napi_callback_info info) {
  (void)info;
  CHECK(tlhip_counters_reset());
  return undefined(env);
}

NAPI_MODULE_INIT() {
#define FN(name, fn) {name, 0, fn, 0, 0, 0, napi_enumerable, 0}
  const napi_property_descriptor d[] = {
      FN("init", Init), FN("shutdown", Shutdown), FN("deviceInfo", DeviceInfo), FN("malloc", Malloc), FN("free", Free),
      FN("memset", Memset), FN("memcpyH2D", MemcpyH2D), FN("memcpyD2H", MemcpyD2H), FN("memcpyD2D", MemcpyD2D),
      FN("synchronize", Synchronize), FN("graphBeginCapture", GraphBeginCapture),
      FN("graphEndCapture", GraphEndCapture), FN("graphLaunch", GraphLaunch), FN("graphDestroy", GraphDestroy),
      FN("f32ToF16Bits", F32ToF16Bits), FN("f16BitsToF32", F16BitsToF32),
      FN("quantizeInt8Grouped", QuantizeInt8Grouped), FN("quantizeInt8GroupedDevice", QuantizeInt8GroupedDevice),
      FN("dequant", Dequant), FN("matmulQuantized", MatmulQuantized), FN("matmulQuantizedOps", MatmulQuantizedOps), FN("gemvPrologue", GemvPrologue),
      FN("gemvGrouped", GemvGrouped), FN("gemvGroupedRows", GemvGroupedRows), FN("gemvNoalloc", GemvNoalloc), FN("mlpDecode", MlpDecode), FN("sequenceStatus", SequenceStatus), FN("biasAdd", BiasAdd), FN("unary", Unary), FN("cast", Cast),
      FN("rmsnorm", RmsNorm), FN("gatedMul", GatedMul), FN("topk", TopK), FN("selectedConfig", SelectedConfig),
      FN("candidates", Candidates), FN("autotune", Autotune), FN("tuneCacheSeed", TuneCacheSeed),
      FN("setAutotuneEnabled", SetAutotuneEnabled), FN("isAutotuneEnabled", IsAutotuneEnabled),
      FN("pretuneMatmulShapes", PretuneMatmulShapes), FN("tuneCacheExport", TuneCacheExport),
      FN("tuneCacheImport", TuneCacheImport), FN("tuneCacheClear", TuneCacheClear), FN("counter", Counter),
      FN("countersReset", CountersReset),
  };
#undef FN
  napi_define_properties(env, exports, sizeof d / sizeof d[0], d);
  return exports;
}
