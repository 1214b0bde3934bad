/*
 * tlhip.h — C ABI of the MI355X (gfx950) `hip` backend for torchlette's
 * quantized-weight linear path.
 *
 * This is the boundary a torchlette `Backend` object binds through a Node
 * N-API addon (or any FFI): plain pointers, sizes and enums, no C++ or torch
 * types.  Each entry point cites the reference interface it stands in for
 * (paths relative to the torchlette source tree).
 *
 * Conventions
 *  - Every function that can fail returns int: 0 = ok, non-zero = error.  The
 *    message is kept per thread and read with tlhip_last_error(); a binding
 *    turns non-zero into `throw new Error(msg)`, the reference's only error
 *    channel (src/backend/webgpu/ops/matmul-ops.ts:121-126).
 *  - Pointers are DEVICE pointers unless the parameter name starts with host_.
 *  - Work is enqueued on `stream` in order, as WebGPU queue submission is
 *    (one JavaScript thread, ops enqueue, only `read` waits).  NULL means the
 *    library's own stream, created by tlhip_init.
 *  - There is no CPU fallback: without a usable gfx950 device every compute
 *    entry point fails with an error.
 */
#ifndef TLHIP_H
#define TLHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TLHIP_OK 0
#define TLHIP_ERR_INVALID 1 /* bad argument / unsupported combination */
#define TLHIP_ERR_DEVICE 2  /* a HIP call failed */
#define TLHIP_ERR_STATE 3   /* library not initialised */
#define TLHIP_ERR_UNSUPPORTED 4 /* valid request that no built kernel covers; the caller has a fallback */

typedef void* tlhip_stream_t;
typedef void* tlhip_event_t;
typedef void* tlhip_graph_t;

/* Storage format of a packed weight: the values of
 * StorageFormat.packing.scheme (src/backend/types.ts:46-55).  INT8_GROUPED is
 * the reference's "int8-grouped"; INT4_GROUPED is the value its design doc
 * plans (docs/quantization-design.md:69-75); INT8_ROW is int8 with one f32
 * scale per output row (same byte packing, quantize.ts:121-125). */
typedef enum {
  TLHIP_FMT_INT8_GROUPED = 0, /* u32 [N,K/4]; f16 abs-max per group; w=(q/127)*s */
  TLHIP_FMT_INT8_ROW = 1,     /* u32 [N,K/4]; f32 scale per row;      w=q*s      */
  TLHIP_FMT_INT4_GROUPED = 2  /* u32 [N,K/8]; f16 scale per group;    w=q*s      */
} tlhip_format_t;

/* DType subset used on this path (src/backend/types.ts DType "f32" | "f16"). */
typedef enum { TLHIP_F32 = 0, TLHIP_F16 = 1, TLHIP_I32 = 2 } tlhip_dtype_t;

/* Unary epilogue ops: the GEMV epilogue vocabulary
 * (src/backend/webgpu/matmul/gemv.ts:135-143); formulas from
 * src/ops/semantic/catalog.ts:81-109 and composite.ts:40-65. */
typedef enum {
  TLHIP_UNARY_NONE = 0,
  TLHIP_UNARY_RELU = 1,
  TLHIP_UNARY_SILU = 2,
  TLHIP_UNARY_GELU_TANH = 3, /* the reference's "gelu" / "gelu_tanh" */
  TLHIP_UNARY_GELU_ERF = 4,
  TLHIP_UNARY_SIGMOID = 5,
  TLHIP_UNARY_TANH = 6
} tlhip_unary_t;

typedef enum {
  TLHIP_EPI_NONE = 0,
  TLHIP_EPI_BIAS = 1,
  TLHIP_EPI_UNARY = 2,
  TLHIP_EPI_BINARY = 3,  /* add / sub / mul with an [M,N] input, indexed by output element */
  TLHIP_EPI_CAST_F16 = 4 /* {kind: "cast", toDtype: "f16"}: the value is rounded to f16 at this point of the chain */
} tlhip_epilogue_kind_t;

/* The op of a BINARY step (`op` of {kind: "binary"}: "add", "sub", "mul";
 * src/schedule/matmul-skeleton.ts:934-955). */
typedef enum { TLHIP_BINARY_ADD = 0, TLHIP_BINARY_SUB = 1, TLHIP_BINARY_MUL = 2 } tlhip_binary_t;

#define TLHIP_MAX_EPILOGUE_OPS 4

/* One step of an epilogue chain: EpilogueOp
 * (src/backend/webgpu/matmul/types.ts:13-24).  BIAS adds input[n] (indexed by
 * output column); UNARY applies `unary`; BINARY combines the value with
 * input[m*N + n] (an [M,N] tensor, contiguous: value + input, value - input or
 * value * input; a residual add, a gate); CAST_F16 rounds the value to f16.
 * The reference's op names a typed tensor (`inputIndex`); the C ABI sees a pointer, so
 * the caller states the input's shape in `rows` ([rows, N], contiguous) and every entry
 * point refuses, before any launch, a BIAS whose rows is not 1 and a BINARY whose rows is
 * not the call's m (TLHIP_ERR_INVALID): the kernels index a BINARY input by output
 * element, and a shorter buffer would be read past its end. */
typedef struct {
  int32_t kind;        /* tlhip_epilogue_kind_t */
  int32_t unary;       /* tlhip_unary_t for kind == UNARY, tlhip_binary_t for kind == BINARY */
  const void* input;   /* device [N] for kind == BIAS, device [M,N] for kind == BINARY */
  int32_t input_dtype; /* tlhip_dtype_t of input (f32 or f16) */
  int32_t rows;        /* rows of input: 1 for BIAS, the call's m for BINARY; ignored otherwise */
} tlhip_epilogue_op_t;

/* EpilogueConfig: ops are applied in order to acc*alpha in f32, then the value
 * is cast to the output dtype (src/schedule/matmul-skeleton.ts:916-966). */
typedef struct {
  int32_t n_ops;
  int32_t reserved;
  tlhip_epilogue_op_t ops[TLHIP_MAX_EPILOGUE_OPS];
} tlhip_epilogue_t;

/* The checks every compute entry point makes on (weight, m, epilogue) before it launches
 * anything, on their own: needs no device and no tlhip_init.  TLHIP_OK or
 * TLHIP_ERR_INVALID with the message in tlhip_last_error. */
/* A packed weight operand: what BackendTensor.format + .scales describe
 * (src/backend/types.ts:5-28) for the logical [N,K] Linear weight.
 *   packed  u32 words, row-major [N, K/4] (int8) or [N, K/8] (int4)
 *   scales  INT8_GROUPED/INT4_GROUPED: f16 bit patterns [N, K/G], contiguous
 *           (the reference's two-per-u32 upload, engine.ts:2077-2087, is the
 *           same bytes);  INT8_ROW: f32 [N] */
/* Limits.  packed and scales are 16-byte aligned.  K <= 2^24, N <= 2^30.  The decode
 * kernels keep activation rows in LDS: K <= 57344 for f16 activations, K <= 28672 for f32
 * activations (longer rows: TLHIP_ERR_INVALID).  For the grouped formats the prefill
 * GEMMs (m > 16) round each dequantised weight q*s once to f16 before the matrix cores,
 * so |q*s| must stay inside f16's normal range: scales between 6.2e-5 / 1 and 65504 / 8
 * (int4) or 65504 / 127 (int8-grouped).  The decode kernels (m <= 16) apply the scale in
 * f32 and have no such limit, and neither has INT8_ROW at any m (its prefill GEMMs
 * multiply the bare integers and apply the row's scale to the f32 sums). */
typedef struct {
  int32_t format;     /* tlhip_format_t */
  int32_t group_size; /* G along K; ignored for INT8_ROW */
  int64_t n;
  int64_t k;
  const void* packed;
  const void* scales;
} tlhip_qweight_t;

int tlhip_epilogue_check(const tlhip_qweight_t* w, int64_t m, const tlhip_epilogue_t* epilogue);

typedef struct {
  char name[64];     /* device name */
  char arch[32];     /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
  int32_t compute_units;
  int32_t wavefront_size;
  int32_t lds_bytes_per_block;
  int32_t clock_khz;
  int32_t memory_clock_khz;
  int32_t memory_bus_bits;
  int64_t total_memory_bytes;
  int64_t l2_bytes;
} tlhip_device_info_t;

/* ---- runtime: what the WebGPU context/queue provides to the reference
 * backend (src/backend/webgpu/gpu-context.ts; creation.ts:51-87; `read`). ---- */
/* tlhip_init also imports the tuning file that ships next to the library
 * (<directory of libtlhip.so>/tuning/mi355x.json; the environment variable
 * TLHIP_TUNING_FILE names another file, "none" none), as importTuningCache would:
 * every binding runs the committed kernel choices, re-gated on applicability.
 * The library serves ONE device per process, the one given here, and makes it the
 * calling thread's current HIP device; a thread that calls the library later must
 * have the same device current (allocations and launches go to the current device). */
int tlhip_init(int device_index);
int tlhip_shutdown(void);
const char* tlhip_last_error(void);
int tlhip_device_info(tlhip_device_info_t* host_out);
int tlhip_malloc(size_t bytes, void** host_out_ptr);
int tlhip_free(void* ptr);
int tlhip_memset(void* ptr, int value, size_t bytes, tlhip_stream_t stream);
int tlhip_memcpy_h2d(void* dst, const void* host_src, size_t bytes, tlhip_stream_t stream);
int tlhip_memcpy_d2h(void* host_dst, const void* src, size_t bytes, tlhip_stream_t stream);
int tlhip_memcpy_d2d(void* dst, const void* src, size_t bytes, tlhip_stream_t stream);
int tlhip_host_alloc(size_t bytes, void** host_out_ptr); /* pinned */
int tlhip_host_free(void* host_ptr);
int tlhip_stream_create(tlhip_stream_t* host_out);
int tlhip_stream_destroy(tlhip_stream_t stream);
int tlhip_stream_synchronize(tlhip_stream_t stream);
int tlhip_event_create(tlhip_event_t* host_out);
int tlhip_event_destroy(tlhip_event_t ev);
int tlhip_event_record(tlhip_event_t ev, tlhip_stream_t stream);
int tlhip_event_synchronize(tlhip_event_t ev);
int tlhip_event_elapsed_us(tlhip_event_t start, tlhip_event_t stop, double* host_out_us);

/* Record the work enqueued on `stream` between begin and end into a graph that
 * can be replayed with one call.  The reference batches a decode step's
 * dispatches into one command-buffer submission
 * (src/backend/webgpu/shared-encoder.ts); a captured graph is the HIP
 * counterpart.  Rules:
 *  - the compute entry points enqueue kernels only, so all of them may be captured;
 *    tlhip_memset returns TLHIP_ERR_STATE on a capturing stream, and lazy autotuning
 *    is skipped there;
 *  - a kernel that splits K across workgroups (and tlhip_topk) works through the
 *    stream's workspace, which is created on the stream's first such call: make that
 *    call once before capturing, or the call under capture returns TLHIP_ERR_STATE
 *    (tlhip_gemv_noalloc never needs this);
 *  - the workspace pointers are part of the captured kernels' arguments: a graph
 *    replays on the stream it was captured on (another stream: TLHIP_ERR_INVALID),
 *    in order with that stream's other launches; the workspace stays allocated until
 *    the stream AND every graph captured on it are destroyed; tlhip_shutdown destroys
 *    graphs that are still alive;
 *  - a replay that is aborted half-way (device reset) can leave arrival counters
 *    non-zero; nothing short of tlhip_shutdown / tlhip_init clears them. */
int tlhip_graph_begin_capture(tlhip_stream_t stream);
int tlhip_graph_end_capture(tlhip_stream_t stream, tlhip_graph_t* host_out);
int tlhip_graph_launch(tlhip_graph_t graph, tlhip_stream_t stream);
int tlhip_graph_destroy(tlhip_graph_t graph);

/* ---- host-side weight preparation: src/backend/quantize.ts ---- */
/* f32ToF16Bits (quantize.ts:22-47), including its round-half-up subnormals. */
uint16_t tlhip_f32_to_f16_bits(float value);
/* f16BitsToF32 (quantize.ts:50-60). */
float tlhip_f16_bits_to_f32(uint16_t bits);
/* quantizeLinearWeight (quantize.ts:77-131).  Host in, host out:
 * host_packed u32[n*k/4] (overwritten), host_scales u16[n*k/group_size].
 * Fails if k%4 != 0 or k%group_size != 0, with the reference's messages. */
int tlhip_quantize_int8_grouped(const float* host_weight, int64_t n, int64_t k, int64_t group_size,
                                uint32_t* host_packed, uint16_t* host_scales);

/* The same quantizer on the device, for weights already resident in HBM
 * (quantize-at-load, examples/qwen3/loader.ts:228-254): `weight` f32 [n,k],
 * `packed` u32 [n,k/4], `scales` u16 [n,k/group_size], all device pointers.
 * Bit-identical to tlhip_quantize_int8_grouped.  group_size must also be a
 * multiple of 4 here. */
int tlhip_quantize_int8_grouped_device(const float* weight, int64_t n, int64_t k, int64_t group_size,
                                       uint32_t* packed, uint16_t* scales, tlhip_stream_t stream);

/* ---- compute ---- */

/* Explicit dequantisation to f32 [N,K], bit-exact against dequantizeToF32
 * (quantize.ts:138-156) for INT8_GROUPED and against f32(q*s) for the other
 * two formats.  Stands in for dispatchDequantizeInt8Grouped
 * (src/backend/webgpu/matmul/dispatch.ts:949-1037). */
int tlhip_dequant(const tlhip_qweight_t* w, float* out, tlhip_stream_t stream);

/* Decode GEMV / skinny GEMM with fused dequant: y[m,n] = epilogue(alpha *
 * sum_k x[m,k] * w[n,k]), 1 <= m <= 16, f32 accumulation.  x is row-major
 * [m,k] of x_dtype, y row-major [m,n] of y_dtype.  Stands in for
 * dispatchQuantizedGemvNT (dispatch.ts:875-931), extended to m <= 16, f16
 * activations/outputs and the epilogue chain.  epilogue may be NULL. */
int tlhip_gemv(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y,
               int y_dtype, float alpha, const tlhip_epilogue_t* epilogue, tlhip_stream_t stream);

/* tlhip_gemv for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, kernels and results as tlhip_gemv,
 * but where tlhip_gemv combines K slices of different workgroups through a workspace
 * the library allocates on a stream's first use, this entry point uses a fixed
 * device array inside the library (4 MiB of partial tiles + 4096 counters per GPU,
 * resolved at tlhip_init) and calls no hipMalloc / hipFree.  A problem whose
 * configuration needs more (output rows / 16 * K slices * 1 KiB above 4 MiB, or more
 * than 65536 output rows with K slices) fails with TLHIP_ERR_INVALID.  All calls on a
 * GPU share the array: calls that overlap on one GPU (two streams, or a replaying
 * graph next to eager calls) race. */
int tlhip_gemv_noalloc(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y,
                       int y_dtype, float alpha, const tlhip_epilogue_t* epilogue,
                       tlhip_stream_t stream);

/* Up to 4 decode GEMVs of one shape class in ONE launch (q/k/v or gate/up of a
 * decode step: the frontend issues them back to back on the same activations,
 * src/frontend/torchlette.ts:878-894 once per Linear, and each is too small to
 * fill the chip while every launch costs 2-3 us).  All problems: m = 1, f16
 * activations, the same format, group size, K and output type; N, pointers and
 * epilogues are per problem.  Results are those of `count` tlhip_gemv calls.
 * Falls back to separate launches when the selected kernel configuration has no
 * grouped form. */
typedef struct {
  tlhip_qweight_t w;
  const void* x;
  void* y;
  const tlhip_epilogue_t* epilogue; /* may be NULL */
} tlhip_gemv_problem_t;
int tlhip_gemv_grouped(const tlhip_gemv_problem_t* problems, int count, int x_dtype, int y_dtype, float alpha,
                       tlhip_stream_t stream);
/* The same for a batched decode step: every problem has `m` (<= 16) activation rows.
 * Problems that share ONE activation pointer (q/k/v on the normed hidden state,
 * gate/up; packages/qwen3-browser/src/model.ts:341-361) run as one launch of the
 * matrix-core kernels when the configuration selected for their combined rows is one of
 * theirs (variants gemv_mfma and gemv_mfma_xreg: f16 activations); anything else runs as
 * separate launches (m = 1: as the VALU kernel's grouped launch).  Results are those of `count` tlhip_gemv calls. */
int tlhip_gemv_grouped_rows(const tlhip_gemv_problem_t* problems, int count, int x_dtype, int64_t m,
                            int y_dtype, float alpha, tlhip_stream_t stream);

/* A SEQUENCE of decode Linears in ONE launch.  The reference issues a decoder layer's
 * Linears one after the other, each its own dispatch, with the elementwise op of the MLP
 * between them (packages/qwen3-browser/src/model.ts:341-361: q/k/v, o, then
 * down(mul(silu(gate(x)), up(x))); packages/gemma2-browser/src/model.ts:411-415 with gelu);
 * at decode sizes every launch costs as much as the weights it streams.  Here up to 16 steps
 * run as one launch: the weight stream never stops between them, and a step whose
 * activations (or epilogue inputs) are written by an earlier step of the call (`wait`) is
 * ordered behind ALL earlier steps inside the kernel.  A step without `wait` must not read
 * or write anything an earlier step of the call writes, nor write what one reads.
 * A GATED step computes y = epilogue(x w^T) * (x w_up^T) on two weights of one shape (the
 * MLP's act(gate) * up: the epilogue carries the activation) and writes only the product.
 * All steps: int4 weights with group size 32, K a multiple of 256 up to 12288, f16
 * activations, the same m <= 16; anything else is
 * TLHIP_ERR_UNSUPPORTED (run the steps through tlhip_gemv instead).  Results are those of
 * the same steps through tlhip_gemv (f32 accumulation of exact products: the order of the
 * sums differs), bit-identical from launch to launch.
 * The waits inside the kernel are bounded: if one expires (it cannot while every workgroup
 * of the launch is resident, which the library ensures by launching one workgroup per CU)
 * the kernel sets an error word and leaves; tlhip_sequence_status reports it.  Like a
 * K-sliced GEMV, a stream's first sequence call must not happen under graph capture. */
typedef struct {
  tlhip_qweight_t w;      /* the weight; of a gated step: the gate projection */
  tlhip_qweight_t w_up;   /* gated steps only: the up projection (same format and shape as w) */
  const void* x;          /* device [m, K] f16 */
  void* y;                /* device [m, N] */
  const tlhip_epilogue_t* epilogue; /* may be NULL; gated: applied to the gate side */
  int32_t y_dtype;        /* tlhip_dtype_t of y (f16 or f32) */
  int32_t gated;          /* nonzero: y = epilogue(x w^T) * (x w_up^T) */
  int32_t wait;           /* nonzero: starts only when all earlier steps of the call are complete */
  int32_t reserved;
} tlhip_sequence_step_t;
int tlhip_gemv_sequence(const tlhip_sequence_step_t* steps, int count, int x_dtype, int64_t m, float alpha,
                        tlhip_stream_t stream);
/* The MLP block of a decoder layer from one call:
 * h = unary(x gate^T) * (x up^T)  (f16 [m, gate.N], caller-provided),  y = epilogue(h down^T).
 * f16 activations, 1..16 rows, any weight format.  The library runs the form that measures
 * faster: today three launches (gate and up grouped on the shared activations, the gated
 * multiply, down; gate and up are rounded to f16 in between, as the model's own ops would),
 * with 2 MiB of the stream's workspace between them, so a stream's first call must not be
 * captured.  TLHIP_MLP_ONE_LAUNCH=1 in the environment selects the sequence launch (a gated
 * step and the down projection waiting for it: int4 g32 only, the product rounded once). */
int tlhip_mlp_decode(const tlhip_qweight_t* gate, const tlhip_qweight_t* up, const tlhip_qweight_t* down, int unary,
                     const void* x, int x_dtype, int64_t m, void* h, void* y, int y_dtype,
                     const tlhip_epilogue_t* down_epilogue, tlhip_stream_t stream);
/* Waits for `stream` and reports whether a sequence launch on it gave up a wait
 * (*error != 0, return TLHIP_ERR_DEVICE; the state is cleared for the next launch). */
int tlhip_sequence_status(tlhip_stream_t stream, int* error);
/* Test hook: fault != 0 makes every wait of later sequence launches unsatisfiable, and
 * spin_limit (0 = the default) bounds the polls of a wait, so that the give-up path can be
 * exercised from the host with every workgroup still leaving normally. */
int tlhip_debug_sequence(int fault, uint32_t spin_limit);

/* Prefill GEMM with dequant fused into the LDS stage: same contract as
 * tlhip_gemv for any m >= 1; x must be f16.  Stands in for the explicit
 * dequant + stock matmul the reference runs when M > 1
 * (matmul-ops.ts:163-181) with the tiled kernel's epilogue
 * (src/schedule/matmul-skeleton.ts:738-966). */
int tlhip_gemm_prefill(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y,
                       int y_dtype, float alpha, const tlhip_epilogue_t* epilogue,
                       tlhip_stream_t stream);

/* The matmul seam for a packed B operand: matmulQuantizedB
 * (matmul-ops.ts:113-182).  Routes small m to the GEMV kernels and larger m to
 * the prefill GEMM.  A few more rows than 16 on a matrix that gives far fewer
 * tiles than the chip has CUs (batched decode at batch 32..128) go through the
 * skinny matrix-core GEMV, up to 64 rows per launch, while the library's cost
 * model puts that below one tiled launch; a tuned entry of the problem itself
 * overrides the model.  f32 activations: up to 16 rows run on the VALU kernel in
 * f32 arithmetic; from 17 rows on they are rounded to f16 (the operand
 * type of the matrix cores; |x| above 65504 becomes inf) by a cast launch into
 * the stream's workspace and take the prefill GEMM of the f16 problem, which is
 * the configuration tlhip_selected_config then reports.  Like a K-sliced GEMV,
 * a stream's first such call must not happen under graph capture. */
int tlhip_matmul_quantized(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m,
                           void* y, int y_dtype, float alpha, const tlhip_epilogue_t* epilogue,
                           tlhip_stream_t stream);

/* The ops the frontend issues either side of the matmul when nothing is fused
 * (BackendOps.add / relu / silu / gelu / cast, src/backend/types.ts:340-679;
 * api.linear adds the bias as a separate op, src/frontend/torchlette.ts:892-894).
 * bias_add: out[r,c] = in[r,c] + bias[c] over an [m,n] tensor of `dtype`.
 * unary: out[i] = op(in[i]).  cast: f32 <-> f16.  In-place (out == in) is fine. */
int tlhip_bias_add(const void* in, int dtype, const void* bias, int bias_dtype, void* out, int64_t m,
                   int64_t n, tlhip_stream_t stream);
int tlhip_unary(int op, const void* in, int dtype, void* out, int64_t count, tlhip_stream_t stream);
int tlhip_cast(const void* in, int in_dtype, void* out, int out_dtype, int64_t count,
               tlhip_stream_t stream);

/* The two steps that produce a decode Linear's input (the GEMV's x).
 * rmsnorm: y[r,:] = x[r,:] * rsqrt(mean(x[r,:]^2) + eps) * weight, f32 arithmetic;
 *   fusedRMSNormForward (src/backend/types.ts:635-640, the kernel in
 *   src/backend/webgpu/rmsnorm-kernel.ts:31-66; CPU form
 *   src/frontend/decomposed-ops.ts:221-233).  x [m,d] of x_dtype, weight f32 [d],
 *   y [m,d] of y_dtype.
 * gated_mul: out[i] = unary(gate[i]) * up[i], the MLP's `mul(act(gate), up)`
 *   (packages/qwen3-browser/src/model.ts:357-361, gemma2-browser model.ts:411-415);
 *   gate, up and out share `dtype`; f32 arithmetic, one rounding to `dtype`. */
int tlhip_rmsnorm(const void* x, int x_dtype, const float* weight, void* y, int y_dtype, int64_t m,
                  int64_t d, float eps, tlhip_stream_t stream);
int tlhip_gated_mul(int unary, const void* gate, const void* up, int dtype, void* out, int64_t count,
                    tlhip_stream_t stream);

/* The same two steps fused into the decode GEMV that consumes them: the kernel
 * stages f(x) instead of x in LDS, so the normalised / gated activations never
 * travel through HBM and one launch per Linear disappears.
 *   RMSNORM  : f(x)[m,k] = x[m,k] * rsqrt(mean_k x[m,:]^2 + eps) * operand[k]
 *              (operand: f32 [K], the norm weight)
 *   GATED_MUL: f(x)[m,k] = unary(x[m,k]) * operand[m,k]
 *              (x is the gate, operand the up projection, [m,K] of x_dtype)
 * With f16 activations f(x) is rounded to f16 once, as the unfused kernel's f16
 * output would be.  Built into the VALU kernel only: m <= 4; for more rows the
 * call returns TLHIP_ERR_UNSUPPORTED and the caller runs the two steps apart.
 * tlhip_gemv_grouped_prologue: the same prologue for every problem of the group
 * (q/k/v and gate/up share their input). */
typedef enum { TLHIP_PRO_NONE = 0, TLHIP_PRO_RMSNORM = 1, TLHIP_PRO_GATED_MUL = 2 } tlhip_prologue_kind_t;
typedef struct {
  int32_t kind;        /* tlhip_prologue_kind_t */
  int32_t unary;       /* tlhip_unary_t, GATED_MUL */
  float eps;           /* RMSNORM */
  int32_t reserved;
  const void* operand; /* device; see above */
} tlhip_prologue_t;
int tlhip_gemv_prologue(const tlhip_qweight_t* w, const tlhip_prologue_t* prologue, const void* x, int x_dtype,
                        int64_t m, void* y, int y_dtype, float alpha, const tlhip_epilogue_t* epilogue,
                        tlhip_stream_t stream);
int tlhip_gemv_grouped_prologue(const tlhip_gemv_problem_t* problems, int count,
                                const tlhip_prologue_t* prologue, int x_dtype, int y_dtype, float alpha,
                                tlhip_stream_t stream);

/* Top-k of logits[offset .. offset+length) (f32, device): the k largest values in
 * descending order, ties towards the smaller index, NaN below every number;
 * out_values f32[k], out_indices [k] relative to `offset`, as TLHIP_I32 or (the
 * packed form deviceTopK returns) TLHIP_F32; device pointers.  Fewer than k
 * elements: the rest is (-3.4028234e38, -1).  The sampling
 * prefilter readTopK / deviceTopK (src/backend/types.ts:632-634, 669-678;
 * src/backend/webgpu/topk-kernel.ts): the consumer of the LM-head GEMV. */
int tlhip_topk(const float* logits, int64_t offset, int64_t length, int k, float* out_values,
               void* out_indices, int index_dtype, tlhip_stream_t stream);

/* ---- kernel choice: variant registry + autotuner
 * (src/backend/webgpu/matmul/variants.ts:54-260; autotune.ts:48-547;
 * dispatch.ts:60-207, 405-578) ---- */

/* A launch configuration.  variant 0 = "gemv" (VALU dot), 1 = "gemv_mfma"
 * (skinny MFMA: up to 16 rows, and 17..64 rows for one problem with at most 8
 * waves per workgroup and, above 32 rows, at most 2 iterations in flight),
 * 2 = "tiled" (prefill MFMA GEMM, both operands through LDS),
 * 3 = "tiled_direct" (prefill MFMA GEMM whose weights stay packed up to the
 * operand registers; fields as "tiled" with tile K 128; int4-grouped on the tiles
 * (M, N, waves M, waves N) 256x256 2x4, 256x128 2x4, 128x256 2x4, 256x128 4x2,
 * 128x128 2x2, 256x256 2x2, 128x256 1x4, 128x192 2x2; int8-row, and int8-grouped
 * with a group size that is a multiple of 64, on 256x256 2x4, 256x128 2x4, 128x256
 * 2x4, 128x128 2x2; p5 = 2, 4, 8 or 16: that many workgroups share a tile, each walking a
 * slice of K, and a second launch adds their partial sums in slice order - for
 * launches of far fewer tiles than the chip has CUs),
 * 4 = "gemv_mfma_xreg" (skinny MFMA for int4 g32 with the activations held in
 * registers: p0 waves per workgroup, p1 iterations in flight, p2 workgroups per
 * CU, p3 K slices across workgroups, p4 = 1: every weight load of a wave issued
 * before the first is consumed (at most 4 row blocks per workgroup), p5 = 1: a
 * workgroup barrier between the activation loads and the weight loads).  Unused
 * fields are 0. */
typedef struct {
  int32_t variant;
  int32_t p0; /* gemv: lanes per row (16/32/64)   gemv_mfma: waves per workgroup   tiled: tile M */
  int32_t p1; /* gemv: rows per lane-group        gemv_mfma: iterations in flight  tiled: tile N */
  int32_t p2; /* gemv: waves per workgroup        gemv_mfma: K-split waves (0 = all)  tiled: tile K */
  int32_t p3; /* gemv: K-split waves (LDS combine) gemv_mfma: K slices across workgroups (0/1 = none)  tiled: waves M */
  int32_t p4; /* gemv: chunks in flight (2/4/8)    tiled: waves N */
  int32_t p5; /* gemv: 1 = dot products on the 4x4x4 matrix-core instruction (int4, f16 x, m <= 4, p0 = 16, p1 = 1)
               * gemv_mfma: 1 = whole-line weight loads through a wave-private LDS patch (int8 with
               * K % 128 == 0 or int4-g32 with K % 256 == 0; p1 = 2 or 4)
               * tiled, tiled_direct: K slices across workgroups (0/1 = none; 2..16: that many
               * workgroups share a tile and a second launch adds their partial sums) */
  int32_t p6;
} tlhip_kernel_config_t;

/* As tlhip_matmul_quantized but with an explicit configuration
 * (dispatchMatmul's explicit `config`, dispatch.ts:171-176).  Fails if the
 * configuration is not applicable to the shape. */
int tlhip_matmul_quantized_config(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m,
                                  void* y, int y_dtype, float alpha,
                                  const tlhip_epilogue_t* epilogue,
                                  const tlhip_kernel_config_t* config, tlhip_stream_t stream);

/* Number of candidate configurations for a problem, and the i-th one
 * (variant.candidates, variants.ts:54-90). */
int tlhip_candidate_count(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype,
                          int* host_out_count);
int tlhip_candidate_get(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype, int index,
                        tlhip_kernel_config_t* host_out);
/* The configuration tlhip_matmul_quantized would use now: the tuned winner of this
 * exact problem if cached, else the winner of the nearest tuned problem of the same
 * shape class (autotune.ts:269-300), else the heuristic default — selectMatmulChoice,
 * dispatch.ts:171-192.  Every level is re-gated on applicability.  Where the rows
 * go in several launches (see tlhip_matmul_quantized) it is the configuration of
 * the first launch. */
/* The whole route: `chunk_rows` rows per launch with configuration `first` (0: all rows in
 * one launch, or the kernel's own passes) and `last` for the rows that remain.  Which route
 * is taken between decode and prefill sizes depends on a cost model whose fitted numbers
 * travel with the tuning cache (the "model" object of tlhip_tune_cache_export / import;
 * tlhip_tune_cache_clear returns to the built-in values).  Needs no device. */
int tlhip_selected_route(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype, int64_t* chunk_rows,
                         tlhip_kernel_config_t* first, tlhip_kernel_config_t* last);
int tlhip_selected_config(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype,
                          tlhip_kernel_config_t* host_out);

/* setAutotuneEnabled / isAutotuneEnabled (dispatch.ts:128-141).  Also switched
 * on by the environment variable TORCHLETTE_AUTOTUNE=1 (dispatch.ts:559). */
int tlhip_set_autotune_enabled(int enabled);
int tlhip_is_autotune_enabled(void);
/* Benchmark every candidate for this problem (2 warm-up launches + 3 timed batches
 * each, median, after dispatch.ts:324-397) and cache the winner under the key
 * (m, n, k, format, group, x dtype, y dtype) and under its shape class.  Runs on the
 * library stream with the defaults of tlhip_autotune_pool. */
int tlhip_autotune(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y,
                   int y_dtype, double* host_out_best_us);
/* The same with the knobs exposed, an epilogue and a caller's stream.
 * `weights` are `weight_count` buffers of ONE weight shape (format, n, k, group size;
 * the same or different contents), rotated launch by launch: a 9-28 MB decode weight
 * stays resident in the 256 MB last-level cache when one buffer is launched over and
 * over, and the candidates would be ranked by a rate no decode step ever sees.  With
 * weight_count == 1 the tuner makes alias copies itself, up to options->pool_bytes
 * (freed before it returns; never under graph capture, where tuning is skipped).
 * Each candidate: 2 untimed launches, then `batches` event pairs around `reps`
 * back-to-back launches, median; the `retime_top` fastest are timed once more, three
 * times as long.  quick = 1 searches only the neighbours of the current choice
 * (generateNeighborConfigs, autotune.ts:419-465).  options == NULL: the defaults
 * (reps sized to about 300 us per batch, 3 batches, top 3, 30 ms warm-up, 640 MiB). */
typedef struct {
  int32_t reps;       /* launches per event pair; 0 = automatic (20..100) */
  int32_t batches;    /* 0 = 3 */
  int32_t retime_top; /* 0 = 3; 1 = no second pass */
  int32_t quick;
  double warm_ms;     /* < 0 = 30 */
  uint64_t pool_bytes;
} tlhip_autotune_options_t;
int tlhip_autotune_pool(const tlhip_qweight_t* weights, int weight_count, const void* x, int x_dtype,
                        int64_t m, void* y, int y_dtype, const tlhip_epilogue_t* epilogue,
                        const tlhip_autotune_options_t* options, tlhip_stream_t stream,
                        double* host_out_best_us);
/* seedPerShapeMatmulChoice (dispatch.ts:99-107): record a winner for this
 * problem without benchmarking (tests, pre-seeded caches, a caller's own
 * timing loop).  Fails if the configuration is not applicable. */
int tlhip_tune_cache_seed(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype,
                          const tlhip_kernel_config_t* config);
/* Backend.pretuneMatmulShapes (src/backend/types.ts:688): [m,n,k] triples.
 * The hook carries no operand format, so it only records shape hints; tuning
 * happens at first dispatch of a matching packed operand when enabled. */
int tlhip_pretune_matmul_shapes(const int64_t* host_mnk, int count);
/* exportTuningCache / importTuningCache (autotune.ts:309-329): JSON text.
 * export writes at most cap bytes (NUL-terminated) and the needed size. */
int tlhip_tune_cache_export(char* host_buf, size_t cap, size_t* host_out_needed);
int tlhip_tune_cache_import(const char* host_json);
int tlhip_tune_cache_clear(void);

/* Dispatch counters, the reference's test hooks (dispatch.ts:79-83, 832-864,
 * 943-947): "quant_gemv_dispatches", "quant_gemm_dispatches",
 * "dequant_dispatches", "autotune_runs", and "tuning_entries_loaded" (entries
 * imported from the tuning file at tlhip_init).  Unknown names return 0. */
uint64_t tlhip_counter(const char* name);
int tlhip_counters_reset(void);

#ifdef __cplusplus
}
#endif
#endif /* TLHIP_H */
