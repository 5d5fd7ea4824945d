/*
 * tfjs_hip.h — C ABI of libtfjs_hip.so, the MI355X (gfx950) device library behind the
 * `hip` backend for tfjs-core's KernelBackend plugin API.
 *
 * Everything the JavaScript backend class (through the N-API addon), the Python ctypes
 * driver and any C/C++ caller needs goes through these entry points: plain pointers,
 * integers and sizes only.  The shape of the interface follows the reference's own
 * native precedent, the WASM backend, which keys device tensors by an integer data id
 * chosen by the host (tfjs-backend-wasm/src/lib.cc:55-134, backend_wasm.ts:35-51,166-187)
 * and passes ids of pre-registered outputs to each kernel call (lib.cc:102-124).
 *
 * Conventions
 *  - Every call returns 0 on success or a TFHIP_E* code; tfhip_last_error() then holds a
 *    message.  The JS shim turns non-zero into `throw new Error(msg)`, which is how
 *    backend_cpu reports errors (backend_cpu.ts:119-127).
 *  - All device work is queued on the context's single in-order stream and returns
 *    immediately; only tfhip_read / tfhip_sync / tfhip_time_end wait for the device.
 *  - A data id owns one device buffer whose element type was fixed at register time.
 *    Several tensors may alias one id (reshape and widening casts do,
 *    backends/backend_util.ts:34-82), so kernels convert from the *stored* dtype.
 *  - Tensors are dense row-major; images are NHWC, filters HWIO.
 */
#ifndef TFJS_HIP_H_
#define TFJS_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tfhip_ctx tfhip_ctx;

/* dtype codes 0..2 are the reference's (tfjs-backend-wasm/src/lib.cc:26-30);
 * UINT8Q holds affine-quantised weights (io/types.ts:100-107) kept as bytes in HBM. */
enum { TFHIP_FLOAT32 = 0, TFHIP_INT32 = 1, TFHIP_BOOL = 2, TFHIP_UINT8Q = 3 };

enum {
  TFHIP_OK = 0,
  TFHIP_EINVAL = 1,   /* bad argument / shape mismatch */
  TFHIP_ENOENT = 2,   /* unknown data id */
  TFHIP_EEXIST = 3,   /* data id registered twice (backend_cpu.ts:119-121) */
  TFHIP_EDEVICE = 4,  /* HIP runtime error */
  TFHIP_ENOTSUP = 5   /* legal in the reference but not built here */
};

/* Activation applied in the epilogue of the dense kernels.  LINEAR/RELU/PRELU are the
 * reference's Activation type (ops/fused_util.ts:19); RELU6 is clip(x,0,6)
 * (backend_cpu.ts:1265-1275) folded into the same epilogue. */
enum { TFHIP_ACT_LINEAR = 0, TFHIP_ACT_RELU = 1, TFHIP_ACT_PRELU = 2, TFHIP_ACT_RELU6 = 3 };

/* Mirrors Conv2DInfo (ops/conv_util.ts:43-64), channelsLast only. */
typedef struct tfhip_conv2d_info {
  int32_t batch;
  int32_t in_h, in_w, in_c;
  int32_t out_h, out_w, out_c;
  int32_t stride_h, stride_w;
  int32_t dilation_h, dilation_w;
  int32_t filter_h, filter_w;
  int32_t pad_top, pad_left, pad_bottom, pad_right;
} tfhip_conv2d_info;

/* Affine dequantisation of a TFHIP_UINT8Q operand: w = q*scale + min evaluated in double
 * and rounded once to float32, as decodeWeights does (io/io_utils.ts:133-136). */
typedef struct tfhip_qparams {
  double scale;
  double min;
} tfhip_qparams;

/* ---- context --------------------------------------------------------------------- */
/* Factory of the backend (engine.ts:261-307 calls it): picks the device, creates the
 * stream and the buffer pool. */
int tfhip_init(int device, tfhip_ctx** out);
/* KernelBackend.dispose (backend.ts:646): frees every buffer and the stream. */
void tfhip_destroy(tfhip_ctx* ctx);
/* Message of the last failed call on this context (ctx may be NULL after a failed init). */
const char* tfhip_last_error(tfhip_ctx* ctx);

/* ---- storage (KernelBackend.register/write/read/readSync/disposeData/memory,
 *      backend.ts:92-126; CPU implementation backend_cpu.ts:102-129,199-254) ---------- */
int tfhip_register(tfhip_ctx* ctx, int64_t id, const int32_t* shape, int rank, int dtype);
int tfhip_write(tfhip_ctx* ctx, int64_t id, const void* host, size_t nbytes);
int tfhip_read(tfhip_ctx* ctx, int64_t id, void* host, size_t nbytes);
int tfhip_dispose(tfhip_ctx* ctx, int64_t id);
/* How the copies are ordered.  Kernels run on one in-order stream.  tfhip_write sends up to
 * 64 KiB through a pinned slot on that stream and returns without waiting; larger writes run on
 * a second stream, so that they overlap with the kernels queued before them, and the first
 * kernel that uses the buffer waits for the copy (the device backends of the reference upload
 * lazily for the same reason: tfjs-webgpu/src/backend_webgpu.ts:191-245,
 * backends/webgl/backend_webgl.ts:425-499).  From ordinary memory the call returns when the
 * copy is done (the caller's array is its own again).  From memory of tfhip_host_alloc the call
 * returns at once and the copy reads the caller's buffer later: leave it unchanged until
 * tfhip_sync, tfhip_read or a finished asynchronous read of a result that depends on it — the
 * contract of the reference's CPU backend, whose write keeps the caller's array
 * (backend_cpu.ts:122-129).
 *
 * Pinned host memory for such uploads.  Process-wide (no context), safe from any thread.
 * tfhip_host_free waits for copies that still use the memory. */
int tfhip_host_alloc(size_t nbytes, void** ptr);
int tfhip_host_free(void* ptr);
/* KernelBackend.read (backend.ts:33-35) returns a promise: a read in three steps, so that the
 * host's thread never waits for the device.
 *   tfhip_read_begin   queues, behind the kernels queued so far, a copy of the buffer into
 *                      pinned staging memory on a third stream, and returns at once.  The
 *                      buffer may be disposed or overwritten right away.
 *   tfhip_read_wait    blocks until that copy is done.  The only call of this interface that may
 *                      run on another thread than the context's (a worker of the host's thread
 *                      pool); it touches nothing but the ticket.
 *   tfhip_read_finish  copies the staged bytes to `host` (nbytes must be the buffer's size; NULL
 *                      drops the data), waiting first if nobody has, and frees the ticket.  ctx
 *                      may be NULL when the context was destroyed in the meantime. */
typedef struct tfhip_pending_read tfhip_pending_read;
int tfhip_read_begin(tfhip_ctx* ctx, int64_t id, tfhip_pending_read** out);
int tfhip_read_wait(tfhip_pending_read* r);
int tfhip_read_finish(tfhip_ctx* ctx, tfhip_pending_read* r, void* host, size_t nbytes);
/* bytes held by live ids / bytes parked in the pool / number of live ids */
int tfhip_mem_info(tfhip_ctx* ctx, size_t* in_use, size_t* pooled, size_t* num_ids);
int tfhip_sync(tfhip_ctx* ctx);

/* No counterpart in the reference (its backends queue everything on one context).  A context has
 * two compute streams; calls that queue work use the selected one (0 after tfhip_init).  Work
 * queued under one index runs in the order of the calls; work under different indices is not
 * ordered against each other and may overlap on the device: two independent passes (batch i
 * under index 0, batch i + 1 under index 1 of a serving loop) then fill each other's idle
 * phases.  What orders them is the buffers they share: a stream that meets a buffer whose
 * contents were written under another index waits, once per buffer, for the work queued under that
 * index so far (an event, no host wait), and a block goes back to the pool behind the work of
 * every stream that used it.  Buffers that are only read (weights) cost nothing to share.
 * (The contents of a buffer count as written by the first work queued on it, or by tfhip_write:
 * tensors are written once.  A caller that has a kernel overwrite a live buffer under another
 * index than the one that wrote it first orders that itself, with tfhip_sync.)
 * tfhip_read / tfhip_read_begin follow the buffer's own stream, tfhip_sync waits for both.
 * A captured graph writes its tensors again on every replay, so replays are ordered as a whole:
 * a replay runs on the stream it was recorded on, behind everything queued under the other
 * index so far (new input data copied there by a small tfhip_write, kernels that still read the
 * previous replay's results) and behind asynchronous reads of its tensors that are still
 * copying; after it, the tensors the recorded work produced count as written anew on that
 * stream, so the next consumer under the other index waits for the replay.
 * Not inside a timed region or a graph capture. */
int tfhip_select_stream(tfhip_ctx* ctx, int index);
/* KernelBackend.time (backend.ts:92, backend_cpu.ts:239-244): device time of the work queued
 * between the two calls (two events on the stream).  Regions nest (up to 8 deep), as tf.time()
 * calls may.  BackendTimingInfo.getExtraProfileInfo (backend.ts:27-31) is fed by the per-kernel
 * figures: while a region is open every kernel is launched with a start and a stop event
 * attached to its own dispatch, so the time of a kernel is its execution on the device, as a
 * profiler's kernel trace reports it (idle time between kernels is in the region's total
 * only).  The WebGL backend of the reference times each program with timer queries
 * (backends/webgl/backend_webgl.ts:547-620).
 *   tfhip_time_kernel_count / tfhip_time_kernel  the launches of the region that ended last, in
 *                      launch order: name of the kernel variant (as tfhip_last_kernel reports
 *                      it; the entry point's name for kernels without variants) and its time.
 *                      The name stays valid until the next tfhip_time_end.
 *   tfhip_time_per_kernel(ctx, 0) switches the per-launch events off (no figures per kernel);
 *                      1, the default, switches them on. */
int tfhip_time_begin(tfhip_ctx* ctx);
int tfhip_time_end(tfhip_ctx* ctx, float* ms);
int tfhip_time_per_kernel(tfhip_ctx* ctx, int enable);
int tfhip_time_kernel_count(tfhip_ctx* ctx, int* count);
int tfhip_time_kernel(tfhip_ctx* ctx, int index, const char** name, float* ms);
/* Captured graphs: no counterpart in the reference, whose backends run every op eagerly.  A
 * chain of small kernels (a batch-1 forward pass is 32 launches of a few microseconds) is bound by
 * the host's cost per launch; captured once, it replays with a single launch.
 *   tfhip_graph_begin  starts recording the work queued on the context's stream.  Until
 *                      tfhip_graph_end, write / read / sync / time fail, and the pool must already
 *                      hold every block the work needs (run it once before capturing it).
 *   tfhip_graph_end    stops recording and returns a graph id.  The blocks the recorded work
 *                      used stay out of the pool while the graph lives: a replay writes them again.
 *   tfhip_graph_launch queues one replay (on the compute stream of the capture).  The tensors the recorded work read that were created
 *                      before the capture (weights, the input) must still exist; new input data is
 *                      written into the same tensor with tfhip_write.  Results appear in the buffers
 *                      of the tensors the recorded work produced.
 *   tfhip_graph_destroy waits for queued replays and gives the blocks back. */
int tfhip_graph_begin(tfhip_ctx* ctx);
int tfhip_graph_end(tfhip_ctx* ctx, int64_t* graph_id);
int tfhip_graph_launch(tfhip_ctx* ctx, int64_t graph_id);
int tfhip_graph_destroy(tfhip_ctx* ctx, int64_t graph_id);

/* Name of the kernel variant the last dense / image call launched (tile shape, operand
 * layout), for matching launches to profiler rows.  Not part of the reference interface. */
const char* tfhip_last_kernel(tfhip_ctx* ctx);
/* Raw device address of an id's buffer (for callers that share the device, e.g. a
 * harness that generates inputs in HBM).  Not part of the reference interface. */
int tfhip_device_ptr(tfhip_ctx* ctx, int64_t id, void** ptr, size_t* nbytes);

/* ---- dense contractions ------------------------------------------------------------ */
/* How a bias / prelu-alpha operand lines up with the [rows, N] result of a dense kernel.
 * The reference accepts any shape broadcastable to the result (ops/fused_ops.ts:114-120,
 * 340-346); the three layouts below are fused into the epilogue, any other shape is
 * handled by the host as the reference's separate add / prelu pass. */
enum {
  TFHIP_BCAST_NONE = 0,    /* operand absent (id ignored) */
  TFHIP_BCAST_SCALAR = 1,  /* 1 element */
  TFHIP_BCAST_COLUMN = 2,  /* N elements, one per output column / channel */
  TFHIP_BCAST_FULL = 3     /* same number of elements as the result */
};
/* batchMatMul / fusedBatchMatMul (backend.ts:128-138; backend_cpu.ts:491-555).
 * a: [batch,M,K] (or [batch,K,M] when transpose_a), b: [batch,K,N] (or [batch,N,K]),
 * out: [batch,M,N] float32.  q: non-NULL iff b is stored as TFHIP_UINT8Q. */
int tfhip_matmul(tfhip_ctx* ctx, int64_t a, int64_t b, int64_t out, int batch, int m, int n,
                 int k, int transpose_a, int transpose_b, int64_t bias, int bias_kind, int act,
                 int64_t prelu, int prelu_kind, const tfhip_qparams* q);
/* tfhip_matmul for callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, same kernels and same results as tfhip_matmul; it calls no
 * hipMalloc / hipFree and takes no block from the pool.  Where tfhip_matmul would take scratch
 * memory from the pool (the partial tiles of a product that is cut along K because it has too
 * few tiles to fill the GPU), this entry point uses a static device array of 8 MiB that the
 * library holds on every GPU it runs on until the process ends.  A product whose partial
 * tiles need more fails with TFHIP_ENOTSUP, as does an operand that is not stored as float32
 * (its converted copy would need a block; b may be TFHIP_UINT8Q).  All calls on one GPU share
 * the array: calls that overlap on one GPU (two contexts, two threads) race on it.  Calls on
 * one context do not: under one stream index they run in order, a call under the other index
 * (and a replay of a captured graph that recorded such a call) is put behind the array's last
 * user with an event. */
int tfhip_matmul_noalloc(tfhip_ctx* ctx, int64_t a, int64_t b, int64_t out, int batch, int m,
                         int n, int k, int transpose_a, int transpose_b, int64_t bias,
                         int bias_kind, int act, int64_t prelu, int prelu_kind,
                         const tfhip_qparams* q);
/* conv2d / fusedConv2d (backend.ts:414-421; backend_cpu.ts:1536-1616): x NHWC,
 * filter [fh,fw,in_c,out_c], out NHWC float32.  bias/prelu/q as for tfhip_matmul with
 * N = out_c and rows = batch*out_h*out_w. */
int tfhip_conv2d(tfhip_ctx* ctx, int64_t x, int64_t filter, int64_t out,
                 const tfhip_conv2d_info* info, int64_t bias, int bias_kind, int act,
                 int64_t prelu, int prelu_kind, const tfhip_qparams* q);

/* A depthwise convolution followed by a pointwise (1x1) one, the block of depthwise-separable
 * networks (separableConv2d, ops/conv.ts:588-660, composes depthwiseConv2d and conv2d;
 * backend_cpu.ts:1979-2035, 1552-1616), with the add + clip/relu that follows each folded in:
 *   out = act_pw(conv1x1(act_dw(depthwise(x, dw_filter) + dw_bias), pw_filter) + pw_bias).
 * dw_info is the Conv2DInfo of the depthwise half; pw_filter is [1,1,dw_info.out_c,out_c] and
 * out [batch,out_h,out_w,out_c].  Biases NONE / SCALAR / COLUMN, activations LINEAR / RELU /
 * RELU6; either filter may be TFHIP_UINT8Q with its qparams.  For 3x3 filters, multiplier 1 and
 * (channels, stride) in {(32->64, 1), (64->128, 2), (128->128, 1)} on large images one kernel computes both
 * halves and the intermediate never reaches HBM; so does another for small problems (float32, 3x3,
 * 32 <= channels <= 1024, at most two tiles of 16 pixels x 64 output columns per CU: the layers of a
 * network for one or a few images); every other shape runs the two kernels with
 * the intermediate in a pool block.  Results are those of the two calls (the single kernels may sum
 * the pointwise products in another order: equal within float32 round-off).
 * tfhip_separable_single_kernel(ctx, 0) forces the two-kernel form (1 restores the default). */
int tfhip_separable_conv2d(tfhip_ctx* ctx, int64_t x, int64_t dw_filter, int64_t pw_filter,
                           int64_t out, const tfhip_conv2d_info* dw_info, int64_t dw_bias,
                           int dw_bias_kind, int dw_act, int64_t pw_bias, int pw_bias_kind,
                           int pw_act, const tfhip_qparams* dw_q, const tfhip_qparams* pw_q);
int tfhip_separable_single_kernel(tfhip_ctx* ctx, int enable);

/* ---- memory-bound image kernels ------------------------------------------------------ */
/* depthwiseConv2D (backend.ts:431-434; backend_cpu.ts:1979-2035): filter
 * [fh,fw,in_c,ch_mul], out_c = in_c*ch_mul.  bias (NONE / SCALAR / COLUMN over out_c) and
 * act (LINEAR/RELU/RELU6) fold the add + clip that follow it in MobileNet into the same
 * pass; the reference issues them as separate add/clip calls.  q: filter may be UINT8Q. */
int tfhip_depthwise_conv2d(tfhip_ctx* ctx, int64_t x, int64_t filter, int64_t out,
                           const tfhip_conv2d_info* info, int64_t bias, int bias_kind, int act,
                           const tfhip_qparams* q);
/* avgPool / maxPool (backend.ts:453-462; backend_cpu.ts:2273-2345, 2869-2873). */
enum { TFHIP_POOL_AVG = 0, TFHIP_POOL_MAX = 1 };
int tfhip_pool2d(tfhip_ctx* ctx, int64_t x, int64_t out, const tfhip_conv2d_info* info,
                 int kind);

/* ---- elementwise ------------------------------------------------------------------- */
/* add/subtract/multiply/realDivide/prelu/maximum/minimum (backend.ts:164-177, 247, 258, 328;
 * backend_cpu.ts:440-481,557-580,1203-1209,3515-3549) with N-d broadcasting
 * (ops/broadcast_util.ts:27-87).  Shapes are right-aligned, rank <= 6. */
enum {
  TFHIP_ADD = 0, TFHIP_SUB = 1, TFHIP_MUL = 2, TFHIP_DIV = 3, TFHIP_PRELU = 4,
  TFHIP_MAXIMUM = 5, TFHIP_MINIMUM = 6,
  /* equal/notEqual/less/lessEqual/greater/greaterEqual/logicalAnd/logicalOr
   * (backend.ts:202-233; backend_cpu.ts:747-820): out must be TFHIP_BOOL; NaN compares
   * like JavaScript (only != is true). */
  TFHIP_EQUAL = 7, TFHIP_NOT_EQUAL = 8, TFHIP_LESS = 9, TFHIP_LESS_EQUAL = 10,
  TFHIP_GREATER = 11, TFHIP_GREATER_EQUAL = 12, TFHIP_LOGICAL_AND = 13, TFHIP_LOGICAL_OR = 14,
  /* pow/squaredDifference/mod/floorDiv/atan2/eluDer (backend.ts:166-181, 260-262, 363-366;
   * backend_cpu.ts:483-489, 582-588, 893-904, 984-991, 1227-1242, 1425-1431) with JavaScript's
   * Math.pow (1 ** +-Infinity and x ** NaN are NaN) and % (sign of the dividend).  floorDiv
   * writes int32.  eluDer(dy, y) = y >= 1 ? dy : dy * (y + 1). */
  TFHIP_POW = 15, TFHIP_SQUARED_DIFFERENCE = 16, TFHIP_MOD = 17, TFHIP_FLOOR_DIV = 18,
  TFHIP_ATAN2 = 19, TFHIP_ELU_DER = 20
};
int tfhip_binary(tfhip_ctx* ctx, int op, int64_t a, const int32_t* a_shape, int a_rank,
                 int64_t b, const int32_t* b_shape, int b_rank, int64_t out);
/* relu/clip/exp/log/neg/abs/sigmoid/sqrt/square/tanh/rsqrt
 * (backend.ts:160, 300-357, 392; backend_cpu.ts:1094-1126,1191-1201,1265-1275).  p0,p1: clip min,max. */
enum {
  TFHIP_RELU = 0, TFHIP_CLIP = 1, TFHIP_EXP = 2, TFHIP_LOG = 3, TFHIP_NEG = 4,
  TFHIP_ABS = 5, TFHIP_SIGMOID = 6, TFHIP_SQRT = 7, TFHIP_SQUARE = 8, TFHIP_TANH = 9,
  TFHIP_RSQRT = 10,
  /* floor/ceil/round/sign/expm1/log1p/reciprocal, the trigonometric and hyperbolic functions
   * and their inverses, erf/elu/selu/softplus/step (backend.ts:264-298, 306-322, 330-338,
   * 344-390; backend_cpu.ts:993-1030, 1071-1189, 1211-1225, 1244-1263, 1321-1535): round is
   * round-half-to-even, sign(NaN) = 0, erf is the reference's polynomial (also for x < 0),
   * step(x) = NaN for NaN, 1 for x > 0, else p0. */
  TFHIP_FLOOR = 11, TFHIP_CEIL = 12, TFHIP_ROUND = 13, TFHIP_SIGN = 14, TFHIP_EXPM1 = 15,
  TFHIP_LOG1P = 16, TFHIP_RECIPROCAL = 17, TFHIP_SIN = 18, TFHIP_COS = 19, TFHIP_TAN = 20,
  TFHIP_ASIN = 21, TFHIP_ACOS = 22, TFHIP_ATAN = 23, TFHIP_SINH = 24, TFHIP_COSH = 25,
  TFHIP_ASINH = 26, TFHIP_ACOSH = 27, TFHIP_ATANH = 28, TFHIP_ERF = 29, TFHIP_ELU = 30,
  TFHIP_SELU = 31, TFHIP_SOFTPLUS = 32, TFHIP_STEP = 33,
  /* isNaN/isInf/isFinite (backend.ts:284-290; backend_cpu.ts:1032-1069): out must be TFHIP_BOOL */
  TFHIP_IS_NAN = 34, TFHIP_IS_INF = 35, TFHIP_IS_FINITE = 36
};
int tfhip_unary(tfhip_ctx* ctx, int op, int64_t x, int64_t out, float p0, float p1);
/* cast / int (backend.ts:340, 484; backend_cpu.ts:1299-1308, 2861-2863; backends/backend_util.ts:34-71):
 * converts from x's stored dtype to out's stored dtype (float->int32 truncates,
 * ->bool is x != 0). */
int tfhip_cast(tfhip_ctx* ctx, int64_t x, int64_t out);
/* decodeWeights, quantised branch (io/io_utils.ts:122-147): x TFHIP_UINT8Q -> out float32,
 * w = q*scale + min in double, rounded once.  The dense kernels do this while staging
 * their B tile; this entry materialises the float weights for any other consumer.
 * When x holds two bytes per element of out, they are the 16-bit codes of a 'uint16'
 * quantisation, low byte first as in the weights file: the bytes of such a shard go to the
 * device as they are and are expanded here, once, at load time. */
int tfhip_dequantize(tfhip_ctx* ctx, int64_t x, int64_t out, const tfhip_qparams* q);
/* fill/zerosLike/onesLike (backend.ts:629-640; backend_cpu.ts:3816-3836). */
int tfhip_fill(tfhip_ctx* ctx, int64_t out, double value);

/* ---- reductions over the innermost axis ---------------------------------------------- */
/* sum/max/min/argMax/argMin (backend.ts:183, 195-200, 244, 255; backend_cpu.ts:590-611,686-712,906-929):
 * x viewed as [outer, inner]; out has `outer` elements (int32 for ARG*). */
enum {
  TFHIP_SUM = 0, TFHIP_MAX = 1, TFHIP_MIN = 2, TFHIP_ARGMAX = 3, TFHIP_ARGMIN = 4,
  /* prod/all/any (backend.ts:185-193, 249-253; backend_cpu.ts:613-633, 938-982): prod like sum;
   * all/any read and write bool */
  TFHIP_PROD = 5, TFHIP_ALL = 6, TFHIP_ANY = 7
};
int tfhip_reduce(tfhip_ctx* ctx, int op, int64_t x, int64_t out, int64_t outer, int64_t inner);
/* One-pass row softmax; same result as the reference's 10-call composite
 * (ops/softmax.ts:45-79, ops/reduction_ops.ts:56-74) within float32 tolerance. */
int tfhip_softmax_rows(tfhip_ctx* ctx, int64_t x, int64_t out, int64_t rows, int64_t cols);

/* ---- data movement ------------------------------------------------------------------- */
/* gather (backend.ts:501; backend_cpu.ts:2204-2223): x viewed as
 * [outer, axis_dim, inner]; out [outer, n_indices, inner]; indices int32. */
int tfhip_gather(tfhip_ctx* ctx, int64_t x, int64_t indices, int64_t out, int64_t outer,
                 int64_t axis_dim, int64_t inner, int64_t n_indices);
/* transpose (backend.ts:497; backend_cpu.ts:2178-2200), rank <= 6. */
int tfhip_transpose(tfhip_ctx* ctx, int64_t x, const int32_t* x_shape, int rank,
                    const int32_t* perm, int64_t out);
/* Device-to-device copy between ids of equal byte size (identity / clone). */
int tfhip_copy(tfhip_ctx* ctx, int64_t x, int64_t out);
/* Copy of a rank-d box between two strided views (rank <= 8, element strides, may be zero or
 * negative on the source side):
 *   out[out_offset + sum_d i_d*out_strides[d]] = x[x_offset + sum_d i_d*x_strides[d]],
 *   0 <= i_d < region[d].
 * One entry point for slice / stridedSlice / reverse (backend.ts:140-158; backend_cpu.ts:292-391),
 * concat (backend.ts:160; backend_cpu.ts:393-433), pad (backend.ts:486; backend_cpu.ts:2157-2176, after
 * tfhip_fill with the constant) and tile (backend.ts:484; backend_cpu.ts:2152-2155): the host
 * states the box.  x and out must have the same element size; every touched index is checked
 * against the buffers on the host. */
int tfhip_strided_copy(tfhip_ctx* ctx, int64_t x, int64_t out, int rank, const int32_t* region,
                       const int64_t* x_strides, int64_t x_offset, const int64_t* out_strides,
                       int64_t out_offset);

/* cumsum along the innermost axis (backend.ts:240-242; backend_cpu.ts:714-745): x viewed as
 * [outer, inner]; out float32 or int32 (upcastType(x.dtype, 'int32')). */
int tfhip_cumsum(tfhip_ctx* ctx, int64_t x, int64_t out, int64_t outer, int64_t inner,
                 int exclusive, int reverse);
/* topk along the innermost axis (backend.ts:236-238; backends/topk_impl.ts:25-60): x viewed as
 * [rows, cols] (float32 or int32); values [rows, k] in x's dtype, indices [rows, k] int32, in
 * descending value order, equal values in ascending index order. */
int tfhip_topk(tfhip_ctx* ctx, int64_t x, int64_t values, int64_t indices, int64_t rows,
               int64_t cols, int k);
/* localResponseNormalization4D and LRNGrad (backend.ts:600-610; backend_cpu.ts:3211-3281) over
 * [pixels, channels] float32: the window is the channels within depth_radius of each one. */
int tfhip_lrn(tfhip_ctx* ctx, int64_t x, int64_t out, int64_t pixels, int channels,
              int depth_radius, float bias, float alpha, float beta);
int tfhip_lrn_grad(tfhip_ctx* ctx, int64_t dy, int64_t x, int64_t y, int64_t dx, int64_t pixels,
                   int channels, int depth_radius, float bias, float alpha, float beta);

/* ---- further forward kernels of converter graphs ---------------------------------------- */
/* logicalNot (backend.ts:225; backend_cpu.ts:795-804): bool -> bool. */
int tfhip_logical_not(tfhip_ctx* ctx, int64_t x, int64_t out);
/* batchNormalization (backend.ts:464-468; backend_cpu.ts:3167-3213):
 *   out[i] = offset[i % |offset|] + (x[i] - mean[i % |mean|]) * scale[i % |scale|] /
 *            sqrt(variance[i % |variance|] + epsilon);  scale / offset may be -1 (1 and 0). */
int tfhip_batchnorm(tfhip_ctx* ctx, int64_t x, int64_t mean, int64_t variance, int64_t offset,
                    int64_t scale, float epsilon, int64_t out);
/* resizeBilinear (backend.ts:589-592; backend_cpu.ts:2875-2936): x [batch, in_h, in_w, c] ->
 * out [batch, out_h, out_w, c] float32. */
int tfhip_resize_bilinear(tfhip_ctx* ctx, int64_t x, int64_t out, int batch, int in_h, int in_w,
                          int channels, int out_h, int out_w, int align_corners);
/* oneHot (backend.ts:614-616; backend_cpu.ts:3325-3339): indices int32 [n] -> out [n, depth]
 * (int32 or float32 storage); an index outside [0, depth) leaves its row at off_value. */
int tfhip_one_hot(tfhip_ctx* ctx, int64_t indices, int64_t out, int depth, float on_value,
                  float off_value);

/* resizeNearestNeighbor (backend.ts:594-598; backend_cpu.ts:3016-3067): as resizeBilinear, the
 * source pixel is floor(ratio * r), or Math.round(ratio * r) with align_corners. */
int tfhip_resize_nearest(tfhip_ctx* ctx, int64_t x, int64_t out, int batch, int in_h, int in_w,
                         int channels, int out_h, int out_w, int align_corners);
/* select (backend.ts:236-238; backend_cpu.ts:822-845): out[i] = condition[i / inner] ? a[i] :
 * b[i]; inner = 1 when the condition has the shape of a, = the size of a row of `a` when the
 * condition is rank 1 over the first axis (ops/logical_ops.ts:140-156).  a, b, out share one
 * storage dtype (the host upcasts, backend_cpu.ts:828). */
int tfhip_select(tfhip_ctx* ctx, int64_t condition, int64_t a, int64_t b, int64_t out,
                 int64_t inner);
/* gatherND (backend.ts:499; backend_cpu.ts:3771-3803): x of shape x_shape[rank]; indices
 * [num_slices, slice_rank] int32 address its first slice_rank dimensions; out
 * [num_slices, product of the remaining dimensions] in x's element size.  An index outside x
 * fails with "Invalid indices: <index> does not index into <shape>" (:3796-3799); the check
 * waits for the device, so the call is not available during a graph capture. */
int tfhip_gather_nd(tfhip_ctx* ctx, int64_t x, int64_t indices, int64_t out,
                    const int32_t* x_shape, int rank, int64_t num_slices, int slice_rank);
/* scatterND, sparseToDense and unsortedSegmentSum (backend.ts:193, 499-503, 624-627;
 * backend_cpu.ts:635-660, 3759-3769, 3805-3814, 3842-3889): out of shape out_shape[rank]
 * (float32 or int32) starts at default_value; update i (a slice of the trailing
 * rank - slice_rank dimensions, or one value shared by all) goes to the slice
 * indices[i, :] addresses, in ascending i.  flags:
 *   TFHIP_SCATTER_SUM           add to what is there (scatterND); without it the update
 *                               replaces it and the last one wins (sparseToDense)
 *   TFHIP_SCATTER_SKIP_INVALID  an index outside the result is skipped (unsortedSegmentSum
 *                               ignores such segment ids); without it the call fails as
 *                               tfhip_gather_nd does
 *   TFHIP_SCATTER_WIDE_SUM      float32 sums are kept in double and rounded once
 *                               (unsortedSegmentSum); without it every addition rounds to
 *                               float32 as the reference's typed array does */
enum { TFHIP_SCATTER_SUM = 1, TFHIP_SCATTER_SKIP_INVALID = 2, TFHIP_SCATTER_WIDE_SUM = 4 };
int tfhip_scatter_nd(tfhip_ctx* ctx, int64_t indices, int64_t updates, int64_t out,
                     const int32_t* out_shape, int rank, int64_t num_updates, int slice_rank,
                     double default_value, int flags);
/* fft / ifft (backend.ts:618-622; backend_cpu.ts:3343-3467): x and out are float32 buffers
 * holding batch rows of n interleaved (real, imaginary) pairs, which is how the host keeps a
 * complex64 tensor; inverse = 1 changes the sign of the exponent and divides by n. */
int tfhip_fft(tfhip_ctx* ctx, int64_t x, int64_t out, int64_t batch, int64_t n, int inverse);
/* cropAndResize (backend.ts:612-616; backend_cpu.ts:3622-3757): images [batch,h,w,c]; boxes
 * [num_boxes,4] float32 rows (y1,x1,y2,x2) in normalised coordinates; box_index [num_boxes]
 * int32; out [num_boxes,crop_h,crop_w,c] float32.  Samples outside the image get
 * extrapolation_value; a box whose image index is outside the batch yields zeros. */
enum { TFHIP_RESIZE_BILINEAR = 0, TFHIP_RESIZE_NEAREST = 1 };
int tfhip_crop_and_resize(tfhip_ctx* ctx, int64_t images, int64_t boxes, int64_t box_index,
                          int64_t out, int batch, int image_h, int image_w, int channels,
                          int64_t num_boxes, int crop_h, int crop_w, int method,
                          float extrapolation_value);

/* ---- backward kernels (training) ---------------------------------------------------------- */
/* `info` is the Conv2DInfo of the FORWARD op in every call below (in_* = x, out_* = y).
 * conv2dDerInput (backend.ts:423-425; backend_cpu.ts:1686-1762): dy [batch,out_h,out_w,out_c],
 * filter [fh,fw,in_c,out_c] -> dx [batch,in_h,in_w,in_c] float32.  Also the forward pass of
 * conv2dTranspose (ops/conv.ts:783-790).  Dilation must be 1 (ops/conv.ts:240-243). */
int tfhip_conv2d_der_input(tfhip_ctx* ctx, int64_t dy, int64_t filter, int64_t dx,
                           const tfhip_conv2d_info* info);
/* conv2dDerFilter (backend.ts:427-429; backend_cpu.ts:1849-1898): x, dy -> dW
 * [fh,fw,in_c,out_c] float32. */
int tfhip_conv2d_der_filter(tfhip_ctx* ctx, int64_t x, int64_t dy, int64_t dw,
                            const tfhip_conv2d_info* info);
/* depthwiseConv2DDerInput / depthwiseConv2DDerFilter (backend.ts:435-441;
 * backend_cpu.ts:2037-2150): filter and dW are [fh,fw,in_c,ch_mul]. */
int tfhip_depthwise_conv2d_der_input(tfhip_ctx* ctx, int64_t dy, int64_t filter, int64_t dx,
                                     const tfhip_conv2d_info* info);
int tfhip_depthwise_conv2d_der_filter(tfhip_ctx* ctx, int64_t x, int64_t dy, int64_t dw,
                                      const tfhip_conv2d_info* info);
/* maxPoolBackprop / avgPoolBackprop (backend.ts:456-465; backend_cpu.ts:2347-2509): dy, the
 * forward input x (values used by TFHIP_POOL_MAX only; first strict maximum of a window wins,
 * NaN never does) -> dx float32.  avg multiplies by 1 / (fh * fw) whatever part of a window
 * lay inside the image, as the reference does.  Dilation is allowed (tf.pool). */
int tfhip_pool2d_backprop(tfhip_ctx* ctx, int64_t dy, int64_t x, int64_t dx,
                          const tfhip_conv2d_info* info, int kind);
/* resizeBilinearBackprop / resizeNearestNeighborBackprop (backend.ts:591-598;
 * backend_cpu.ts:2938-3013, 3070-3165): dy [batch,y_h,y_w,c] float32 -> dx [batch,x_h,x_w,c]
 * float32, the gradient of the resize of an x_h x x_w image to y_h x y_w.  Contributions to
 * one dx element are added in the reference's order, so the results do not depend on
 * scheduling.  (The reference labels the bilinear result [batch,x_w,x_h,c]; the data is in
 * [batch,x_h,x_w,c] order in both.) */
int tfhip_resize_bilinear_backprop(tfhip_ctx* ctx, int64_t dy, int64_t dx, int batch, int x_h,
                                   int x_w, int channels, int y_h, int y_w, int align_corners);
int tfhip_resize_nearest_backprop(tfhip_ctx* ctx, int64_t dy, int64_t dx, int batch, int x_h,
                                  int x_w, int channels, int y_h, int y_w, int align_corners);

#ifdef __cplusplus
}
#endif
#endif /* TFJS_HIP_H_ */
