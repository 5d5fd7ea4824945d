/*
 * tfjs_hip.node — raw N-API binding of the C ABI in include/tfjs_hip.h.
 *
 * Deliberately thin: every exported function converts its JavaScript arguments to plain
 * C values, calls the entry point of the same name in libtfjs_hip.so and turns a non-zero
 * status into a thrown Error carrying tfhip_last_error().  Tensors never cross this
 * boundary except in write() (TypedArray -> device) and read() (device -> TypedArray);
 * kernels are addressed by integer data ids.  Plays the role of the Emscripten glue of
 * the reference's WASM backend (tfjs-backend-wasm/src/backend_wasm.ts:166-187).
 */
#include <node_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tfjs_hip.h"

#define MAX_ARGS 18

#define NAPI_OK(env, call)                                              \
  do {                                                                  \
    if ((call) != napi_ok) {                                            \
      napi_throw_error((env), NULL, "tfjs_hip.node: N-API call failed: " #call); \
      return NULL;                                                      \
    }                                                                   \
  } while (0)

static napi_value throw_status(napi_env env, tfhip_ctx* ctx, int rc) {
  const char* msg = tfhip_last_error(ctx);
  char buf[640];
  snprintf(buf, sizeof buf, "%s", (msg && msg[0]) ? msg : "hip backend call failed");
  (void)rc;
  napi_throw_error(env, NULL, buf);
  return NULL;
}

static napi_value undefined(napi_env env) {
  napi_value u;
  napi_get_undefined(env, &u);
  return u;
}

/* ---- argument helpers -------------------------------------------------------------- */
static int get_args(napi_env env, napi_callback_info info, size_t want, napi_value* argv) {
  size_t argc = MAX_ARGS;
  if (napi_get_cb_info(env, info, &argc, argv, NULL, NULL) != napi_ok || argc < want) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: wrong number of arguments");
    return 0;
  }
  return 1;
}

static int arg_ctx(napi_env env, napi_value v, tfhip_ctx** out) {
  void* p = NULL;
  if (napi_get_value_external(env, v, &p) != napi_ok || !p) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: first argument must be a context");
    return 0;
  }
  *out = (tfhip_ctx*)p;
  return 1;
}

static int arg_i64(napi_env env, napi_value v, int64_t* out) {
  double d;
  if (napi_get_value_double(env, v, &d) != napi_ok) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: expected a number");
    return 0;
  }
  *out = (int64_t)d;
  return 1;
}

static int arg_int(napi_env env, napi_value v, int* out) {
  int64_t t;
  if (!arg_i64(env, v, &t)) return 0;
  *out = (int)t;
  return 1;
}

static int arg_f64(napi_env env, napi_value v, double* out) {
  if (napi_get_value_double(env, v, out) != napi_ok) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: expected a number");
    return 0;
  }
  return 1;
}

/* Int32Array -> pointer + length */
static int arg_i32_array(napi_env env, napi_value v, const int32_t** data, size_t* len) {
  napi_typedarray_type type;
  void* p;
  if (napi_get_typedarray_info(env, v, &type, len, &p, NULL, NULL) != napi_ok ||
      type != napi_int32_array) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: expected an Int32Array");
    return 0;
  }
  *data = (const int32_t*)p;
  return 1;
}

/* any TypedArray -> pointer + byte length */
static int arg_bytes(napi_env env, napi_value v, void** data, size_t* nbytes) {
  napi_typedarray_type type;
  size_t len;
  if (napi_get_typedarray_info(env, v, &type, &len, data, NULL, NULL) != napi_ok) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: expected a TypedArray");
    return 0;
  }
  size_t w = 1;
  switch (type) {
    case napi_int8_array: case napi_uint8_array: case napi_uint8_clamped_array: w = 1; break;
    case napi_int16_array: case napi_uint16_array: w = 2; break;
    case napi_int32_array: case napi_uint32_array: case napi_float32_array: w = 4; break;
    default: w = 8; break;
  }
  *nbytes = len * w;
  return 1;
}

/* [scale, min] Float64Array(2) or null/undefined */
static int arg_qparams(napi_env env, napi_value v, tfhip_qparams* q, const tfhip_qparams** out) {
  napi_valuetype t;
  napi_typeof(env, v, &t);
  if (t == napi_undefined || t == napi_null) {
    *out = NULL;
    return 1;
  }
  napi_typedarray_type type;
  size_t len;
  void* p;
  if (napi_get_typedarray_info(env, v, &type, &len, &p, NULL, NULL) != napi_ok ||
      type != napi_float64_array || len != 2) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: qparams must be a Float64Array(2)");
    return 0;
  }
  q->scale = ((double*)p)[0];
  q->min = ((double*)p)[1];
  *out = q;
  return 1;
}

static int arg_conv_info(napi_env env, napi_value v, tfhip_conv2d_info* ci) {
  const int32_t* p;
  size_t len;
  if (!arg_i32_array(env, v, &p, &len)) return 0;
  if (len * sizeof(int32_t) != sizeof(tfhip_conv2d_info)) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: conv info must be an Int32Array(17)");
    return 0;
  }
  memcpy(ci, p, sizeof *ci);
  return 1;
}

#define ARGS(n)                                  \
  napi_value argv[MAX_ARGS];                     \
  tfhip_ctx* ctx;                                \
  if (!get_args(env, info, (n), argv)) return NULL; \
  if (!arg_ctx(env, argv[0], &ctx)) return NULL
#define I64(i, name) int64_t name; if (!arg_i64(env, argv[i], &name)) return NULL
#define INT(i, name) int name; if (!arg_int(env, argv[i], &name)) return NULL
#define F64(i, name) double name; if (!arg_f64(env, argv[i], &name)) return NULL
#define CHECK(rc) do { int rc_ = (rc); if (rc_) return throw_status(env, ctx, rc_); } while (0)

/* contexts that js_destroy has not seen yet: a read may finish after its backend is gone */
#define MAX_LIVE 64
static tfhip_ctx* live_ctx[MAX_LIVE];
static void ctx_born(tfhip_ctx* c) {
  for (int i = 0; i < MAX_LIVE; i++) if (!live_ctx[i]) { live_ctx[i] = c; return; }
}
static void ctx_died(tfhip_ctx* c) {
  for (int i = 0; i < MAX_LIVE; i++) if (live_ctx[i] == c) live_ctx[i] = NULL;
}
static int ctx_alive(tfhip_ctx* c) {
  for (int i = 0; i < MAX_LIVE; i++) if (live_ctx[i] == c) return 1;
  return 0;
}

/* ---- context / storage ------------------------------------------------------------- */
/* Contexts are destroyed explicitly by backend.dispose() (KernelBackend.dispose,
 * backend.ts:646); the external carries no finalizer so a context still referenced by
 * queued work is never torn down by the garbage collector. */
static napi_value js_init(napi_env env, napi_callback_info info) {
  napi_value argv[MAX_ARGS];
  if (!get_args(env, info, 1, argv)) return NULL;
  int device;
  if (!arg_int(env, argv[0], &device)) return NULL;
  tfhip_ctx* ctx = NULL;
  int rc = tfhip_init(device, &ctx);
  if (rc) return throw_status(env, NULL, rc);
  ctx_born(ctx);
  napi_value ext;
  NAPI_OK(env, napi_create_external(env, ctx, NULL, NULL, &ext));
  return ext;
}

static napi_value js_destroy(napi_env env, napi_callback_info info) {
  ARGS(1);
  ctx_died(ctx);
  tfhip_destroy(ctx);
  return undefined(env);
}

static napi_value js_register(napi_env env, napi_callback_info info) {
  ARGS(4);
  I64(1, id);
  const int32_t* shape; size_t rank;
  if (!arg_i32_array(env, argv[2], &shape, &rank)) return NULL;
  INT(3, dtype);
  CHECK(tfhip_register(ctx, id, shape, (int)rank, dtype));
  return undefined(env);
}

static napi_value js_write(napi_env env, napi_callback_info info) {
  ARGS(3);
  I64(1, id);
  void* data; size_t nbytes;
  if (!arg_bytes(env, argv[2], &data, &nbytes)) return NULL;
  CHECK(tfhip_write(ctx, id, data, nbytes));
  return undefined(env);
}

static napi_value js_read(napi_env env, napi_callback_info info) {
  ARGS(3);
  I64(1, id);
  void* data; size_t nbytes;
  if (!arg_bytes(env, argv[2], &data, &nbytes)) return NULL;
  CHECK(tfhip_read(ctx, id, data, nbytes));
  return argv[2];
}

static napi_value js_dispose(napi_env env, napi_callback_info info) {
  ARGS(2);
  I64(1, id);
  CHECK(tfhip_dispose(ctx, id));
  return undefined(env);
}

static napi_value js_mem_info(napi_env env, napi_callback_info info) {
  ARGS(1);
  size_t in_use, pooled, ids;
  CHECK(tfhip_mem_info(ctx, &in_use, &pooled, &ids));
  napi_value arr, v;
  NAPI_OK(env, napi_create_array_with_length(env, 3, &arr));
  napi_create_double(env, (double)in_use, &v); napi_set_element(env, arr, 0, v);
  napi_create_double(env, (double)pooled, &v); napi_set_element(env, arr, 1, v);
  napi_create_double(env, (double)ids, &v); napi_set_element(env, arr, 2, v);
  return arr;
}

static napi_value js_sync(napi_env env, napi_callback_info info) {
  ARGS(1);
  CHECK(tfhip_sync(ctx));
  return undefined(env);
}

/* selectStream(ctx, index) */
static napi_value js_select_stream(napi_env env, napi_callback_info info) {
  ARGS(2);
  int index;
  if (!arg_int(env, argv[1], &index)) return NULL;
  CHECK(tfhip_select_stream(ctx, index));
  return undefined(env);
}

static napi_value js_time_begin(napi_env env, napi_callback_info info) {
  ARGS(1);
  CHECK(tfhip_time_begin(ctx));
  return undefined(env);
}

static napi_value js_time_end(napi_env env, napi_callback_info info) {
  ARGS(1);
  float ms = 0;
  CHECK(tfhip_time_end(ctx, &ms));
  napi_value v;
  NAPI_OK(env, napi_create_double(env, ms, &v));
  return v;
}

/* timeKernels(ctx) -> [[name, ms], ...] of the time() region that ended last */
static napi_value js_time_kernels(napi_env env, napi_callback_info info) {
  ARGS(1);
  int n = 0;
  CHECK(tfhip_time_kernel_count(ctx, &n));
  napi_value arr;
  NAPI_OK(env, napi_create_array_with_length(env, (size_t)n, &arr));
  for (int i = 0; i < n; i++) {
    const char* name = "";
    float ms = 0;
    CHECK(tfhip_time_kernel(ctx, i, &name, &ms));
    napi_value pair, vn, vm;
    NAPI_OK(env, napi_create_array_with_length(env, 2, &pair));
    NAPI_OK(env, napi_create_string_utf8(env, name, NAPI_AUTO_LENGTH, &vn));
    NAPI_OK(env, napi_create_double(env, ms, &vm));
    napi_set_element(env, pair, 0, vn);
    napi_set_element(env, pair, 1, vm);
    napi_set_element(env, arr, (uint32_t)i, pair);
  }
  return arr;
}

static napi_value js_time_per_kernel(napi_env env, napi_callback_info info) {
  ARGS(2);
  INT(1, enable);
  CHECK(tfhip_time_per_kernel(ctx, enable));
  return undefined(env);
}

/* hostAlloc(nbytes) -> ArrayBuffer over pinned host memory (freed when it is collected) */
static void free_pinned(napi_env env, void* data, void* hint) {
  (void)env; (void)hint;
  tfhip_host_free(data);
}

static napi_value js_host_alloc(napi_env env, napi_callback_info info) {
  napi_value argv[MAX_ARGS];
  if (!get_args(env, info, 1, argv)) return NULL;
  double nbytes;
  if (!arg_f64(env, argv[0], &nbytes)) return NULL;
  void* p = NULL;
  if (nbytes < 1 || tfhip_host_alloc((size_t)nbytes, &p) != TFHIP_OK) {
    napi_throw_error(env, NULL, "hip backend: could not allocate pinned host memory");
    return NULL;
  }
  napi_value buf;
  if (napi_create_external_arraybuffer(env, p, (size_t)nbytes, free_pinned, NULL, &buf) != napi_ok) {
    tfhip_host_free(p);
    napi_throw_error(env, NULL, "tfjs_hip.node: could not wrap pinned memory");
    return NULL;
  }
  return buf;
}

/* readAsync(ctx, id) -> Promise<ArrayBuffer>: the copy is queued here, a worker of the thread
 * pool waits for it, and the promise resolves on the JavaScript thread
 * (KernelBackend.read, backend.ts:33-35). */
typedef struct {
  tfhip_ctx* ctx;
  tfhip_pending_read* ticket;
  size_t nbytes;
  int wait_rc;
  napi_deferred deferred;
  napi_async_work work;
} read_job;

static void read_execute(napi_env env, void* data) {
  (void)env;
  read_job* job = (read_job*)data;
  job->wait_rc = tfhip_read_wait(job->ticket);
}

static void read_complete(napi_env env, napi_status status, void* data) {
  read_job* job = (read_job*)data;
  tfhip_ctx* ctx = ctx_alive(job->ctx) ? job->ctx : NULL;
  napi_value result = NULL, err = NULL, msg;
  void* dst = NULL;
  int rc = (status == napi_ok) ? job->wait_rc : TFHIP_EDEVICE;
  if (rc == TFHIP_OK && napi_create_arraybuffer(env, job->nbytes, &dst, &result) != napi_ok) {
    rc = TFHIP_EDEVICE;
    dst = NULL;
  }
  int frc = tfhip_read_finish(ctx, job->ticket, rc == TFHIP_OK ? dst : NULL, job->nbytes);
  if (rc == TFHIP_OK) rc = frc;
  if (rc == TFHIP_OK) {
    napi_resolve_deferred(env, job->deferred, result);
  } else {
    const char* text = ctx ? tfhip_last_error(ctx) : "";
    napi_create_string_utf8(env, (text && text[0]) ? text : "hip backend: asynchronous read failed",
                            NAPI_AUTO_LENGTH, &msg);
    napi_create_error(env, NULL, msg, &err);
    napi_reject_deferred(env, job->deferred, err);
  }
  napi_delete_async_work(env, job->work);
  free(job);
}

static napi_value js_read_async(napi_env env, napi_callback_info info) {
  ARGS(3);
  I64(1, id);
  F64(2, nbytes);
  read_job* job = (read_job*)calloc(1, sizeof *job);
  if (!job) {
    napi_throw_error(env, NULL, "tfjs_hip.node: out of memory");
    return NULL;
  }
  job->ctx = ctx;
  job->nbytes = (size_t)nbytes;
  int rc = tfhip_read_begin(ctx, id, &job->ticket);
  if (rc) {
    free(job);
    return throw_status(env, ctx, rc);
  }
  napi_value promise, name;
  if (napi_create_promise(env, &job->deferred, &promise) != napi_ok ||
      napi_create_string_utf8(env, "tfhip.read", NAPI_AUTO_LENGTH, &name) != napi_ok ||
      napi_create_async_work(env, NULL, name, read_execute, read_complete, job, &job->work) != napi_ok ||
      napi_queue_async_work(env, job->work) != napi_ok) {
    tfhip_read_finish(ctx, job->ticket, NULL, 0);
    free(job);
    napi_throw_error(env, NULL, "tfjs_hip.node: could not queue the read");
    return NULL;
  }
  return promise;
}

static napi_value js_last_kernel(napi_env env, napi_callback_info info) {
  ARGS(1);
  napi_value v;
  NAPI_OK(env, napi_create_string_utf8(env, tfhip_last_kernel(ctx), NAPI_AUTO_LENGTH, &v));
  return v;
}

/* ---- kernels ----------------------------------------------------------------------- */
/* matmul(ctx, a, b, out, batch, m, n, k, tA, tB, bias, biasKind, act, prelu, preluKind, q) */
static napi_value js_matmul(napi_env env, napi_callback_info info) {
  ARGS(16);
  I64(1, a); I64(2, b); I64(3, out);
  INT(4, batch); INT(5, m); INT(6, n); INT(7, k); INT(8, ta); INT(9, tb);
  I64(10, bias); INT(11, bias_kind); INT(12, act); I64(13, prelu); INT(14, prelu_kind);
  tfhip_qparams q; const tfhip_qparams* qp;
  if (!arg_qparams(env, argv[15], &q, &qp)) return NULL;
  CHECK(tfhip_matmul(ctx, a, b, out, batch, m, n, k, ta, tb, bias, bias_kind, act, prelu,
                     prelu_kind, qp));
  return undefined(env);
}

/* matmulNoalloc: the same arguments; allocates no device memory (tfhip_matmul_noalloc) */
static napi_value js_matmul_noalloc(napi_env env, napi_callback_info info) {
  ARGS(16);
  I64(1, a); I64(2, b); I64(3, out);
  INT(4, batch); INT(5, m); INT(6, n); INT(7, k); INT(8, ta); INT(9, tb);
  I64(10, bias); INT(11, bias_kind); INT(12, act); I64(13, prelu); INT(14, prelu_kind);
  tfhip_qparams q; const tfhip_qparams* qp;
  if (!arg_qparams(env, argv[15], &q, &qp)) return NULL;
  CHECK(tfhip_matmul_noalloc(ctx, a, b, out, batch, m, n, k, ta, tb, bias, bias_kind, act, prelu,
                             prelu_kind, qp));
  return undefined(env);
}

/* conv2d(ctx, x, filter, out, info, bias, biasKind, act, prelu, preluKind, q) */
static napi_value js_conv2d(napi_env env, napi_callback_info info) {
  ARGS(11);
  I64(1, x); I64(2, w); I64(3, out);
  tfhip_conv2d_info ci;
  if (!arg_conv_info(env, argv[4], &ci)) return NULL;
  I64(5, bias); INT(6, bias_kind); INT(7, act); I64(8, prelu); INT(9, prelu_kind);
  tfhip_qparams q; const tfhip_qparams* qp;
  if (!arg_qparams(env, argv[10], &q, &qp)) return NULL;
  CHECK(tfhip_conv2d(ctx, x, w, out, &ci, bias, bias_kind, act, prelu, prelu_kind, qp));
  return undefined(env);
}

/* depthwiseConv2d(ctx, x, filter, out, info, bias, biasKind, act, q) */
static napi_value js_depthwise(napi_env env, napi_callback_info info) {
  ARGS(9);
  I64(1, x); I64(2, w); I64(3, out);
  tfhip_conv2d_info ci;
  if (!arg_conv_info(env, argv[4], &ci)) return NULL;
  I64(5, bias); INT(6, bias_kind); INT(7, act);
  tfhip_qparams q; const tfhip_qparams* qp;
  if (!arg_qparams(env, argv[8], &q, &qp)) return NULL;
  CHECK(tfhip_depthwise_conv2d(ctx, x, w, out, &ci, bias, bias_kind, act, qp));
  return undefined(env);
}

/* separableConv2d(ctx, x, dwFilter, pwFilter, out, dwInfo, dwBias, dwBiasKind, dwAct, pwBias,
 *                 pwBiasKind, pwAct, dwQ, pwQ) */
static napi_value js_separable(napi_env env, napi_callback_info info) {
  ARGS(14);
  I64(1, x); I64(2, dw); I64(3, pw); I64(4, out);
  tfhip_conv2d_info ci;
  if (!arg_conv_info(env, argv[5], &ci)) return NULL;
  I64(6, dw_bias); INT(7, dw_bias_kind); INT(8, dw_act);
  I64(9, pw_bias); INT(10, pw_bias_kind); INT(11, pw_act);
  tfhip_qparams dq, pq; const tfhip_qparams* dqp; const tfhip_qparams* pqp;
  if (!arg_qparams(env, argv[12], &dq, &dqp) || !arg_qparams(env, argv[13], &pq, &pqp)) return NULL;
  CHECK(tfhip_separable_conv2d(ctx, x, dw, pw, out, &ci, dw_bias, dw_bias_kind, dw_act, pw_bias,
                               pw_bias_kind, pw_act, dqp, pqp));
  return undefined(env);
}

static napi_value js_separable_single_kernel(napi_env env, napi_callback_info info) {
  ARGS(2);
  INT(1, enable);
  CHECK(tfhip_separable_single_kernel(ctx, enable));
  return undefined(env);
}

/* pool2d(ctx, x, out, info, kind) */
static napi_value js_pool2d(napi_env env, napi_callback_info info) {
  ARGS(5);
  I64(1, x); I64(2, out);
  tfhip_conv2d_info ci;
  if (!arg_conv_info(env, argv[3], &ci)) return NULL;
  INT(4, kind);
  CHECK(tfhip_pool2d(ctx, x, out, &ci, kind));
  return undefined(env);
}

/* resizeNearest(ctx, x, out, batch, inH, inW, channels, outH, outW, alignCorners) */
static napi_value js_resize_nearest(napi_env env, napi_callback_info info) {
  ARGS(10);
  I64(1, x); I64(2, out);
  INT(3, batch); INT(4, in_h); INT(5, in_w); INT(6, ch); INT(7, out_h); INT(8, out_w); INT(9, align);
  CHECK(tfhip_resize_nearest(ctx, x, out, batch, in_h, in_w, ch, out_h, out_w, align));
  return undefined(env);
}

/* gatherND(ctx, x, indices, out, xShape:Int32Array, numSlices, sliceRank) */
static napi_value js_gather_nd(napi_env env, napi_callback_info info) {
  ARGS(7);
  I64(1, x); I64(2, indices); I64(3, out);
  const int32_t* shape; size_t rank;
  if (!arg_i32_array(env, argv[4], &shape, &rank)) return NULL;
  I64(5, num_slices); INT(6, slice_rank);
  CHECK(tfhip_gather_nd(ctx, x, indices, out, shape, (int)rank, num_slices, slice_rank));
  return undefined(env);
}

/* scatterND(ctx, indices, updates, out, outShape:Int32Array, numUpdates, sliceRank, defaultValue, sumDupes) */
static napi_value js_scatter_nd(napi_env env, napi_callback_info info) {
  ARGS(9);
  I64(1, indices); I64(2, updates); I64(3, out);
  const int32_t* shape; size_t rank;
  if (!arg_i32_array(env, argv[4], &shape, &rank)) return NULL;
  I64(5, num_updates); INT(6, slice_rank); F64(7, default_value); INT(8, sum_dupes);
  CHECK(tfhip_scatter_nd(ctx, indices, updates, out, shape, (int)rank, num_updates, slice_rank,
                         default_value, sum_dupes));
  return undefined(env);
}

/* cropAndResize(ctx, images, boxes, boxIndex, out, batch, h, w, channels, numBoxes, cropH, cropW, method, extrapolation) */
static napi_value js_crop_and_resize(napi_env env, napi_callback_info info) {
  ARGS(14);
  I64(1, images); I64(2, boxes); I64(3, box_index); I64(4, out);
  INT(5, batch); INT(6, h); INT(7, w); INT(8, ch); I64(9, num_boxes); INT(10, crop_h); INT(11, crop_w);
  INT(12, method); F64(13, extrapolation);
  CHECK(tfhip_crop_and_resize(ctx, images, boxes, box_index, out, batch, h, w, ch, num_boxes, crop_h,
                              crop_w, method, (float)extrapolation));
  return undefined(env);
}

/* resizeBilinearBackprop / resizeNearestBackprop(ctx, dy, dx, batch, xH, xW, channels, yH, yW, alignCorners) */
static napi_value js_resize_bilinear_backprop(napi_env env, napi_callback_info info) {
  ARGS(10);
  I64(1, dy); I64(2, dx);
  INT(3, batch); INT(4, x_h); INT(5, x_w); INT(6, ch); INT(7, y_h); INT(8, y_w); INT(9, align);
  CHECK(tfhip_resize_bilinear_backprop(ctx, dy, dx, batch, x_h, x_w, ch, y_h, y_w, align));
  return undefined(env);
}
static napi_value js_resize_nearest_backprop(napi_env env, napi_callback_info info) {
  ARGS(10);
  I64(1, dy); I64(2, dx);
  INT(3, batch); INT(4, x_h); INT(5, x_w); INT(6, ch); INT(7, y_h); INT(8, y_w); INT(9, align);
  CHECK(tfhip_resize_nearest_backprop(ctx, dy, dx, batch, x_h, x_w, ch, y_h, y_w, align));
  return undefined(env);
}

/* fft(ctx, x, out, batch, n, inverse) */
static napi_value js_fft(napi_env env, napi_callback_info info) {
  ARGS(6);
  I64(1, x); I64(2, out); I64(3, batch); I64(4, n); INT(5, inverse);
  CHECK(tfhip_fft(ctx, x, out, batch, n, inverse));
  return undefined(env);
}

/* graphBegin(ctx), graphEnd(ctx) -> id, graphLaunch(ctx, id), graphDestroy(ctx, id) */
static napi_value js_graph_begin(napi_env env, napi_callback_info info) {
  ARGS(1);
  CHECK(tfhip_graph_begin(ctx));
  return undefined(env);
}
static napi_value js_graph_end(napi_env env, napi_callback_info info) {
  ARGS(1);
  int64_t id = 0;
  CHECK(tfhip_graph_end(ctx, &id));
  napi_value out;
  if (napi_create_double(env, (double)id, &out) != napi_ok) return NULL;
  return out;
}
static napi_value js_graph_launch(napi_env env, napi_callback_info info) {
  ARGS(2);
  I64(1, id);
  CHECK(tfhip_graph_launch(ctx, id));
  return undefined(env);
}
static napi_value js_graph_destroy(napi_env env, napi_callback_info info) {
  ARGS(2);
  I64(1, id);
  CHECK(tfhip_graph_destroy(ctx, id));
  return undefined(env);
}

/* topk(ctx, x, values, indices, rows, cols, k) */
static napi_value js_topk(napi_env env, napi_callback_info info) {
  ARGS(7);
  I64(1, x); I64(2, values); I64(3, indices); I64(4, rows); I64(5, cols); INT(6, k);
  CHECK(tfhip_topk(ctx, x, values, indices, rows, cols, k));
  return undefined(env);
}

/* cumsum(ctx, x, out, outer, inner, exclusive, reverse) */
static napi_value js_cumsum(napi_env env, napi_callback_info info) {
  ARGS(7);
  I64(1, x); I64(2, out); I64(3, outer); I64(4, inner); INT(5, exclusive); INT(6, reverse);
  CHECK(tfhip_cumsum(ctx, x, out, outer, inner, exclusive, reverse));
  return undefined(env);
}

/* lrn(ctx, x, out, pixels, channels, depthRadius, bias, alpha, beta) */
static napi_value js_lrn(napi_env env, napi_callback_info info) {
  ARGS(9);
  I64(1, x); I64(2, out); I64(3, pixels); INT(4, channels); INT(5, radius);
  F64(6, bias); F64(7, alpha); F64(8, beta);
  CHECK(tfhip_lrn(ctx, x, out, pixels, channels, radius, (float)bias, (float)alpha, (float)beta));
  return undefined(env);
}

/* lrnGrad(ctx, dy, x, y, dx, pixels, channels, depthRadius, bias, alpha, beta) */
static napi_value js_lrn_grad(napi_env env, napi_callback_info info) {
  ARGS(11);
  I64(1, dy); I64(2, x); I64(3, y); I64(4, dx); I64(5, pixels); INT(6, channels); INT(7, radius);
  F64(8, bias); F64(9, alpha); F64(10, beta);
  CHECK(tfhip_lrn_grad(ctx, dy, x, y, dx, pixels, channels, radius, (float)bias, (float)alpha,
                       (float)beta));
  return undefined(env);
}

/* select(ctx, condition, a, b, out, inner) */
static napi_value js_select(napi_env env, napi_callback_info info) {
  ARGS(6);
  I64(1, c); I64(2, a); I64(3, b); I64(4, out); I64(5, inner);
  CHECK(tfhip_select(ctx, c, a, b, out, inner));
  return undefined(env);
}

/* Backward kernels: name(ctx, a, b, out, info) with info = the forward op's Conv2DInfo.
 * conv2dDerInput(ctx, dy, filter, dx, info), conv2dDerFilter(ctx, x, dy, dW, info) and their
 * depthwise twins. */
#define BACKWARD_BINDING(js_fn, c_fn)                                   \
  static napi_value js_fn(napi_env env, napi_callback_info info) {      \
    ARGS(5);                                                            \
    I64(1, a); I64(2, b); I64(3, out);                                  \
    tfhip_conv2d_info ci;                                               \
    if (!arg_conv_info(env, argv[4], &ci)) return NULL;                 \
    CHECK(c_fn(ctx, a, b, out, &ci));                                   \
    return undefined(env);                                              \
  }
BACKWARD_BINDING(js_conv2d_der_input, tfhip_conv2d_der_input)
BACKWARD_BINDING(js_conv2d_der_filter, tfhip_conv2d_der_filter)
BACKWARD_BINDING(js_depthwise_der_input, tfhip_depthwise_conv2d_der_input)
BACKWARD_BINDING(js_depthwise_der_filter, tfhip_depthwise_conv2d_der_filter)

/* pool2dBackprop(ctx, dy, x, dx, info, kind) */
static napi_value js_pool2d_backprop(napi_env env, napi_callback_info info) {
  ARGS(6);
  I64(1, dy); I64(2, x); I64(3, dx);
  tfhip_conv2d_info ci;
  if (!arg_conv_info(env, argv[4], &ci)) return NULL;
  INT(5, kind);
  CHECK(tfhip_pool2d_backprop(ctx, dy, x, dx, &ci, kind));
  return undefined(env);
}

/* binary(ctx, op, a, aShape, b, bShape, out) */
static napi_value js_binary(napi_env env, napi_callback_info info) {
  ARGS(7);
  INT(1, op); I64(2, a);
  const int32_t* as; size_t ar;
  if (!arg_i32_array(env, argv[3], &as, &ar)) return NULL;
  I64(4, b);
  const int32_t* bs; size_t br;
  if (!arg_i32_array(env, argv[5], &bs, &br)) return NULL;
  I64(6, out);
  CHECK(tfhip_binary(ctx, op, a, as, (int)ar, b, bs, (int)br, out));
  return undefined(env);
}

/* unary(ctx, op, x, out, p0, p1) */
static napi_value js_unary(napi_env env, napi_callback_info info) {
  ARGS(6);
  INT(1, op); I64(2, x); I64(3, out); F64(4, p0); F64(5, p1);
  CHECK(tfhip_unary(ctx, op, x, out, (float)p0, (float)p1));
  return undefined(env);
}

static napi_value js_cast(napi_env env, napi_callback_info info) {
  ARGS(3);
  I64(1, x); I64(2, out);
  CHECK(tfhip_cast(ctx, x, out));
  return undefined(env);
}

static napi_value js_copy(napi_env env, napi_callback_info info) {
  ARGS(3);
  I64(1, x); I64(2, out);
  CHECK(tfhip_copy(ctx, x, out));
  return undefined(env);
}

/* dequantize(ctx, x, out, q) */
static napi_value js_dequantize(napi_env env, napi_callback_info info) {
  ARGS(4);
  I64(1, x); I64(2, out);
  tfhip_qparams q; const tfhip_qparams* qp;
  if (!arg_qparams(env, argv[3], &q, &qp)) return NULL;
  CHECK(tfhip_dequantize(ctx, x, out, qp));
  return undefined(env);
}

static napi_value js_fill(napi_env env, napi_callback_info info) {
  ARGS(3);
  I64(1, out); F64(2, value);
  CHECK(tfhip_fill(ctx, out, value));
  return undefined(env);
}

/* reduce(ctx, op, x, out, outer, inner) */
static napi_value js_reduce(napi_env env, napi_callback_info info) {
  ARGS(6);
  INT(1, op); I64(2, x); I64(3, out); I64(4, outer); I64(5, inner);
  CHECK(tfhip_reduce(ctx, op, x, out, outer, inner));
  return undefined(env);
}

static napi_value js_softmax_rows(napi_env env, napi_callback_info info) {
  ARGS(5);
  I64(1, x); I64(2, out); I64(3, rows); I64(4, cols);
  CHECK(tfhip_softmax_rows(ctx, x, out, rows, cols));
  return undefined(env);
}

/* gather(ctx, x, indices, out, outer, axisDim, inner, nIndices) */
static napi_value js_gather(napi_env env, napi_callback_info info) {
  ARGS(8);
  I64(1, x); I64(2, idx); I64(3, out); I64(4, outer); I64(5, axis_dim); I64(6, inner); I64(7, n);
  CHECK(tfhip_gather(ctx, x, idx, out, outer, axis_dim, inner, n));
  return undefined(env);
}

/* transpose(ctx, x, xShape, perm, out) */
static napi_value js_transpose(napi_env env, napi_callback_info info) {
  ARGS(5);
  I64(1, x);
  const int32_t* shape; size_t rank;
  if (!arg_i32_array(env, argv[2], &shape, &rank)) return NULL;
  const int32_t* perm; size_t plen;
  if (!arg_i32_array(env, argv[3], &perm, &plen)) return NULL;
  I64(4, out);
  if (plen != rank) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: perm and shape differ in length");
    return NULL;
  }
  CHECK(tfhip_transpose(ctx, x, shape, (int)rank, perm, out));
  return undefined(env);
}

/* Float64Array -> pointer + length (element strides and offsets: exact up to 2^53) */
static int arg_f64_array(napi_env env, napi_value v, const double** data, size_t* len) {
  napi_typedarray_type type;
  void* p;
  if (napi_get_typedarray_info(env, v, &type, len, &p, NULL, NULL) != napi_ok ||
      type != napi_float64_array) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: expected a Float64Array");
    return 0;
  }
  *data = (const double*)p;
  return 1;
}

/* stridedCopy(ctx, x, out, region Int32Array, xStrides Float64Array, xOffset,
 *             outStrides Float64Array, outOffset) */
static napi_value js_strided_copy(napi_env env, napi_callback_info info) {
  ARGS(8);
  I64(1, x); I64(2, out);
  const int32_t* region; size_t rank;
  if (!arg_i32_array(env, argv[3], &region, &rank)) return NULL;
  const double *xs, *os; size_t nx, no;
  if (!arg_f64_array(env, argv[4], &xs, &nx)) return NULL;
  I64(5, x_off);
  if (!arg_f64_array(env, argv[6], &os, &no)) return NULL;
  I64(7, out_off);
  if (nx != rank || no != rank || rank > 8) {
    napi_throw_type_error(env, NULL, "tfjs_hip.node: box arrays differ in length or rank > 8");
    return NULL;
  }
  int64_t xs64[8], os64[8];
  for (size_t i = 0; i < rank; i++) {
    xs64[i] = (int64_t)xs[i];
    os64[i] = (int64_t)os[i];
  }
  CHECK(tfhip_strided_copy(ctx, x, out, (int)rank, region, xs64, x_off, os64, out_off));
  return undefined(env);
}

/* logicalNot(ctx, x, out) */
static napi_value js_logical_not(napi_env env, napi_callback_info info) {
  ARGS(3);
  I64(1, x); I64(2, out);
  CHECK(tfhip_logical_not(ctx, x, out));
  return undefined(env);
}

/* batchnorm(ctx, x, mean, variance, offset|-1, scale|-1, epsilon, out) */
static napi_value js_batchnorm(napi_env env, napi_callback_info info) {
  ARGS(8);
  I64(1, x); I64(2, mean); I64(3, variance); I64(4, offset); I64(5, scale);
  double eps;
  if (!arg_f64(env, argv[6], &eps)) return NULL;
  I64(7, out);
  CHECK(tfhip_batchnorm(ctx, x, mean, variance, offset, scale, (float)eps, out));
  return undefined(env);
}

/* resizeBilinear(ctx, x, out, batch, inH, inW, channels, outH, outW, alignCorners) */
static napi_value js_resize_bilinear(napi_env env, napi_callback_info info) {
  ARGS(10);
  I64(1, x); I64(2, out);
  int v[7];
  for (int i = 0; i < 7; i++)
    if (!arg_int(env, argv[3 + i], &v[i])) return NULL;
  CHECK(tfhip_resize_bilinear(ctx, x, out, v[0], v[1], v[2], v[3], v[4], v[5], v[6]));
  return undefined(env);
}

/* oneHot(ctx, indices, out, depth, onValue, offValue) */
static napi_value js_one_hot(napi_env env, napi_callback_info info) {
  ARGS(6);
  I64(1, idx); I64(2, out);
  int depth;
  if (!arg_int(env, argv[3], &depth)) return NULL;
  double on, off;
  if (!arg_f64(env, argv[4], &on) || !arg_f64(env, argv[5], &off)) return NULL;
  CHECK(tfhip_one_hot(ctx, idx, out, depth, (float)on, (float)off));
  return undefined(env);
}

static napi_value module_init(napi_env env, napi_value exports) {
  static const struct { const char* name; napi_callback fn; } fns[] = {
      {"init", js_init}, {"destroy", js_destroy}, {"register", js_register},
      {"write", js_write}, {"read", js_read}, {"dispose", js_dispose},
      {"memInfo", js_mem_info}, {"sync", js_sync}, {"selectStream", js_select_stream}, {"timeBegin", js_time_begin},
      {"timeEnd", js_time_end}, {"timeKernels", js_time_kernels},
      {"timePerKernel", js_time_per_kernel}, {"hostAlloc", js_host_alloc},
      {"readAsync", js_read_async}, {"lastKernel", js_last_kernel}, {"matmul", js_matmul}, {"matmulNoalloc", js_matmul_noalloc},
      {"conv2d", js_conv2d}, {"depthwiseConv2d", js_depthwise}, {"separableConv2d", js_separable},
      {"separableSingleKernel", js_separable_single_kernel}, {"pool2d", js_pool2d},
      {"binary", js_binary}, {"unary", js_unary}, {"cast", js_cast}, {"copy", js_copy},
      {"dequantize", js_dequantize}, {"fill", js_fill}, {"reduce", js_reduce},
      {"softmaxRows", js_softmax_rows}, {"gather", js_gather}, {"transpose", js_transpose},
      {"stridedCopy", js_strided_copy}, {"logicalNot", js_logical_not},
      {"batchnorm", js_batchnorm}, {"resizeBilinear", js_resize_bilinear},
      {"oneHot", js_one_hot}, {"conv2dDerInput", js_conv2d_der_input},
      {"conv2dDerFilter", js_conv2d_der_filter},
      {"depthwiseConv2dDerInput", js_depthwise_der_input},
      {"depthwiseConv2dDerFilter", js_depthwise_der_filter},
      {"pool2dBackprop", js_pool2d_backprop}, {"resizeNearest", js_resize_nearest},
      {"select", js_select}, {"cumsum", js_cumsum}, {"lrn", js_lrn}, {"lrnGrad", js_lrn_grad},
      {"graphBegin", js_graph_begin}, {"graphEnd", js_graph_end}, {"graphLaunch", js_graph_launch},
      {"graphDestroy", js_graph_destroy}, {"topk", js_topk}, {"gatherNd", js_gather_nd},
      {"scatterNd", js_scatter_nd}, {"cropAndResize", js_crop_and_resize},
      {"resizeBilinearBackprop", js_resize_bilinear_backprop},
      {"resizeNearestBackprop", js_resize_nearest_backprop}, {"fft", js_fft}};
  for (size_t i = 0; i < sizeof fns / sizeof fns[0]; i++) {
    napi_value f;
    if (napi_create_function(env, fns[i].name, NAPI_AUTO_LENGTH, fns[i].fn, NULL, &f) != napi_ok ||
        napi_set_named_property(env, exports, fns[i].name, f) != napi_ok) {
      napi_throw_error(env, NULL, "tfjs_hip.node: could not export a function");
      return NULL;
    }
  }
  return exports;
}

NAPI_MODULE(NODE_GYP_MODULE_NAME, module_init)
