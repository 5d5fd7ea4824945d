// Elementwise kernels: broadcasting binary ops, unary ops, cast, fill, copy.
// Replaces backend_cpu.ts:440-481, 557-580, 1094-1126, 1191-1209, 1265-1308, 3515-3549,
// 3816-3836 of the reference.  All of them stream HBM once: coalesced 16-byte accesses
// on the contiguous paths, grid sized to a few waves per CU with a grid-stride loop.
#include <type_traits>

#include "tfhip_internal.h"

namespace tfhip {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float load_f(const void* p, int dtype, int64_t i) {
  switch (dtype) {
    case TFHIP_FLOAT32: return static_cast<const float*>(p)[i];
    case TFHIP_INT32: return (float)static_cast<const int32_t*>(p)[i];
    default: return (float)static_cast<const uint8_t*>(p)[i];
  }
}
__device__ __forceinline__ int64_t load_i(const void* p, int dtype, int64_t i) {
  switch (dtype) {
    case TFHIP_INT32: return static_cast<const int32_t*>(p)[i];
    case TFHIP_FLOAT32: return (int64_t)static_cast<const float*>(p)[i];
    default: return static_cast<const uint8_t*>(p)[i];
  }
}

// Int32Array store of a JavaScript number: truncate, NaN/inf -> 0, wrap modulo 2^32.
__device__ __forceinline__ int32_t to_int32(float v) {
  if (!(fabsf(v) < 9.0e18f)) return 0;  // NaN, inf, and |v| >= 2^63 (a multiple of 2^32)
  return (int32_t)(uint32_t)(int64_t)v;
}

__device__ __forceinline__ float bin_f(int op, float a, float b) {
  switch (op) {
    case TFHIP_ADD: return a + b;
    case TFHIP_SUB: return a - b;
    case TFHIP_MUL: return a * b;
    case TFHIP_DIV: return a / b;
    case TFHIP_PRELU: return a < 0.f ? b * a : a;
    case TFHIP_MAXIMUM: return (a != a || b != b) ? NAN : (a > b ? a : b);
    case TFHIP_MINIMUM: return (a != a || b != b) ? NAN : (a < b ? a : b);
    case TFHIP_EQUAL: return a == b;
    case TFHIP_NOT_EQUAL: return a != b;
    case TFHIP_LESS: return a < b;
    case TFHIP_LESS_EQUAL: return a <= b;
    case TFHIP_GREATER: return a > b;
    case TFHIP_GREATER_EQUAL: return a >= b;
    case TFHIP_LOGICAL_AND: return (a != 0.f) && (b != 0.f);
    case TFHIP_LOGICAL_OR: return (a != 0.f) || (b != 0.f);
    case TFHIP_POW:
      // Math.pow: NaN exponent and (+-1) ** +-Infinity give NaN where C gives 1
      if (b != b || (fabsf(a) == 1.f && isinf(b))) return NAN;
      return powf(a, b);
    case TFHIP_SQUARED_DIFFERENCE: return (a - b) * (a - b);
    case TFHIP_MOD: {
      const float rem = fmodf(a, b);
      if ((a < 0.f && b < 0.f) || (a >= 0.f && b >= 0.f)) return rem;
      return fmodf(rem + b, b);
    }
    case TFHIP_FLOOR_DIV: return floorf(a / b);
    case TFHIP_ATAN2: return atan2f(a, b);
    default: return b >= 1.f ? a : a * (b + 1.f);  // eluDer(dy, y)
  }
}
__device__ __forceinline__ int64_t bin_i(int op, int64_t a, int64_t b) {
  switch (op) {
    case TFHIP_ADD: return a + b;
    case TFHIP_SUB: return a - b;
    case TFHIP_MUL: return a * b;
    case TFHIP_PRELU: return a < 0 ? b * a : a;
    case TFHIP_MAXIMUM: return a > b ? a : b;
    case TFHIP_MINIMUM: return a < b ? a : b;
    case TFHIP_EQUAL: return a == b;
    case TFHIP_NOT_EQUAL: return a != b;
    case TFHIP_LESS: return a < b;
    case TFHIP_LESS_EQUAL: return a <= b;
    case TFHIP_GREATER: return a > b;
    case TFHIP_GREATER_EQUAL: return a >= b;
    case TFHIP_LOGICAL_AND: return a && b;
    default: return a || b;
  }
}

constexpr int MAXR = 6;
struct BcastArgs {
  int rank;
  int out_dim[MAXR];
  int64_t a_stride[MAXR], b_stride[MAXR];
};

// mode 0: same number of elements in a, b, out.  mode 1: index = i % len (what
// backend_cpu's no-broadcast-dims fast path does, :3526-3530; covers scalars and a [C]
// operand against [...,C]).  mode 2: general N-d broadcast by strides.
template <typename OutT>
__global__ void binary_kernel(int op, const void* a, int a_dt, int64_t a_len, const void* b,
                              int b_dt, int64_t b_len, OutT* out, int64_t n, int mode,
                              BcastArgs bc) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    int64_t ia, ib;
    if (mode == 0) {
      ia = ib = i;
    } else if (mode == 1) {
      ia = a_len == n ? i : i % a_len;
      ib = b_len == n ? i : i % b_len;
    } else {
      int64_t rem = i;
      ia = ib = 0;
#pragma unroll
      for (int d = MAXR - 1; d >= 0; d--) {
        if (d < bc.rank) {
          const int c = (int)(rem % bc.out_dim[d]);
          rem /= bc.out_dim[d];
          ia += c * bc.a_stride[d];
          ib += c * bc.b_stride[d];
        }
      }
    }
    if (a_dt != TFHIP_FLOAT32 && b_dt != TFHIP_FLOAT32 && op != TFHIP_DIV && op < TFHIP_POW) {
      // integer arithmetic when neither operand is float (int32 / bool tensors)
      const int64_t r = bin_i(op, load_i(a, a_dt, ia), load_i(b, b_dt, ib));
      if (std::is_same<OutT, float>::value) out[i] = (OutT)r;
      else out[i] = (OutT)(int32_t)(uint32_t)r;   // comparisons yield 0 / 1
    } else {
      const float r = bin_f(op, load_f(a, a_dt, ia), load_f(b, b_dt, ib));
      if (std::is_same<OutT, float>::value) out[i] = (OutT)r;
      else if (sizeof(OutT) == 1) out[i] = (OutT)(r != 0.f);
      else out[i] = (OutT)to_int32(r);
    }
  }
}

// float32 x float32 -> float32, equal sizes, 16-byte aligned: the common case.
__global__ void binary_f32_vec_kernel(int op, const f32x4* a, const f32x4* b, f32x4* out,
                                      int64_t n4) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
    const f32x4 x = a[i], y = b[i];
    f32x4 r;
#pragma unroll
    for (int e = 0; e < 4; e++) r[e] = bin_f(op, x[e], y[e]);
    out[i] = r;
  }
}

// float32 [rows, C] (op) float32 [C] with C % 4 == 0: bias add / per-channel prelu.
__global__ void binary_f32_rowvec_kernel(int op, const f32x4* a, const f32x4* b, f32x4* out,
                                         int64_t n4, int c4, int b_is_first) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
    const f32x4 x = a[i], y = b[i % c4];
    f32x4 r;
#pragma unroll
    for (int e = 0; e < 4; e++) r[e] = b_is_first ? bin_f(op, y[e], x[e]) : bin_f(op, x[e], y[e]);
    out[i] = r;
  }
}

__device__ __forceinline__ float unary_f(int op, float v, float p0, float p1) {
  switch (op) {
    case TFHIP_RELU: return (v > 0.f || v != v) ? v : 0.f;
    case TFHIP_CLIP: return v > p1 ? p1 : (v < p0 ? p0 : v);
    case TFHIP_EXP: return expf(v);
    case TFHIP_LOG: return logf(v);
    case TFHIP_NEG: return -v;
    case TFHIP_ABS: return fabsf(v);
    case TFHIP_SIGMOID: return 1.f / (1.f + expf(-v));
    case TFHIP_SQRT: return sqrtf(v);
    case TFHIP_SQUARE: return v * v;
    case TFHIP_TANH: return tanhf(v);
    case TFHIP_RSQRT: return 1.f / sqrtf(v);
    case TFHIP_FLOOR: return floorf(v);
    case TFHIP_CEIL: return ceilf(v);
    case TFHIP_ROUND: return rintf(v);  // round half to even (backend_cpu.ts:1077-1090)
    case TFHIP_SIGN: return v < 0.f ? -1.f : (v > 0.f ? 1.f : 0.f);
    case TFHIP_EXPM1: return expm1f(v);
    case TFHIP_LOG1P: return log1pf(v);
    case TFHIP_RECIPROCAL: return 1.f / v;
    case TFHIP_SIN: return sinf(v);
    case TFHIP_COS: return cosf(v);
    case TFHIP_TAN: return tanf(v);
    case TFHIP_ASIN: return asinf(v);
    case TFHIP_ACOS: return acosf(v);
    case TFHIP_ATAN: return atanf(v);
    case TFHIP_SINH: return sinhf(v);
    case TFHIP_COSH: return coshf(v);
    case TFHIP_ASINH: return asinhf(v);
    case TFHIP_ACOSH: return acoshf(v);
    case TFHIP_ATANH: return atanhf(v);
    case TFHIP_ERF: {
      // ops/erf_util.ts:18-23, backend_cpu.ts:1509-1516 (no sign handling: as the reference)
      const float t = 1.f / (1.f + 0.3275911f * v);
      const float poly = ((((1.061405429f * t + -1.453152027f) * t + 1.421413741f) * t +
                           -0.284496736f) * t + 0.254829592f) * t;
      return 1.f - poly * expf(-v * v);
    }
    case TFHIP_ELU: return v >= 0.f ? v : expm1f(v);
    case TFHIP_SELU:  // ops/selu_util.ts:18-19
      return v >= 0.f ? 1.0507009873554804934193349852946f * v
                      : 1.7580993408473768599402175208123f * expm1f(v);
    case TFHIP_SOFTPLUS: {
      // backend_cpu.ts:1326-1353: threshold = log(2^-23) + 2
      const float threshold = -13.942385f;
      if (v < threshold) return expf(v);
      if (v > -threshold) return v;
      return log1pf(expf(v));
    }
    case TFHIP_STEP: return v != v ? NAN : (v > 0.f ? 1.f : p0);
    case TFHIP_IS_NAN: return v != v;
    case TFHIP_IS_INF: return isinf(v);
    default: return isfinite(v);
  }
}

template <typename OutT>
__global__ void unary_kernel(int op, const void* x, int x_dt, OutT* out, int64_t n, float p0,
                             float p1) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float r = unary_f(op, load_f(x, x_dt, i), p0, p1);
    if (std::is_same<OutT, float>::value) out[i] = (OutT)r;
    else if (sizeof(OutT) == 1) out[i] = (OutT)(r != 0.f);
    else out[i] = (OutT)to_int32(r);
  }
}

__global__ void unary_f32_vec_kernel(int op, const f32x4* x, f32x4* out, int64_t n4, float p0,
                                     float p1) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
    const f32x4 v = x[i];
    f32x4 r;
#pragma unroll
    for (int e = 0; e < 4; e++) r[e] = unary_f(op, v[e], p0, p1);
    out[i] = r;
  }
}

__global__ void convert_kernel(const void* src, int src_dt, void* dst, int dst_dt, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    if (dst_dt == TFHIP_FLOAT32) {
      static_cast<float*>(dst)[i] = load_f(src, src_dt, i);
    } else if (dst_dt == TFHIP_INT32) {
      static_cast<int32_t*>(dst)[i] = src_dt == TFHIP_FLOAT32
                                          ? to_int32(static_cast<const float*>(src)[i])
                                          : (int32_t)load_i(src, src_dt, i);
    } else {  // bool: x != 0 (NaN counts as true, as notEqual(x, 0) does)
      const bool t = src_dt == TFHIP_FLOAT32 ? !(static_cast<const float*>(src)[i] == 0.f)
                                             : load_i(src, src_dt, i) != 0;
      static_cast<uint8_t*>(dst)[i] = t ? 1 : 0;
    }
  }
}

__global__ void dequantize_kernel(const uint8_t* q, float* out, int64_t n, double scale,
                                  double mn) {
#pragma clang fp contract(off)
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    double v = (double)q[i] * scale;
    v = v + mn;
    out[i] = (float)v;
  }
}

// The same for 16-bit codes: two bytes per weight, low byte first (the byte order of a weights
// file read into a Uint16Array, io/io_utils.ts:131-133).  Read as bytes: a shard places a tensor
// at any byte offset.
__global__ void dequantize16_kernel(const uint8_t* q, float* out, int64_t n, double scale,
                                    double mn) {
#pragma clang fp contract(off)
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const unsigned code = (unsigned)q[2 * i] | ((unsigned)q[2 * i + 1] << 8);
    double v = (double)code * scale;
    v = v + mn;
    out[i] = (float)v;
  }
}

template <typename T>
__global__ void fill_kernel(T* out, int64_t n, T value) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = value;
}

static int grid_for(tfhip_ctx* ctx, int64_t work_items, int block) {
  const int64_t want = ceil_div(work_items, block);
  const int64_t cap = (int64_t)ctx->num_cus * 16;
  return (int)(want < 1 ? 1 : (want > cap ? cap : want));
}

int launch_convert(tfhip_ctx* ctx, const void* src, int src_dtype, void* dst, int dst_dtype,
                   int64_t n) {
  if (n == 0) return TFHIP_OK;
  tfhip::launch(ctx, convert_kernel, dim3(grid_for(ctx, n, 256)), dim3(256), 0, src,
                     src_dtype, dst, dst_dtype, n);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_binary(tfhip_ctx* ctx, int op, int64_t a, const int32_t* a_shape,
                            int a_rank, int64_t b, const int32_t* b_shape, int b_rank,
                            int64_t out) {
  if (!ctx) return TFHIP_EINVAL;
  if (op < TFHIP_ADD || op > TFHIP_ELU_DER) return ctx->fail(TFHIP_EINVAL, "binary: unknown op %d", op);
  const bool predicate = op >= TFHIP_EQUAL && op <= TFHIP_LOGICAL_OR;
  if (a_rank < 0 || b_rank < 0 || a_rank > MAXR || b_rank > MAXR)
    return ctx->fail(TFHIP_ENOTSUP, "binary: rank above %d", MAXR);
  TFHIP_GET(ctx, ba, a);
  TFHIP_GET(ctx, bb, b);
  TFHIP_GET(ctx, bo, out);
  if (ba->dtype == TFHIP_UINT8Q || bb->dtype == TFHIP_UINT8Q || bo->dtype == TFHIP_UINT8Q ||
      (bo->dtype == TFHIP_BOOL) != predicate)
    return ctx->fail(TFHIP_EINVAL, "binary: unsupported storage dtype (comparisons and logical "
                                   "ops write bool, arithmetic writes float32 or int32)");
  // assertAndGetBroadcastShape (ops/broadcast_util.ts:61-87)
  const int rank = a_rank > b_rank ? a_rank : b_rank;
  BcastArgs bc = {};
  bc.rank = rank;
  int64_t n = 1, a_len = 1, b_len = 1;
  bool a_bcast = false, b_bcast = false;
  for (int i = 0; i < a_rank; i++) a_len *= a_shape[i];
  for (int i = 0; i < b_rank; i++) b_len *= b_shape[i];
  int64_t sa = 1, sb = 1;
  for (int i = 0; i < rank; i++) {  // i counts from the innermost dimension
    const int ad = i < a_rank ? a_shape[a_rank - 1 - i] : 1;
    const int bd = i < b_rank ? b_shape[b_rank - 1 - i] : 1;
    int od;
    if (ad == 1) od = bd;
    else if (bd == 1) od = ad;
    else if (ad != bd)
      return ctx->fail(TFHIP_EINVAL, "Operands could not be broadcast together");
    else od = ad;
    const int d = rank - 1 - i;
    bc.out_dim[d] = od;
    bc.a_stride[d] = (i < a_rank && !(ad == 1 && od > 1)) ? sa : 0;
    bc.b_stride[d] = (i < b_rank && !(bd == 1 && od > 1)) ? sb : 0;
    if (i < a_rank && ad == 1 && od > 1) a_bcast = true;  // getBroadcastDims (:27-42)
    if (i < b_rank && bd == 1 && od > 1) b_bcast = true;
    sa *= ad;
    sb *= bd;
    n *= od;
  }
  if (ba->numel != a_len || bb->numel != b_len || bo->numel != n)
    return ctx->fail(TFHIP_EINVAL, "binary: buffer sizes do not match the shapes given");
  if (n == 0) return TFHIP_OK;
  const bool all_f32 = ba->dtype == TFHIP_FLOAT32 && bb->dtype == TFHIP_FLOAT32 &&
                       bo->dtype == TFHIP_FLOAT32;
  const int block = 256;
  if (!predicate && all_f32 && a_len == n && b_len == n && n % 4 == 0 && aligned16(ba->ptr) &&
      aligned16(bb->ptr) && aligned16(bo->ptr)) {
    tfhip::launch(ctx, binary_f32_vec_kernel, dim3(grid_for(ctx, n / 4, block)), dim3(block), 0, op, (const f32x4*)ba->ptr, (const f32x4*)bb->ptr,
                       (f32x4*)bo->ptr, n / 4);
    TFHIP_LAUNCH_CHECK(ctx);
    return TFHIP_OK;
  }
  const int last = rank ? bc.out_dim[rank - 1] : 1;
  if (!predicate && all_f32 && !a_bcast && !b_bcast && last % 4 == 0 && aligned16(ba->ptr) &&
      aligned16(bb->ptr) && aligned16(bo->ptr) &&
      ((a_len == n && b_len == last) || (b_len == n && a_len == last))) {
    const bool b_small = b_len == last && a_len == n;
    tfhip::launch(ctx, binary_f32_rowvec_kernel, dim3(grid_for(ctx, n / 4, block)), dim3(block), 0, op, (const f32x4*)(b_small ? ba->ptr : bb->ptr),
                       (const f32x4*)(b_small ? bb->ptr : ba->ptr), (f32x4*)bo->ptr, n / 4,
                       last / 4, b_small ? 0 : 1);
    TFHIP_LAUNCH_CHECK(ctx);
    return TFHIP_OK;
  }
  const int mode = (a_len == n && b_len == n) ? 0 : (!a_bcast && !b_bcast) ? 1 : 2;
  const dim3 grid(grid_for(ctx, n, block));
  if (bo->dtype == TFHIP_FLOAT32)
    tfhip::launch(ctx, binary_kernel<float>, grid, dim3(block), 0, op, ba->ptr,
                       ba->dtype, a_len, bb->ptr, bb->dtype, b_len, (float*)bo->ptr, n, mode, bc);
  else if (bo->dtype == TFHIP_BOOL)
    tfhip::launch(ctx, binary_kernel<uint8_t>, grid, dim3(block), 0, op, ba->ptr,
                       ba->dtype, a_len, bb->ptr, bb->dtype, b_len, (uint8_t*)bo->ptr, n, mode, bc);
  else
    tfhip::launch(ctx, binary_kernel<int32_t>, grid, dim3(block), 0, op, ba->ptr,
                       ba->dtype, a_len, bb->ptr, bb->dtype, b_len, (int32_t*)bo->ptr, n, mode, bc);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_unary(tfhip_ctx* ctx, int op, int64_t x, int64_t out, float p0, float p1) {
  if (!ctx) return TFHIP_EINVAL;
  if (op < TFHIP_RELU || op > TFHIP_IS_FINITE) return ctx->fail(TFHIP_EINVAL, "unary: unknown op %d", op);
  const bool predicate = op >= TFHIP_IS_NAN;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (bx->numel != bo->numel) return ctx->fail(TFHIP_EINVAL, "unary: size mismatch");
  if (bx->dtype == TFHIP_UINT8Q || bo->dtype == TFHIP_UINT8Q ||
      (bo->dtype == TFHIP_BOOL) != predicate)
    return ctx->fail(TFHIP_EINVAL, "unary: unsupported storage dtype (isNaN/isInf/isFinite write "
                                   "bool, the others float32 or int32)");
  const int64_t n = bx->numel;
  if (n == 0) return TFHIP_OK;
  const int block = 256;
  if (bx->dtype == TFHIP_FLOAT32 && bo->dtype == TFHIP_FLOAT32 && n % 4 == 0 &&
      aligned16(bx->ptr) && aligned16(bo->ptr)) {
    tfhip::launch(ctx, unary_f32_vec_kernel, dim3(grid_for(ctx, n / 4, block)), dim3(block), 0, op, (const f32x4*)bx->ptr, (f32x4*)bo->ptr, n / 4, p0, p1);
  } else if (bo->dtype == TFHIP_FLOAT32) {
    tfhip::launch(ctx, unary_kernel<float>, dim3(grid_for(ctx, n, block)), dim3(block), 0, op, bx->ptr, bx->dtype, (float*)bo->ptr, n, p0, p1);
  } else if (bo->dtype == TFHIP_BOOL) {
    tfhip::launch(ctx, unary_kernel<uint8_t>, dim3(grid_for(ctx, n, block)), dim3(block), 0, op, bx->ptr, bx->dtype, (uint8_t*)bo->ptr, n, p0, p1);
  } else {
    tfhip::launch(ctx, unary_kernel<int32_t>, dim3(grid_for(ctx, n, block)), dim3(block), 0, op, bx->ptr, bx->dtype, (int32_t*)bo->ptr, n, p0, p1);
  }
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_cast(tfhip_ctx* ctx, int64_t x, int64_t out) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (bx->numel != bo->numel) return ctx->fail(TFHIP_EINVAL, "cast: size mismatch");
  if (bx->dtype == TFHIP_UINT8Q || bo->dtype == TFHIP_UINT8Q)
    return ctx->fail(TFHIP_EINVAL, "cast: quantised buffers are dequantised by the dense kernels");
  return launch_convert(ctx, bx->ptr, bx->dtype, bo->ptr, bo->dtype, bx->numel);
}

extern "C" int tfhip_dequantize(tfhip_ctx* ctx, int64_t x, int64_t out, const tfhip_qparams* q) {
  if (!ctx || !q) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  const bool wide = bo->numel > 0 && bx->numel == 2 * bo->numel;  // 16-bit codes
  if (bx->dtype != TFHIP_UINT8Q || bo->dtype != TFHIP_FLOAT32 || (bx->numel != bo->numel && !wide))
    return ctx->fail(TFHIP_EINVAL, "dequantize: needs a quantised input of one or two bytes per "
                                   "element and a float32 output");
  if (bo->numel == 0) return TFHIP_OK;
  tfhip::launch(ctx, wide ? dequantize16_kernel : dequantize_kernel,
                dim3(grid_for(ctx, bo->numel, 256)), dim3(256), 0, (const uint8_t*)bx->ptr,
                (float*)bo->ptr, bo->numel, q->scale, q->min);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_fill(tfhip_ctx* ctx, int64_t out, double value) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bo, out);
  const int64_t n = bo->numel;
  if (n == 0) return TFHIP_OK;
  const dim3 grid(grid_for(ctx, n, 256)), block(256);
  if (bo->dtype == TFHIP_FLOAT32)
    tfhip::launch(ctx, fill_kernel<float>, grid, block, 0, (float*)bo->ptr, n,
                       (float)value);
  else if (bo->dtype == TFHIP_INT32)
    tfhip::launch(ctx, fill_kernel<int32_t>, grid, block, 0, (int32_t*)bo->ptr, n,
                       (int32_t)value);
  else
    tfhip::launch(ctx, fill_kernel<uint8_t>, grid, block, 0, (uint8_t*)bo->ptr, n,
                       (uint8_t)value);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_copy(tfhip_ctx* ctx, int64_t x, int64_t out) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (bx->nbytes != bo->nbytes) return ctx->fail(TFHIP_EINVAL, "copy: size mismatch");
  if (bx->nbytes)
    TFHIP_HIP(ctx, hipMemcpyAsync(bo->ptr, bx->ptr, bx->nbytes, hipMemcpyDeviceToDevice,
                                  ctx->stream));
  return TFHIP_OK;
}
