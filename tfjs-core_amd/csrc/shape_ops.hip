// Data-movement and pointwise kernels that converter graphs use around the convolutions:
// a strided box copy (slice, stridedSlice, reverse, concat, pad, tile), logicalNot,
// batchNormalization, resizeBilinear, oneHot.  Replaces backend_cpu.ts:292-433, 795-804,
// 2152-2176, 2875-2936, 3167-3213, 3325-3339 of the reference.  All of them stream HBM
// once; the innermost dimension of the box runs along the lanes.
#include "tfhip_internal.h"

namespace tfhip {

constexpr int MAXBOX = 8;
struct BoxArgs {
  int rank;
  int region[MAXBOX];
  int64_t x_stride[MAXBOX], out_stride[MAXBOX];
  int64_t x_offset, out_offset;
};

template <typename T>
__global__ void strided_copy_kernel(const T* __restrict__ x, T* __restrict__ out, int64_t n,
                                    BoxArgs b) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    int64_t rem = i, src = b.x_offset, dst = b.out_offset;
#pragma unroll
    for (int d = MAXBOX - 1; d >= 0; d--) {
      if (d < b.rank) {
        const int64_t c = rem % b.region[d];
        rem /= b.region[d];
        src += c * b.x_stride[d];
        dst += c * b.out_stride[d];
      }
    }
    out[dst] = x[src];
  }
}

__global__ void logical_not_kernel(const uint8_t* x, uint8_t* out, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = x[i] ? 0 : 1;
}

// The reference evaluates offset + (x - mean) * scale / sqrt(variance + eps) in double and
// rounds once at the store; float32 arithmetic here stays within 1e-6 relative of that.
__global__ void batchnorm_kernel(const float* x, const float* mean, int64_t n_mean,
                                 const float* variance, int64_t n_var, const float* offset,
                                 int64_t n_off, const float* scale, int64_t n_scale, float eps,
                                 float* out, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float m = mean[i % n_mean], v = variance[i % n_var];
    const float s = scale ? scale[i % n_scale] : 1.f;
    const float o = offset ? offset[i % n_off] : 0.f;
    out[i] = o + (x[i] - m) * s / sqrtf(v + eps);
  }
}

// One lane per output element, channel fastest.  Source coordinates as the reference
// computes them: ratio = effective input size / effective output size, floor / ceil
// neighbours, ceil clamped to the last row / column.
__global__ void resize_bilinear_kernel(const float* x, float* out, int batch, int in_h, int in_w,
                                       int ch, int out_h, int out_w, double ratio_h,
                                       double ratio_w) {
  const int64_t n = (int64_t)batch * out_h * out_w * ch;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int d = (int)(i % ch);
    int64_t t = i / ch;
    const int c = (int)(t % out_w);
    t /= out_w;
    const int r = (int)(t % out_h);
    const int b = (int)(t / out_h);
    // double throughout, like the reference: a float product can land on the other side of
    // an integer and pick different neighbours
    const double fr = ratio_h * r, fc = ratio_w * c;
    const int r0 = (int)floor(fr), c0 = (int)floor(fc);
    const int r1 = min(in_h - 1, (int)ceil(fr)), c1 = min(in_w - 1, (int)ceil(fc));
    const double wr = fr - r0, wc = fc - c0;
    const float* xb = x + (int64_t)b * in_h * in_w * ch + d;
    const double tl = xb[((int64_t)r0 * in_w + c0) * ch], tr = xb[((int64_t)r0 * in_w + c1) * ch];
    const double bl = xb[((int64_t)r1 * in_w + c0) * ch], br = xb[((int64_t)r1 * in_w + c1) * ch];
    const double top = tl + (tr - tl) * wc;
    const double bot = bl + (br - bl) * wc;
    out[i] = (float)(top + (bot - top) * wr);
  }
}

// Nearest neighbour: source row / column = min(in - 1, floor(ratio * r)), or round half up
// (JavaScript's Math.round) with align_corners, in double as the reference computes them.
__global__ void resize_nearest_kernel(const float* x, float* out, int batch, int in_h, int in_w,
                                      int ch, int out_h, int out_w, double ratio_h,
                                      double ratio_w, int align_corners) {
  const int64_t n = (int64_t)batch * out_h * out_w * ch;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int d = (int)(i % ch);
    int64_t t = i / ch;
    const int c = (int)(t % out_w);
    t /= out_w;
    const int r = (int)(t % out_h);
    const int b = (int)(t / out_h);
    const double fr = ratio_h * r, fc = ratio_w * c;
    const int sr = min(in_h - 1, (int)(align_corners ? floor(fr + 0.5) : floor(fr)));
    const int sc = min(in_w - 1, (int)(align_corners ? floor(fc + 0.5) : floor(fc)));
    out[i] = x[(((int64_t)b * in_h + sr) * in_w + sc) * ch + d];
  }
}

// out[i] = cond[i / inner] ? a[i] : b[i]; T = 4-byte (float32 / int32) or 1-byte (bool) elements.
template <typename T>
__global__ void select_kernel(const uint8_t* cond, const T* a, const T* b, T* out, int64_t n,
                              int64_t inner) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = cond[i / inner] == 1 ? a[i] : b[i];
}

template <typename T>
__global__ void one_hot_kernel(const int32_t* idx, T* out, int64_t n_idx, int depth, T on, T off) {
  const int64_t n = n_idx * depth;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t e = i / depth;
    const int k = (int)(i - e * depth);
    out[i] = idx[e] == k ? on : off;
  }
}

static int grid_for(tfhip_ctx* ctx, int64_t work_items, int block) {
  const int64_t want = ceil_div(work_items, block);
  const int64_t cap = (int64_t)ctx->num_cus * 16;
  return (int)(want < 1 ? 1 : (want > cap ? cap : want));
}

}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_strided_copy(tfhip_ctx* ctx, int64_t x, int64_t out, int rank,
                                  const int32_t* region, const int64_t* x_strides,
                                  int64_t x_offset, const int64_t* out_strides,
                                  int64_t out_offset) {
  if (!ctx) return TFHIP_EINVAL;
  if (rank < 0 || rank > MAXBOX) return ctx->fail(TFHIP_ENOTSUP, "strided copy: rank above %d", MAXBOX);
  if (rank > 0 && (!region || !x_strides || !out_strides)) return ctx->fail(TFHIP_EINVAL, "strided copy: null box");
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (bx->dtype == TFHIP_UINT8Q || bo->dtype == TFHIP_UINT8Q || dtype_size(bx->dtype) != dtype_size(bo->dtype))
    return ctx->fail(TFHIP_EINVAL, "strided copy: source and destination element sizes differ");
  BoxArgs b = {};
  b.rank = rank;
  b.x_offset = x_offset;
  b.out_offset = out_offset;
  int64_t n = 1;
  // smallest and largest index the box touches on either side
  int64_t x_lo = x_offset, x_hi = x_offset, o_lo = out_offset, o_hi = out_offset;
  for (int d = 0; d < rank; d++) {
    if (region[d] < 0) return ctx->fail(TFHIP_EINVAL, "strided copy: negative extent");
    b.region[d] = region[d];
    b.x_stride[d] = x_strides[d];
    b.out_stride[d] = out_strides[d];
    n *= region[d];
    if (region[d] > 0) {
      const int64_t xs = x_strides[d] * (region[d] - 1), os = out_strides[d] * (region[d] - 1);
      if (xs < 0) x_lo += xs; else x_hi += xs;
      if (os < 0) o_lo += os; else o_hi += os;
    }
  }
  if (n == 0) return TFHIP_OK;
  if (x_lo < 0 || x_hi >= bx->numel || o_lo < 0 || o_hi >= bo->numel)
    return ctx->fail(TFHIP_EINVAL, "strided copy: the box leaves a buffer (source %lld..%lld of "
                                   "%lld, destination %lld..%lld of %lld)",
                     (long long)x_lo, (long long)x_hi, (long long)bx->numel, (long long)o_lo,
                     (long long)o_hi, (long long)bo->numel);
  if (bx->ptr == bo->ptr) return ctx->fail(TFHIP_EINVAL, "strided copy: in place is not supported");
  const dim3 grid(grid_for(ctx, n, 256)), block(256);
  if (dtype_size(bx->dtype) == 4)
    tfhip::launch(ctx, strided_copy_kernel<int32_t>, grid, block, 0,
                       (const int32_t*)bx->ptr, (int32_t*)bo->ptr, n, b);
  else
    tfhip::launch(ctx, strided_copy_kernel<uint8_t>, grid, block, 0,
                       (const uint8_t*)bx->ptr, (uint8_t*)bo->ptr, n, b);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_logical_not(tfhip_ctx* ctx, int64_t x, int64_t out) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (bx->dtype != TFHIP_BOOL || bo->dtype != TFHIP_BOOL || bx->numel != bo->numel)
    return ctx->fail(TFHIP_EINVAL, "logicalNot: operand and result must be bool of one size");
  if (bx->numel == 0) return TFHIP_OK;
  tfhip::launch(ctx, logical_not_kernel, dim3(grid_for(ctx, bx->numel, 256)), dim3(256), 0, (const uint8_t*)bx->ptr, (uint8_t*)bo->ptr, bx->numel);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_batchnorm(tfhip_ctx* ctx, int64_t x, int64_t mean, int64_t variance,
                               int64_t offset, int64_t scale, float epsilon, int64_t out) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bm, mean);
  TFHIP_GET(ctx, bv, variance);
  TFHIP_GET(ctx, bo, out);
  tfhip::Buf *boff = nullptr, *bs = nullptr;
  if (offset >= 0 && !(boff = ctx->find(offset))) return TFHIP_ENOENT;
  if (scale >= 0 && !(bs = ctx->find(scale))) return TFHIP_ENOENT;
  if (bo->dtype != TFHIP_FLOAT32 || bo->numel != bx->numel)
    return ctx->fail(TFHIP_EINVAL, "batchNorm: result must be float32 of the size of x");
  if (bx->numel == 0) return TFHIP_OK;
  if (bm->numel == 0 || bv->numel == 0 || (boff && boff->numel == 0) || (bs && bs->numel == 0))
    return ctx->fail(TFHIP_EINVAL, "batchNorm: empty statistics");
  Temp tx(ctx), tm(ctx), tv(ctx), to(ctx), ts(ctx);
  const float *xf, *mf, *vf, *of = nullptr, *sf = nullptr;
  int rc;
  if ((rc = as_f32(ctx, bx, &tx, &xf)) || (rc = as_f32(ctx, bm, &tm, &mf)) ||
      (rc = as_f32(ctx, bv, &tv, &vf)))
    return rc;
  if (boff && (rc = as_f32(ctx, boff, &to, &of))) return rc;
  if (bs && (rc = as_f32(ctx, bs, &ts, &sf))) return rc;
  tfhip::launch(ctx, batchnorm_kernel, dim3(grid_for(ctx, bx->numel, 256)), dim3(256), 0, xf, mf, bm->numel, vf, bv->numel, of, boff ? boff->numel : 1, sf,
                     bs ? bs->numel : 1, epsilon, (float*)bo->ptr, bx->numel);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_resize_bilinear(tfhip_ctx* ctx, int64_t x, int64_t out, int batch, int in_h,
                                     int in_w, int channels, int out_h, int out_w,
                                     int align_corners) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (batch < 0 || in_h < 0 || in_w < 0 || channels < 0 || out_h < 0 || out_w < 0)
    return ctx->fail(TFHIP_EINVAL, "resizeBilinear: bad geometry");
  if (bx->numel != (int64_t)batch * in_h * in_w * channels ||
      bo->numel != (int64_t)batch * out_h * out_w * channels || bo->dtype != TFHIP_FLOAT32)
    return ctx->fail(TFHIP_EINVAL, "resizeBilinear: buffers do not match the shapes given");
  if (bo->numel == 0) return TFHIP_OK;
  if (in_h == 0 || in_w == 0) return ctx->fail(TFHIP_EINVAL, "resizeBilinear: empty input image");
  Temp tx(ctx);
  const float* xf;
  int rc;
  if ((rc = as_f32(ctx, bx, &tx, &xf))) return rc;
  // effective sizes and ratios (backend_cpu.ts:2885-2898)
  const double eh_in = (align_corners && out_h > 1) ? in_h - 1 : in_h;
  const double ew_in = (align_corners && out_w > 1) ? in_w - 1 : in_w;
  const double eh_out = (align_corners && out_h > 1) ? out_h - 1 : out_h;
  const double ew_out = (align_corners && out_w > 1) ? out_w - 1 : out_w;
  tfhip::launch(ctx, resize_bilinear_kernel, dim3(grid_for(ctx, bo->numel, 256)), dim3(256), 0, xf, (float*)bo->ptr, batch, in_h, in_w, channels, out_h, out_w,
                     eh_in / eh_out, ew_in / ew_out);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_one_hot(tfhip_ctx* ctx, int64_t indices, int64_t out, int depth,
                             float on_value, float off_value) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bi, indices);
  TFHIP_GET(ctx, bo, out);
  if (bi->dtype != TFHIP_INT32) return ctx->fail(TFHIP_EINVAL, "oneHot: indices must be int32");
  if (depth < 0 || bo->numel != bi->numel * depth ||
      (bo->dtype != TFHIP_INT32 && bo->dtype != TFHIP_FLOAT32))
    return ctx->fail(TFHIP_EINVAL, "oneHot: result must hold indices x depth int32 or float32 values");
  if (bo->numel == 0) return TFHIP_OK;
  const dim3 grid(grid_for(ctx, bo->numel, 256)), block(256);
  if (bo->dtype == TFHIP_INT32)
    tfhip::launch(ctx, one_hot_kernel<int32_t>, grid, block, 0,
                       (const int32_t*)bi->ptr, (int32_t*)bo->ptr, bi->numel, depth,
                       (int32_t)on_value, (int32_t)off_value);
  else
    tfhip::launch(ctx, one_hot_kernel<float>, grid, block, 0,
                       (const int32_t*)bi->ptr, (float*)bo->ptr, bi->numel, depth, on_value,
                       off_value);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_resize_nearest(tfhip_ctx* ctx, int64_t x, int64_t out, int batch, int in_h,
                                    int in_w, int channels, int out_h, int out_w,
                                    int align_corners) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (batch < 0 || in_h < 0 || in_w < 0 || channels < 0 || out_h < 0 || out_w < 0)
    return ctx->fail(TFHIP_EINVAL, "resizeNearestNeighbor: bad geometry");
  if (bx->numel != (int64_t)batch * in_h * in_w * channels ||
      bo->numel != (int64_t)batch * out_h * out_w * channels || bo->dtype != TFHIP_FLOAT32)
    return ctx->fail(TFHIP_EINVAL, "resizeNearestNeighbor: buffers do not match the shapes given");
  if (bo->numel == 0) return TFHIP_OK;
  if (in_h == 0 || in_w == 0) return ctx->fail(TFHIP_EINVAL, "resizeNearestNeighbor: empty input image");
  Temp tx(ctx);
  const float* xf;
  int rc;
  if ((rc = as_f32(ctx, bx, &tx, &xf))) return rc;
  // effective sizes and ratios (backend_cpu.ts:3025-3038)
  const double eh_in = (align_corners && out_h > 1) ? in_h - 1 : in_h;
  const double ew_in = (align_corners && out_w > 1) ? in_w - 1 : in_w;
  const double eh_out = (align_corners && out_h > 1) ? out_h - 1 : out_h;
  const double ew_out = (align_corners && out_w > 1) ? out_w - 1 : out_w;
  tfhip::launch(ctx, resize_nearest_kernel, dim3(grid_for(ctx, bo->numel, 256)), dim3(256), 0, xf, (float*)bo->ptr, batch, in_h, in_w, channels, out_h, out_w,
                     eh_in / eh_out, ew_in / ew_out, align_corners ? 1 : 0);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_select(tfhip_ctx* ctx, int64_t condition, int64_t a, int64_t b, int64_t out,
                            int64_t inner) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bc, condition);
  TFHIP_GET(ctx, ba, a);
  TFHIP_GET(ctx, bb, b);
  TFHIP_GET(ctx, bo, out);
  if (bc->dtype != TFHIP_BOOL) return ctx->fail(TFHIP_EINVAL, "select: condition must be bool");
  if (ba->dtype == TFHIP_UINT8Q || ba->dtype != bb->dtype || ba->dtype != bo->dtype)
    return ctx->fail(TFHIP_EINVAL, "select: a, b and the result must share one storage dtype");
  if (inner < 1 || ba->numel != bb->numel || ba->numel != bo->numel ||
      bc->numel * inner != ba->numel)
    return ctx->fail(TFHIP_EINVAL, "select: sizes do not match (condition %lld x %lld, a %lld, b %lld)",
                     (long long)bc->numel, (long long)inner, (long long)ba->numel,
                     (long long)bb->numel);
  if (bo->numel == 0) return TFHIP_OK;
  const dim3 grid(grid_for(ctx, bo->numel, 256)), block(256);
  const uint8_t* c = static_cast<const uint8_t*>(bc->ptr);
  if (dtype_size(ba->dtype) == 4)
    tfhip::launch(ctx, select_kernel<int32_t>, grid, block, 0, c,
                       (const int32_t*)ba->ptr, (const int32_t*)bb->ptr, (int32_t*)bo->ptr,
                       bo->numel, inner);
  else
    tfhip::launch(ctx, select_kernel<uint8_t>, grid, block, 0, c,
                       (const uint8_t*)ba->ptr, (const uint8_t*)bb->ptr, (uint8_t*)bo->ptr,
                       bo->numel, inner);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}
