// Index-driven data movement and the resampling kernels around it: gatherND, scatterND /
// sparseToDense, resizeBilinearBackprop, resizeNearestNeighborBackprop, cropAndResize.
// Replaces backend_cpu.ts:2938-3013, 3070-3165, 3622-3757, 3759-3836, 3842-3889 of the
// reference.  Every result element is produced by one lane that visits its contributions in
// the order the reference's loops do, so sums round the same way and nothing depends on
// scheduling (no atomics on data).
#include <climits>

#include "tfhip_internal.h"

// The reference rounds every product before it adds it (JavaScript has no fused multiply-add);
// a contracted a * b + c keeps more bits and now and then lands on the neighbouring float32 or
// on the other side of an integer coordinate.
#pragma clang fp contract(off)

namespace tfhip {

constexpr int MAX_SLICE_RANK = 8;
struct SliceStrides {
  int rank;
  int64_t stride[MAX_SLICE_RANK];
};

static unsigned blocks_for(tfhip_ctx* ctx, int64_t items) {
  const int64_t blocks = (items + 255) / 256;
  const int64_t cap = (int64_t)ctx->num_cus * 16;
  return (unsigned)(blocks < 1 ? 1 : blocks > cap ? cap : blocks);
}

__global__ void set_int_kernel(int* p, int v) {
  if (blockIdx.x == 0 && threadIdx.x == 0) *p = v;
}

// flat[i] = sum_j indices[i, j] * stride[j] (in units of slices); the smallest i whose flat
// index falls outside [0, rows) lands in *first_bad.
__global__ void flatten_indices_kernel(const int32_t* indices, int64_t* flat, int64_t n,
                                       SliceStrides s, int64_t rows, int* first_bad) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    int64_t f = 0;
    for (int j = 0; j < s.rank; j++) f += (int64_t)indices[i * s.rank + j] * s.stride[j];
    flat[i] = f;
    if (f < 0 || f >= rows) atomicMin(first_bad, (int)(i < INT_MAX ? i : INT_MAX - 1));
  }
}

template <typename T>
__global__ void gather_rows_kernel(const T* x, const int64_t* flat, T* out, int64_t n_slices,
                                   int64_t slice) {
  const int64_t total = n_slices * slice;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
    const int64_t i = g / slice, k = g - i * slice;
    out[g] = x[flat[i] * slice + k];
  }
}

// The same copy in 16-byte pieces, for slices that are a whole number of them.
__global__ void gather_rows_vec_kernel(const uint4* x, const int64_t* flat, uint4* out, int64_t n_slices,
                                       int64_t slice16) {
  const int64_t total = n_slices * slice16;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
    const int64_t i = g / slice16, k = g - i * slice16;
    out[g] = x[flat[i] * slice16 + k];
  }
}

// One lane per result element (row, k): starts from the default value and walks the updates
// in ascending order, adding (scatterND) or overwriting (sparseToDense: the last one wins)
// whenever an update addresses its row, which is the order backend_cpu.ts:3858-3886 applies
// them in.  Acc = T rounds every sum to the element type as a typed array does; Acc = double
// rounds once at the end, as the masked sums of unsortedSegmentSum do.
template <typename T, typename Acc>
__global__ __launch_bounds__(256) void scatter_rows_kernel(const int64_t* flat, const T* updates, T* out,
                                                           int64_t rows, int64_t slice, int64_t n_updates,
                                                           T start, int sum_dupes, int scalar_update) {
  // the index list passes through LDS 256 entries at a time: every lane of the workgroup walks
  // the same entries, which LDS serves as broadcasts
  __shared__ int chunk[256];  // row of each update, -2 for none (rows fit an int: checked by the host)
  const int64_t total = rows * slice;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  // all lanes of a workgroup make the same number of trips, so the barriers below are uniform
  for (int64_t base = (int64_t)blockIdx.x * blockDim.x; base < total; base += stride) {
    const int64_t g = base + threadIdx.x;
    const bool live = g < total;
    const int row = live ? (int)(g / slice) : -1;
    const int64_t k = live ? g - (int64_t)row * slice : 0;
    Acc acc = start;
    for (int64_t i0 = 0; i0 < n_updates; i0 += 256) {
      __syncthreads();
      const int64_t f = i0 + threadIdx.x < n_updates ? flat[i0 + threadIdx.x] : -2;
      chunk[threadIdx.x] = f >= 0 && f < rows ? (int)f : -2;
      __syncthreads();
      // eight entries per trip, read together so that their LDS latencies overlap
      for (int j0 = 0; j0 < 256; j0 += 8) {
        int c[8];
#pragma unroll
        for (int e = 0; e < 8; e++) c[e] = chunk[j0 + e];
#pragma unroll
        for (int e = 0; e < 8; e++) {
          if (c[e] != row) continue;
          const T u = updates[scalar_update ? 0 : (i0 + j0 + e) * slice + k];
          acc = sum_dupes ? (Acc)(acc + u) : (Acc)u;
        }
      }
    }
    if (live) out[g] = (T)acc;
  }
}

// Source rows / columns of a resized pixel as the reference computes them, in double.
struct Lerp {
  int lo, hi;
  double w;  // weight of hi; 1 - w goes to lo
};
__device__ inline Lerp lerp_at(int r, double scale, int in_size) {
  const double f = r * scale;
  Lerp l;
  l.lo = (int)floor(f);
  l.hi = min((int)ceil(f), in_size - 1);
  l.w = f - l.lo;
  return l;
}
// The resized rows whose source rows can touch input row y: r * scale within (y - 1, y + 1),
// widened by one either side against rounding of the division.
__device__ inline void touching(int y, double scale, int out_size, int* lo, int* hi) {
  if (!(scale > 0.0)) {
    *lo = 0;
    *hi = out_size - 1;
    return;
  }
  const double a = floor((y - 1) / scale) - 1.0, b = ceil((y + 1) / scale) + 1.0;
  *lo = a < 0.0 ? 0 : (a > out_size - 1 ? out_size - 1 : (int)a);
  *hi = b > out_size - 1 ? out_size - 1 : (b < 0.0 ? 0 : (int)b);
}

// dx[b, y, x, d]: every dy pixel (r, c) spreads over its four source pixels with the bilinear
// weights; this lane collects what lands on (y, x), in ascending (r, c) and, within one
// pixel, in the order top-left, top-right, bottom-left, bottom-right (backend_cpu.ts:2967-3009).
// The running sum is a float32 that takes one double-precision add per contribution, like a
// Float32Array element.
__global__ void resize_bilinear_backprop_kernel(const float* dy, float* dx, int batch, int x_h,
                                                int x_w, int ch, int y_h, int y_w,
                                                double scale_h, double scale_w) {
  const int64_t n = (int64_t)batch * x_h * x_w * ch;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int d = (int)(i % ch);
    int64_t t = i / ch;
    const int x = (int)(t % x_w);
    t /= x_w;
    const int y = (int)(t % x_h);
    const int b = (int)(t / x_h);
    int r_lo, r_hi, c_lo, c_hi;
    touching(y, scale_h, y_h, &r_lo, &r_hi);
    touching(x, scale_w, y_w, &c_lo, &c_hi);
    float acc = 0.f;
    for (int r = r_lo; r <= r_hi; r++) {
      const Lerp lr = lerp_at(r, scale_h, x_h);
      const bool top = lr.lo == y, bottom = lr.hi == y;
      if (!top && !bottom) continue;
      for (int c = c_lo; c <= c_hi; c++) {
        const Lerp lc = lerp_at(c, scale_w, x_w);
        const bool left = lc.lo == x, right = lc.hi == x;
        if (!left && !right) continue;
        const double g = dy[(((int64_t)b * y_h + r) * y_w + c) * ch + d];
        if (top && left) acc = (float)((double)acc + g * ((1.0 - lr.w) * (1.0 - lc.w)));
        if (top && right) acc = (float)((double)acc + g * ((1.0 - lr.w) * lc.w));
        if (bottom && left) acc = (float)((double)acc + g * (lr.w * (1.0 - lc.w)));
        if (bottom && right) acc = (float)((double)acc + g * (lr.w * lc.w));
      }
    }
    dx[i] = acc;
  }
}

// dx[b, y, x, d] = sum of the dy pixels whose nearest source pixel is (y, x), added in
// ascending (row, column) in double and rounded once (backend_cpu.ts:3107-3160).  The
// reference searches a window around y / scale; the rows that can qualify lie within
// `touching`, and rows outside its window never qualify, so both visit the same pixels.
__global__ void resize_nearest_backprop_kernel(const float* dy, float* dx, int batch, int x_h,
                                               int x_w, int ch, int y_h, int y_w, double scale_h,
                                               double scale_w, int align_corners) {
  const int64_t n = (int64_t)batch * x_h * x_w * ch;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int d = (int)(i % ch);
    int64_t t = i / ch;
    const int x = (int)(t % x_w);
    t /= x_w;
    const int y = (int)(t % x_h);
    const int b = (int)(t / x_h);
    int r_lo, r_hi, c_lo, c_hi;
    touching(y, scale_h, y_h, &r_lo, &r_hi);
    touching(x, scale_w, y_w, &c_lo, &c_hi);
    double acc = 0.0;
    for (int r = r_lo; r <= r_hi; r++) {
      const double fr = r * scale_h;
      if (min(x_h - 1, (int)(align_corners ? floor(fr + 0.5) : floor(fr))) != y) continue;
      for (int c = c_lo; c <= c_hi; c++) {
        const double fc = c * scale_w;
        if (min(x_w - 1, (int)(align_corners ? floor(fc + 0.5) : floor(fc))) != x) continue;
        acc += dy[(((int64_t)b * y_h + r) * y_w + c) * ch + d];
      }
    }
    dx[i] = (float)acc;
  }
}

// One lane per element of the crops, channel fastest; coordinates in double from the
// float32 box corners, as backend_cpu.ts:3646-3753 computes them.  A box whose image index
// is outside the batch leaves zeros.
__global__ void crop_and_resize_kernel(const float* images, const float* boxes,
                                       const int32_t* box_index, float* out, int batch, int img_h,
                                       int img_w, int ch, int64_t n_boxes, int crop_h, int crop_w,
                                       int nearest, float extrapolation) {
  const int64_t n = n_boxes * crop_h * crop_w * ch;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int c = (int)(i % ch);
    int64_t t = i / ch;
    const int x = (int)(t % crop_w);
    t /= crop_w;
    const int y = (int)(t % crop_h);
    const int64_t b = t / crop_h;
    const double y1 = boxes[b * 4], x1 = boxes[b * 4 + 1], y2 = boxes[b * 4 + 2],
                 x2 = boxes[b * 4 + 3];
    const int img = box_index[b];
    if (img < 0 || img >= batch) {
      out[i] = 0.f;
      continue;
    }
    const double scale_h = crop_h > 1 ? (y2 - y1) * (img_h - 1) / (crop_h - 1) : 0.0;
    const double scale_w = crop_w > 1 ? (x2 - x1) * (img_w - 1) / (crop_w - 1) : 0.0;
    const double fy = crop_h > 1 ? y1 * (img_h - 1) + y * scale_h : 0.5 * (y1 + y2) * (img_h - 1);
    const double fx = crop_w > 1 ? x1 * (img_w - 1) + x * scale_w : 0.5 * (x1 + x2) * (img_w - 1);
    // NaN coordinates fail both comparisons in the reference and read outside the image
    // there; here they extrapolate
    if (!(fy >= 0.0 && fy <= img_h - 1) || !(fx >= 0.0 && fx <= img_w - 1)) {
      out[i] = extrapolation;
      continue;
    }
    const float* im = images + (int64_t)img * img_h * img_w * ch + c;
    if (nearest) {
      const int cy = (int)floor(fy + 0.5), cx = (int)floor(fx + 0.5);
      out[i] = im[((int64_t)cy * img_w + cx) * ch];
    } else {
      const int top = (int)floor(fy), bottom = (int)ceil(fy);
      const int left = (int)floor(fx), right = (int)ceil(fx);
      const double wy = fy - top, wx = fx - left;
      const double tl = im[((int64_t)top * img_w + left) * ch], tr = im[((int64_t)top * img_w + right) * ch];
      const double bl = im[((int64_t)bottom * img_w + left) * ch],
                   br = im[((int64_t)bottom * img_w + right) * ch];
      const double up = tl + (tr - tl) * wx, down = bl + (br - bl) * wx;
      out[i] = (float)(up + (down - up) * wy);
    }
  }
}

// Flat slice indices of `indices` [n, slice_rank] into a tensor of `shape` whose first
// slice_rank dimensions are indexed; fails with the reference's message when one of them is
// out of range (backend_cpu.ts:3796-3799, 3870-3873).  Waits for the device.
static int flatten_checked(tfhip_ctx* ctx, const char* op, const Buf* bi, const int32_t* shape,
                           int rank, int64_t n, int slice_rank, Temp* flat, int64_t* slice_out,
                           int64_t* rows_out, bool check = true) {
  if (check && ctx->capturing)
    return ctx->fail(TFHIP_EINVAL, "%s: checks its indices on the host, which a graph capture cannot do", op);
  if (rank < 0 || rank > MAX_SLICE_RANK || slice_rank < 0 || slice_rank > rank || n < 0)
    return ctx->fail(TFHIP_EINVAL, "%s: bad shape or index depth", op);
  if (bi->dtype != TFHIP_INT32) return ctx->fail(TFHIP_EINVAL, "%s: indices must be int32", op);
  if (bi->numel != n * slice_rank)
    return ctx->fail(TFHIP_EINVAL, "%s: indices do not hold %lld x %d values", op, (long long)n, slice_rank);
  SliceStrides s = {};
  s.rank = slice_rank;
  int64_t slice = 1, rows = 1;
  for (int d = rank - 1; d >= slice_rank; d--) slice *= shape[d];
  for (int d = slice_rank - 1; d >= 0; d--) {
    s.stride[d] = rows;
    rows *= shape[d];
  }
  *slice_out = slice;
  *rows_out = rows;
  if (n == 0) return TFHIP_OK;
  Temp flag(ctx);
  if (!flat->get((size_t)n * sizeof(int64_t)) || !flag.get(sizeof(int))) return TFHIP_EDEVICE;
  int* bad = static_cast<int*>(flag.ptr);
  tfhip::launch(ctx, set_int_kernel, dim3(1), dim3(1), 0, bad, INT_MAX);
  tfhip::launch(ctx, flatten_indices_kernel, dim3(blocks_for(ctx, n)), dim3(256), 0,
                     (const int32_t*)bi->ptr, (int64_t*)flat->ptr, n, s, rows, bad);
  TFHIP_LAUNCH_CHECK(ctx);
  if (!check) return TFHIP_OK;
  int first_bad = INT_MAX;
  TFHIP_HIP(ctx, hipMemcpyAsync(&first_bad, bad, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
  TFHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
  if (first_bad == INT_MAX) return TFHIP_OK;
  int32_t idx[MAX_SLICE_RANK] = {0};
  TFHIP_HIP(ctx, hipMemcpy(idx, (const int32_t*)bi->ptr + (int64_t)first_bad * slice_rank,
                           sizeof(int32_t) * slice_rank, hipMemcpyDeviceToHost));
  char index_text[160] = "", shape_text[160] = "";
  for (int j = 0, at = 0; j < slice_rank && at < 140; j++)
    at += snprintf(index_text + at, sizeof index_text - at, j ? ",%d" : "%d", idx[j]);
  for (int j = 0, at = 0; j < rank && at < 140; j++)
    at += snprintf(shape_text + at, sizeof shape_text - at, j ? ",%d" : "%d", shape[j]);
  return ctx->fail(TFHIP_EINVAL, "Invalid indices: %s does not index into %s", index_text, shape_text);
}

static int resize_backprop_check(tfhip_ctx* ctx, const char* op, const Buf* bdy, const Buf* bdx,
                                 int batch, int x_h, int x_w, int ch, int y_h, int y_w) {
  if (batch < 0 || x_h < 0 || x_w < 0 || ch < 0 || y_h < 0 || y_w < 0)
    return ctx->fail(TFHIP_EINVAL, "%s: bad geometry", op);
  if (bdy->numel != (int64_t)batch * y_h * y_w * ch || bdx->numel != (int64_t)batch * x_h * x_w * ch ||
      bdy->dtype != TFHIP_FLOAT32 || bdx->dtype != TFHIP_FLOAT32)
    return ctx->fail(TFHIP_EINVAL, "%s: float32 buffers of the shapes given are required", op);
  return TFHIP_OK;
}

}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_gather_nd(tfhip_ctx* ctx, int64_t x, int64_t indices, int64_t out,
                               const int32_t* x_shape, int rank, int64_t num_slices,
                               int slice_rank) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bi, indices);
  TFHIP_GET(ctx, bo, out);
  if (rank > 0 && !x_shape) return ctx->fail(TFHIP_EINVAL, "gatherND: shape missing");
  Temp flat(ctx);
  int64_t slice = 0, rows = 0;
  int rc;
  if ((rc = flatten_checked(ctx, "gatherND", bi, x_shape, rank, num_slices, slice_rank, &flat, &slice, &rows)))
    return rc;
  if (bx->numel != rows * slice || bo->numel != num_slices * slice)
    return ctx->fail(TFHIP_EINVAL, "gatherND: buffer sizes do not match the shapes given");
  if (bx->dtype == TFHIP_UINT8Q || dtype_size(bx->dtype) != dtype_size(bo->dtype))
    return ctx->fail(TFHIP_EINVAL, "gatherND: input and output element sizes differ");
  if (bo->numel == 0) return TFHIP_OK;
  const dim3 grid(blocks_for(ctx, bo->numel)), block(256);
  const int64_t slice_bytes = slice * (int64_t)dtype_size(bx->dtype);
  if (slice_bytes % 16 == 0 && reinterpret_cast<uintptr_t>(bx->ptr) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(bo->ptr) % 16 == 0)
    tfhip::launch(ctx, gather_rows_vec_kernel, dim3(blocks_for(ctx, num_slices * (slice_bytes / 16))), block, 0, (const uint4*)bx->ptr, (const int64_t*)flat.ptr, (uint4*)bo->ptr, num_slices,
                       slice_bytes / 16);
  else if (dtype_size(bx->dtype) == 4)
    tfhip::launch(ctx, gather_rows_kernel<int32_t>, grid, block, 0, (const int32_t*)bx->ptr,
                       (const int64_t*)flat.ptr, (int32_t*)bo->ptr, num_slices, slice);
  else
    tfhip::launch(ctx, gather_rows_kernel<uint8_t>, grid, block, 0, (const uint8_t*)bx->ptr,
                       (const int64_t*)flat.ptr, (uint8_t*)bo->ptr, num_slices, slice);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_scatter_nd(tfhip_ctx* ctx, int64_t indices, int64_t updates, int64_t out,
                                const int32_t* out_shape, int rank, int64_t num_updates,
                                int slice_rank, double default_value, int flags) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bi, indices);
  TFHIP_GET(ctx, bu, updates);
  TFHIP_GET(ctx, bo, out);
  if (rank > 0 && !out_shape) return ctx->fail(TFHIP_EINVAL, "scatterND: shape missing");
  if (flags & ~(TFHIP_SCATTER_SUM | TFHIP_SCATTER_SKIP_INVALID | TFHIP_SCATTER_WIDE_SUM))
    return ctx->fail(TFHIP_EINVAL, "scatterND: unknown flag");
  Temp flat(ctx);
  int64_t slice = 0, rows = 0;
  int rc;
  if ((rc = flatten_checked(ctx, "scatterND", bi, out_shape, rank, num_updates, slice_rank, &flat, &slice, &rows,
                            !(flags & TFHIP_SCATTER_SKIP_INVALID))))
    return rc;
  const bool scalar_update = bu->numel == 1 && num_updates * slice != 1;
  if (bo->numel != rows * slice || (!scalar_update && bu->numel != num_updates * slice))
    return ctx->fail(TFHIP_EINVAL, "scatterND: buffer sizes do not match the shapes given");
  if ((bo->dtype != TFHIP_FLOAT32 && bo->dtype != TFHIP_INT32) || bu->dtype != bo->dtype)
    return ctx->fail(TFHIP_EINVAL, "scatterND: updates and result must both be float32 or both int32");
  if (bo->numel == 0) return TFHIP_OK;
  if (rows > INT_MAX) return ctx->fail(TFHIP_ENOTSUP, "scatterND: more than 2^31 - 1 result slices");
  const dim3 grid(blocks_for(ctx, bo->numel)), block(256);
  const int sum = flags & TFHIP_SCATTER_SUM ? 1 : 0, one = scalar_update ? 1 : 0;
  const int64_t* fl = (const int64_t*)flat.ptr;
  if (bo->dtype == TFHIP_INT32)
    tfhip::launch(ctx, (scatter_rows_kernel<int32_t, int32_t>), grid, block, 0, fl,
                       (const int32_t*)bu->ptr, (int32_t*)bo->ptr, rows, slice, num_updates,
                       (int32_t)default_value, sum, one);
  else if (flags & TFHIP_SCATTER_WIDE_SUM)
    tfhip::launch(ctx, (scatter_rows_kernel<float, double>), grid, block, 0, fl,
                       (const float*)bu->ptr, (float*)bo->ptr, rows, slice, num_updates,
                       (float)default_value, sum, one);
  else
    tfhip::launch(ctx, (scatter_rows_kernel<float, float>), grid, block, 0, fl,
                       (const float*)bu->ptr, (float*)bo->ptr, rows, slice, num_updates,
                       (float)default_value, sum, one);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_resize_bilinear_backprop(tfhip_ctx* ctx, int64_t dy, int64_t dx, int batch,
                                              int x_h, int x_w, int channels, int y_h, int y_w,
                                              int align_corners) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bdy, dy);
  TFHIP_GET(ctx, bdx, dx);
  int rc;
  if ((rc = resize_backprop_check(ctx, "resizeBilinearBackprop", bdy, bdx, batch, x_h, x_w, channels, y_h, y_w)))
    return rc;
  if (bdx->numel == 0) return TFHIP_OK;
  // effective sizes and scales (backend_cpu.ts:2952-2963)
  const double eh_x = (align_corners && y_h > 1) ? x_h - 1 : x_h, ew_x = (align_corners && y_w > 1) ? x_w - 1 : x_w;
  const double eh_y = (align_corners && y_h > 1) ? y_h - 1 : y_h, ew_y = (align_corners && y_w > 1) ? y_w - 1 : y_w;
  if (bdy->numel == 0) return tfhip_fill(ctx, dx, 0.0);
  tfhip::launch(ctx, resize_bilinear_backprop_kernel, dim3(blocks_for(ctx, bdx->numel)), dim3(256), 0, (const float*)bdy->ptr, (float*)bdx->ptr, batch, x_h, x_w, channels,
                     y_h, y_w, eh_x / eh_y, ew_x / ew_y);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_resize_nearest_backprop(tfhip_ctx* ctx, int64_t dy, int64_t dx, int batch,
                                             int x_h, int x_w, int channels, int y_h, int y_w,
                                             int align_corners) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bdy, dy);
  TFHIP_GET(ctx, bdx, dx);
  int rc;
  if ((rc = resize_backprop_check(ctx, "resizeNearestNeighborBackprop", bdy, bdx, batch, x_h, x_w, channels, y_h,
                                  y_w)))
    return rc;
  if (bdx->numel == 0) return TFHIP_OK;
  if (bdy->numel == 0) return tfhip_fill(ctx, dx, 0.0);
  // effective sizes and scales (backend_cpu.ts:3083-3094)
  const double eh_x = (align_corners && y_h > 1) ? x_h - 1 : x_h, ew_x = (align_corners && y_w > 1) ? x_w - 1 : x_w;
  const double eh_y = (align_corners && y_h > 1) ? y_h - 1 : y_h, ew_y = (align_corners && y_w > 1) ? y_w - 1 : y_w;
  tfhip::launch(ctx, resize_nearest_backprop_kernel, dim3(blocks_for(ctx, bdx->numel)), dim3(256), 0, (const float*)bdy->ptr, (float*)bdx->ptr, batch, x_h, x_w, channels,
                     y_h, y_w, eh_x / eh_y, ew_x / ew_y, align_corners ? 1 : 0);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_crop_and_resize(tfhip_ctx* ctx, int64_t images, int64_t boxes,
                                     int64_t box_index, int64_t out, int batch, int image_h,
                                     int image_w, int channels, int64_t num_boxes, int crop_h,
                                     int crop_w, int method, float extrapolation_value) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bim, images);
  TFHIP_GET(ctx, bb, boxes);
  TFHIP_GET(ctx, bx, box_index);
  TFHIP_GET(ctx, bo, out);
  if (batch < 0 || image_h < 0 || image_w < 0 || channels < 0 || num_boxes < 0 || crop_h < 0 || crop_w < 0)
    return ctx->fail(TFHIP_EINVAL, "cropAndResize: bad geometry");
  if (method != TFHIP_RESIZE_BILINEAR && method != TFHIP_RESIZE_NEAREST)
    return ctx->fail(TFHIP_EINVAL, "cropAndResize: method must be bilinear or nearest");
  if (bim->numel != (int64_t)batch * image_h * image_w * channels || bb->numel != num_boxes * 4 ||
      bx->numel != num_boxes || bo->numel != num_boxes * crop_h * crop_w * channels)
    return ctx->fail(TFHIP_EINVAL, "cropAndResize: buffers do not match the shapes given");
  if (bb->dtype != TFHIP_FLOAT32 || bx->dtype != TFHIP_INT32 || bo->dtype != TFHIP_FLOAT32)
    return ctx->fail(TFHIP_EINVAL, "cropAndResize: boxes float32, box indices int32, result float32");
  if (bo->numel == 0) return TFHIP_OK;
  if (bim->numel == 0) return ctx->fail(TFHIP_EINVAL, "cropAndResize: empty image");
  Temp tx(ctx);
  const float* imf;
  int rc;
  if ((rc = as_f32(ctx, bim, &tx, &imf))) return rc;
  tfhip::launch(ctx, crop_and_resize_kernel, dim3(blocks_for(ctx, bo->numel)), dim3(256), 0,
                     imf, (const float*)bb->ptr, (const int32_t*)bx->ptr, (float*)bo->ptr, batch, image_h,
                     image_w, channels, num_boxes, crop_h, crop_w, method == TFHIP_RESIZE_NEAREST ? 1 : 0,
                     extrapolation_value);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}
