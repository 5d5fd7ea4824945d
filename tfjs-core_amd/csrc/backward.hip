// Memory-bound backward kernels of the NHWC image ops: depthwiseConv2DDerInput /
// depthwiseConv2DDerFilter (backend_cpu.ts:2037-2150 of the reference) and maxPoolBackprop /
// avgPoolBackprop (:2347-2509).  (conv2dDerInput / conv2dDerFilter are products and live
// with the dense kernels.)
//
// The gradients with respect to an image are gathers: one lane per dx element, output
// channel fastest, so a wavefront reads runs of consecutive dy elements.  The gradient with
// respect to the depthwise filter is a reduction over every output pixel: lanes run along
// the channels, workgroups split the pixels, and a second kernel adds the partial sums in a
// fixed order, so the result does not depend on scheduling.
#include "tfhip_internal.h"

namespace tfhip {

// dx[n, xr, xc, d1] = sum over the output pixels (yr, yc) whose window covers (xr, xc), and
// over the channel multiplier, of dy * w; taps in the order of the reference's loops (output
// row, output column, multiplier).  Accumulated in double, stored once, like the reference.
__global__ void depthwise_der_input_kernel(const float* dy, const float* w, float* dx,
                                           const tfhip_conv2d_info ci, int ch_mul) {
  const int64_t total = (int64_t)ci.batch * ci.in_h * ci.in_w * ci.in_c;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int top_pad = ci.filter_h - 1 - ci.pad_top, left_pad = ci.filter_w - 1 - ci.pad_left;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
    const int d1 = (int)(g % ci.in_c);
    int64_t t = g / ci.in_c;
    const int xc = (int)(t % ci.in_w);
    t /= ci.in_w;
    const int xr = (int)(t % ci.in_h);
    const int n = (int)(t / ci.in_h);
    const int xr_corner = xr - top_pad, xc_corner = xc - left_pad;
    double dot = 0.0;
    for (int wr = 0; wr < ci.filter_h; wr++) {
      const int num_r = xr_corner + wr;  // = yr * stride_h
      if (num_r < 0 || num_r % ci.stride_h != 0) continue;
      const int yr = num_r / ci.stride_h;
      if (yr >= ci.out_h) continue;
      for (int wc = 0; wc < ci.filter_w; wc++) {
        const int num_c = xc_corner + wc;
        if (num_c < 0 || num_c % ci.stride_w != 0) continue;
        const int yc = num_c / ci.stride_w;
        if (yc >= ci.out_w) continue;
        const float* dyp =
            dy + (((int64_t)n * ci.out_h + yr) * ci.out_w + yc) * ci.out_c + (int64_t)d1 * ch_mul;
        const float* wp = w + (((int64_t)(ci.filter_h - 1 - wr) * ci.filter_w +
                                (ci.filter_w - 1 - wc)) * ci.in_c + d1) * ch_mul;
        for (int dm = 0; dm < ch_mul; dm++) dot += (double)dyp[dm] * (double)wp[dm];
      }
    }
    dx[g] = (float)dot;
  }
}

// Partial sums of dW over a slice of the output pixels.  grid = (channel blocks of 64,
// filter taps, pixel slices); a workgroup's 4 wavefronts take every 4th pixel of the slice,
// lane = output channel d2 (so dy, and for multiplier 1 also x, are read in 256-byte runs).
// partial[slice][tap][d2] in double.
__global__ __launch_bounds__(256) void depthwise_der_filter_partial_kernel(
    const float* x, const float* dy, double* partial, const tfhip_conv2d_info ci, int ch_mul,
    int64_t pixels_per_slice) {
  __shared__ double red[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int d2 = blockIdx.x * 64 + lane;
  const int tap = blockIdx.y, wr = tap / ci.filter_w, wc = tap % ci.filter_w;
  const int64_t pixels = (int64_t)ci.batch * ci.out_h * ci.out_w;
  const int64_t p0 = (int64_t)blockIdx.z * pixels_per_slice;
  const int64_t p1 = p0 + pixels_per_slice < pixels ? p0 + pixels_per_slice : pixels;
  const bool live = d2 < ci.out_c;
  const int d1 = live ? d2 / ch_mul : 0;
  double dot = 0.0;
  for (int64_t px = p0 + wave; px < p1; px += 4) {
    const int yc = (int)(px % ci.out_w);
    const int64_t t = px / ci.out_w;
    const int yr = (int)(t % ci.out_h);
    const int n = (int)(t / ci.out_h);
    const int xr = wr + yr * ci.stride_h - ci.pad_top, xc = wc + yc * ci.stride_w - ci.pad_left;
    if ((unsigned)xr >= (unsigned)ci.in_h || (unsigned)xc >= (unsigned)ci.in_w || !live) continue;
    dot += (double)x[(((int64_t)n * ci.in_h + xr) * ci.in_w + xc) * ci.in_c + d1] *
           (double)dy[px * ci.out_c + d2];
  }
  red[wave][lane] = dot;
  __syncthreads();
  if (wave == 0 && live)
    partial[((int64_t)blockIdx.z * gridDim.y + tap) * ci.out_c + d2] =
        ((red[0][lane] + red[1][lane]) + red[2][lane]) + red[3][lane];
}

// dW[tap][d1][dm] = sum of the slices' partial sums, ascending slice order.
__global__ void depthwise_der_filter_finish_kernel(const double* partial, float* dw, int64_t w_n,
                                                   int slices) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= w_n) return;
  double s = 0.0;
  for (int i = 0; i < slices; i++) s += partial[(int64_t)i * w_n + g];
  dw[g] = (float)s;
}

// Position (row-major over the dilated window) of the first strict maximum of the window of
// output pixel (yr, yc), as maxPoolPositions finds it; -1 when nothing is greater than -inf.
__device__ __forceinline__ int max_position(const float* x, const tfhip_conv2d_info& ci, int eff_h,
                                            int eff_w, int n, int yr, int yc, int d) {
  const int xr_corner = yr * ci.stride_h - ci.pad_top, xc_corner = yc * ci.stride_w - ci.pad_left;
  float best = -__builtin_inff();
  int pos = -1;
  for (int wr = 0; wr < eff_h; wr += ci.dilation_h) {
    const int xr = xr_corner + wr;
    if ((unsigned)xr >= (unsigned)ci.in_h) continue;
    for (int wc = 0; wc < eff_w; wc += ci.dilation_w) {
      const int xc = xc_corner + wc;
      if ((unsigned)xc >= (unsigned)ci.in_w) continue;
      const float v = x[(((int64_t)n * ci.in_h + xr) * ci.in_w + xc) * ci.in_c + d];
      if (v > best) {
        best = v;
        pos = wr * eff_w + wc;
      }
    }
  }
  return pos;
}

// One lane per dx element.  kind 1 (max): dy of every covering window whose first maximum is
// this pixel; kind 0 (avg): dy of every covering window times 1 / (filter_h * filter_w).
__global__ void pool2d_backprop_kernel(const float* dy, const float* x, float* dx,
                                       const tfhip_conv2d_info ci, int kind) {
  const int eff_h = ci.filter_h + (ci.filter_h - 1) * (ci.dilation_h - 1);
  const int eff_w = ci.filter_w + (ci.filter_w - 1) * (ci.dilation_w - 1);
  const int pad_top = eff_h - 1 - ci.pad_top, pad_left = eff_w - 1 - ci.pad_left;
  const double avg_multiplier = 1.0 / (double)(ci.filter_h * ci.filter_w);
  const int64_t total = (int64_t)ci.batch * ci.in_h * ci.in_w * ci.in_c;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
    const int d = (int)(g % ci.in_c);
    int64_t t = g / ci.in_c;
    const int xc = (int)(t % ci.in_w);
    t /= ci.in_w;
    const int xr = (int)(t % ci.in_h);
    const int n = (int)(t / ci.in_h);
    const int dyr_corner = xr - pad_top, dyc_corner = xc - pad_left;
    double dot = 0.0;
    for (int wr = 0; wr < eff_h; wr += ci.dilation_h) {
      const int num_r = dyr_corner + wr;
      if (num_r < 0 || num_r % ci.stride_h != 0) continue;
      const int yr = num_r / ci.stride_h;
      if (yr >= ci.out_h) continue;
      for (int wc = 0; wc < eff_w; wc += ci.dilation_w) {
        const int num_c = dyc_corner + wc;
        if (num_c < 0 || num_c % ci.stride_w != 0) continue;
        const int yc = num_c / ci.stride_w;
        if (yc >= ci.out_w) continue;
        if (kind == TFHIP_POOL_MAX) {
          const int max_pos = eff_h * eff_w - 1 - max_position(x, ci, eff_h, eff_w, n, yr, yc, d);
          if (max_pos != wr * eff_w + wc) continue;
        }
        dot += (double)dy[(((int64_t)n * ci.out_h + yr) * ci.out_w + yc) * ci.out_c + d];
      }
    }
    dx[g] = (float)(kind == TFHIP_POOL_MAX ? dot : dot * avg_multiplier);
  }
}

static int check_geometry(tfhip_ctx* ctx, const char* op, const tfhip_conv2d_info* ci,
                          bool dilation_allowed) {
  if (ci->batch < 0 || ci->in_h < 0 || ci->in_w < 0 || ci->in_c < 0 || ci->out_h < 0 ||
      ci->out_w < 0 || ci->out_c < 0 || ci->filter_h <= 0 || ci->filter_w <= 0 ||
      ci->stride_h <= 0 || ci->stride_w <= 0 || ci->dilation_h <= 0 || ci->dilation_w <= 0)
    return ctx->fail(TFHIP_EINVAL, "%s: bad geometry", op);
  if (!dilation_allowed && (ci->dilation_h != 1 || ci->dilation_w != 1))
    return ctx->fail(TFHIP_EINVAL, "%s: dilation rates greater than 1 are not yet supported", op);
  return TFHIP_OK;
}

static unsigned grid_for(tfhip_ctx* ctx, int64_t elements) {
  const int64_t blocks = ceil_div(elements, 256);
  const int64_t cap = (int64_t)ctx->num_cus * 16;
  return (unsigned)(blocks > cap ? cap : blocks);
}

}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_depthwise_conv2d_der_input(tfhip_ctx* ctx, int64_t dy, int64_t filter,
                                                int64_t dx, const tfhip_conv2d_info* ci) {
  if (!ctx || !ci) return TFHIP_EINVAL;
  int rc;
  if ((rc = check_geometry(ctx, "depthwiseConv2DDerInput", ci, false))) return rc;
  TFHIP_GET(ctx, bdy, dy);
  TFHIP_GET(ctx, bw, filter);
  TFHIP_GET(ctx, bdx, dx);
  if (ci->in_c <= 0 || ci->out_c % ci->in_c != 0)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2DDerInput: out channels must be a multiple of in channels");
  const int ch_mul = ci->out_c / ci->in_c;
  const int64_t x_n = (int64_t)ci->batch * ci->in_h * ci->in_w * ci->in_c;
  const int64_t w_n = (int64_t)ci->filter_h * ci->filter_w * ci->out_c;
  const int64_t y_n = (int64_t)ci->batch * ci->out_h * ci->out_w * ci->out_c;
  if (bdy->numel != y_n || bw->numel != w_n || bdx->numel != x_n)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2DDerInput: buffer sizes do not match the geometry");
  if (bdx->dtype != TFHIP_FLOAT32 || bw->dtype == TFHIP_UINT8Q)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2DDerInput: dx must be float32 and the filter not quantised");
  if (x_n == 0) return TFHIP_OK;
  Temp tdy(ctx), tw(ctx);
  const float *dyf, *wf;
  if ((rc = as_f32(ctx, bdy, &tdy, &dyf))) return rc;
  if ((rc = as_f32(ctx, bw, &tw, &wf))) return rc;
  snprintf(ctx->last_kernel, sizeof ctx->last_kernel, "depthwise_der_input");
  hipLaunchKernelGGL(depthwise_der_input_kernel, dim3(grid_for(ctx, x_n)), dim3(256), 0, ctx->stream,
                     dyf, wf, static_cast<float*>(bdx->ptr), *ci, ch_mul);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_depthwise_conv2d_der_filter(tfhip_ctx* ctx, int64_t x, int64_t dy, int64_t dw,
                                                 const tfhip_conv2d_info* ci) {
  if (!ctx || !ci) return TFHIP_EINVAL;
  int rc;
  if ((rc = check_geometry(ctx, "depthwiseConv2DDerFilter", ci, false))) return rc;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bdy, dy);
  TFHIP_GET(ctx, bdw, dw);
  if (ci->in_c <= 0 || ci->out_c % ci->in_c != 0)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2DDerFilter: out channels must be a multiple of in channels");
  const int ch_mul = ci->out_c / ci->in_c;
  const int64_t x_n = (int64_t)ci->batch * ci->in_h * ci->in_w * ci->in_c;
  const int64_t w_n = (int64_t)ci->filter_h * ci->filter_w * ci->out_c;
  const int64_t y_n = (int64_t)ci->batch * ci->out_h * ci->out_w * ci->out_c;
  if (bx->numel != x_n || bdy->numel != y_n || bdw->numel != w_n)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2DDerFilter: buffer sizes do not match the geometry");
  if (bdw->dtype != TFHIP_FLOAT32)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2DDerFilter: dW must be float32");
  if (w_n == 0) return TFHIP_OK;
  const int taps = ci->filter_h * ci->filter_w;
  if (taps > 65535) return ctx->fail(TFHIP_ENOTSUP, "depthwiseConv2DDerFilter: more than 65535 filter taps");
  Temp tx(ctx), tdy(ctx), tpart(ctx);
  const float *xf, *dyf;
  if ((rc = as_f32(ctx, bx, &tx, &xf))) return rc;
  if ((rc = as_f32(ctx, bdy, &tdy, &dyf))) return rc;
  // enough pixel slices to fill the machine, at least 64 pixels each
  const int64_t pixels = (int64_t)ci->batch * ci->out_h * ci->out_w;
  const int64_t channel_blocks = ceil_div(ci->out_c, 64);
  int64_t slices = ceil_div((int64_t)ctx->num_cus * 8, channel_blocks * taps);
  if (slices > ceil_div(pixels, 64)) slices = ceil_div(pixels, 64);
  if (slices < 1) slices = 1;
  if (slices > 65535) slices = 65535;
  const int64_t per_slice = ceil_div(pixels > 0 ? pixels : 1, slices);
  if (!tpart.get((size_t)(slices * w_n) * sizeof(double))) return TFHIP_EDEVICE;
  snprintf(ctx->last_kernel, sizeof ctx->last_kernel, "depthwise_der_filter");
  hipLaunchKernelGGL(depthwise_der_filter_partial_kernel,
                     dim3((unsigned)channel_blocks, (unsigned)taps, (unsigned)slices), dim3(256), 0,
                     ctx->stream, xf, dyf, static_cast<double*>(tpart.ptr), *ci, ch_mul, per_slice);
  TFHIP_LAUNCH_CHECK(ctx);
  hipLaunchKernelGGL(depthwise_der_filter_finish_kernel, dim3((unsigned)ceil_div(w_n, 256)), dim3(256),
                     0, ctx->stream, static_cast<const double*>(tpart.ptr),
                     static_cast<float*>(bdw->ptr), w_n, (int)slices);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_pool2d_backprop(tfhip_ctx* ctx, int64_t dy, int64_t x, int64_t dx,
                                     const tfhip_conv2d_info* ci, int kind) {
  if (!ctx || !ci) return TFHIP_EINVAL;
  int rc;
  if ((rc = check_geometry(ctx, "poolBackprop", ci, true))) return rc;
  if (kind != TFHIP_POOL_AVG && kind != TFHIP_POOL_MAX)
    return ctx->fail(TFHIP_EINVAL, "poolBackprop: unknown kind %d", kind);
  TFHIP_GET(ctx, bdy, dy);
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bdx, dx);
  if (ci->in_c != ci->out_c) return ctx->fail(TFHIP_EINVAL, "poolBackprop: channel counts differ");
  const int64_t x_n = (int64_t)ci->batch * ci->in_h * ci->in_w * ci->in_c;
  const int64_t y_n = (int64_t)ci->batch * ci->out_h * ci->out_w * ci->out_c;
  if (bdy->numel != y_n || bx->numel != x_n || bdx->numel != x_n)
    return ctx->fail(TFHIP_EINVAL, "poolBackprop: buffer sizes do not match the geometry");
  if (bdx->dtype != TFHIP_FLOAT32) return ctx->fail(TFHIP_EINVAL, "poolBackprop: dx must be float32");
  if (x_n == 0) return TFHIP_OK;
  Temp tdy(ctx), tx(ctx);
  const float *dyf, *xf;
  if ((rc = as_f32(ctx, bdy, &tdy, &dyf))) return rc;
  if ((rc = as_f32(ctx, bx, &tx, &xf))) return rc;
  snprintf(ctx->last_kernel, sizeof ctx->last_kernel,
           kind == TFHIP_POOL_MAX ? "max_pool_backprop" : "avg_pool_backprop");
  hipLaunchKernelGGL(pool2d_backprop_kernel, dim3(grid_for(ctx, x_n)), dim3(256), 0, ctx->stream, dyf,
                     xf, static_cast<float*>(bdx->ptr), *ci, kind);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}
