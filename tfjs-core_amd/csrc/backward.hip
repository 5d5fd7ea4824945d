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
#include <cstring>

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

typedef float f32x4 __attribute__((ext_vector_type(4)));

// out[kh][kw][c] = w[KH - 1 - kh][KW - 1 - kw][c] (channel multiplier 1).
__global__ void flip_depthwise_filter_kernel(const float* w, float* out, int KH, int KW, int C) {
  const int g = blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= KH * KW * C) return;
  const int c = g % C, t = g / C;
  const int kw = t % KW, kh = t / KW;
  out[g] = w[((KH - 1 - kh) * KW + (KW - 1 - kw)) * C + c];
}

// Fast variants for channel multiplier 1, C % 4 == 0 and 16-byte aligned buffers: a lane owns
// 4 consecutive channels (16-byte accesses) and sums in float in the same tap order.
// S = 1, 2: the forward stride, known at compile time (no integer division); S = 0: any.
template <int S>
__global__ __launch_bounds__(256) void depthwise_der_input_vec_kernel(
    const float* __restrict__ dy, const float* __restrict__ w, float* __restrict__ dx,
    const tfhip_conv2d_info ci) {
  const int c4 = ci.in_c / 4;
  const int64_t total = (int64_t)ci.batch * ci.in_h * ci.in_w * c4;
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= total) return;
  const int cq = (int)(g % c4);
  int64_t t = g / c4;
  const int xc = (int)(t % ci.in_w);
  t /= ci.in_w;
  const int xr = (int)(t % ci.in_h);
  const int n = (int)(t / ci.in_h);
  const int sh = S ? S : ci.stride_h, sw = S ? S : ci.stride_w;
  const int xr_corner = xr - (ci.filter_h - 1 - ci.pad_top);
  const int xc_corner = xc - (ci.filter_w - 1 - ci.pad_left);
  const float* dyn = dy + (int64_t)n * ci.out_h * ci.out_w * ci.out_c + cq * 4;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int wr = 0; wr < ci.filter_h; wr++) {
    const int num_r = xr_corner + wr;
    const int yr = num_r / sh;
    if (num_r < 0 || yr * sh != num_r || yr >= ci.out_h) continue;
    for (int wc = 0; wc < ci.filter_w; wc++) {
      const int num_c = xc_corner + wc;
      const int yc = num_c / sw;
      if (num_c < 0 || yc * sw != num_c || yc >= ci.out_w) continue;
      const f32x4 d = *reinterpret_cast<const f32x4*>(dyn + ((int64_t)yr * ci.out_w + yc) * ci.out_c);
      const f32x4 f = *reinterpret_cast<const f32x4*>(
          w + ((int64_t)(ci.filter_h - 1 - wr) * ci.filter_w + (ci.filter_w - 1 - wc)) * ci.in_c + cq * 4);
      acc += d * f;
    }
  }
  *reinterpret_cast<f32x4*>(dx + g * 4) = acc;
}

// dW of a 3x3 depthwise filter (multiplier 1): one pass over the output pixels of a slice;
// a lane owns a channel quad and keeps the nine taps' sums, so dy is read once and the nine
// x vectors of a pixel come from neighbouring rows that stay in cache.  The lanes of a
// workgroup that share a quad (several pixels per wavefront when C / 4 < 64, and the four
// wavefronts) are then added in a fixed order through LDS.  partial[slice][tap][c] in double.
__global__ __launch_bounds__(256) void depthwise3x3_der_filter_partial_kernel(
    const float* __restrict__ x, const float* __restrict__ dy, double* __restrict__ partial,
    const tfhip_conv2d_info ci, int quads_per_wave, int64_t pixels_per_slice) {
  extern __shared__ __attribute__((aligned(16))) float red[];  // [256 lanes][9 taps][4]
  const int tid = threadIdx.x;
  const int c4 = ci.in_c / 4;
  const int q_local = tid % quads_per_wave;            // quad within the channel block
  const int sub = tid / quads_per_wave;                // which of the workgroup's pixel lanes
  const int subs = 256 / quads_per_wave;
  const int cq = blockIdx.x * quads_per_wave + q_local;
  const bool live = cq < c4;
  const int64_t pixels = (int64_t)ci.batch * ci.out_h * ci.out_w;
  const int64_t p0 = (int64_t)blockIdx.y * pixels_per_slice;
  const int64_t p1 = p0 + pixels_per_slice < pixels ? p0 + pixels_per_slice : pixels;
  f32x4 acc[9];
#pragma unroll
  for (int k = 0; k < 9; k++) acc[k] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (live) {
    for (int64_t px = p0 + sub; px < p1; px += subs) {
      const int yc = (int)(px % ci.out_w);
      const int64_t t = px / ci.out_w;
      const int yr = (int)(t % ci.out_h);
      const int n = (int)(t / ci.out_h);
      const f32x4 d = *reinterpret_cast<const f32x4*>(dy + px * ci.out_c + cq * 4);
      const int xr0 = yr * ci.stride_h - ci.pad_top, xc0 = yc * ci.stride_w - ci.pad_left;
      const float* xn = x + (int64_t)n * ci.in_h * ci.in_w * ci.in_c + cq * 4;
#pragma unroll
      for (int wr = 0; wr < 3; wr++) {
        const int xr = xr0 + wr;
#pragma unroll
        for (int wc = 0; wc < 3; wc++) {
          const int xc = xc0 + wc;
          f32x4 v = {0.f, 0.f, 0.f, 0.f};
          if ((unsigned)xr < (unsigned)ci.in_h && (unsigned)xc < (unsigned)ci.in_w)
            v = *reinterpret_cast<const f32x4*>(xn + ((int64_t)xr * ci.in_w + xc) * ci.in_c);
          acc[wr * 3 + wc] += v * d;
        }
      }
    }
  }
#pragma unroll
  for (int k = 0; k < 9; k++) *reinterpret_cast<f32x4*>(red + (tid * 9 + k) * 4) = acc[k];
  __syncthreads();
  // thread -> (tap, quad): add the `subs` lanes of that quad in ascending order, in double
  for (int item = tid; item < 9 * quads_per_wave; item += 256) {
    const int k = item / quads_per_wave, q = item % quads_per_wave;
    const int c = (blockIdx.x * quads_per_wave + q) * 4;
    if (c >= ci.in_c) continue;
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    for (int r = 0; r < subs; r++) {
      const float* v = red + ((r * quads_per_wave + q) * 9 + k) * 4;
      s0 += (double)v[0];
      s1 += (double)v[1];
      s2 += (double)v[2];
      s3 += (double)v[3];
    }
    double* out = partial + ((int64_t)blockIdx.y * 9 + k) * ci.in_c + c;
    out[0] = s0;
    out[1] = s1;
    out[2] = s2;
    out[3] = s3;
  }
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

// The same with a lane owning 4 consecutive channels (C % 4 == 0, 16-byte aligned buffers):
// the window scan and the dy gather are 16-byte accesses, the winner is tracked per channel.
__global__ __launch_bounds__(256) void pool2d_backprop_vec_kernel(
    const float* __restrict__ dy, const float* __restrict__ x, float* __restrict__ dx,
    const tfhip_conv2d_info ci, int kind) {
  const int eff_h = ci.filter_h + (ci.filter_h - 1) * (ci.dilation_h - 1);
  const int eff_w = ci.filter_w + (ci.filter_w - 1) * (ci.dilation_w - 1);
  const int pad_top = eff_h - 1 - ci.pad_top, pad_left = eff_w - 1 - ci.pad_left;
  const int c4 = ci.in_c / 4;
  const int64_t total = (int64_t)ci.batch * ci.in_h * ci.in_w * c4;
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= total) return;
  const int cq = (int)(g % c4);
  int64_t t = g / c4;
  const int xc = (int)(t % ci.in_w);
  t /= ci.in_w;
  const int xr = (int)(t % ci.in_h);
  const int n = (int)(t / ci.in_h);
  const float* xn = x + (int64_t)n * ci.in_h * ci.in_w * ci.in_c + cq * 4;
  const float* dyn = dy + (int64_t)n * ci.out_h * ci.out_w * ci.out_c + cq * 4;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int wr = 0; wr < eff_h; wr += ci.dilation_h) {
    const int num_r = xr - pad_top + wr;
    const int yr = num_r / ci.stride_h;
    if (num_r < 0 || yr * ci.stride_h != num_r || yr >= ci.out_h) continue;
    for (int wc = 0; wc < eff_w; wc += ci.dilation_w) {
      const int num_c = xc - pad_left + wc;
      const int yc = num_c / ci.stride_w;
      if (num_c < 0 || yc * ci.stride_w != num_c || yc >= ci.out_w) continue;
      const f32x4 d = *reinterpret_cast<const f32x4*>(dyn + ((int64_t)yr * ci.out_w + yc) * ci.out_c);
      if (kind != TFHIP_POOL_MAX) {
        acc += d;
        continue;
      }
      // first strict maximum of window (yr, yc), per channel; this pixel sits at the
      // flipped position (eff_h - 1 - wr, eff_w - 1 - wc) of that window
      const int xr0 = yr * ci.stride_h - ci.pad_top, xc0 = yc * ci.stride_w - ci.pad_left;
      f32x4 best = {-__builtin_inff(), -__builtin_inff(), -__builtin_inff(), -__builtin_inff()};
      int pos[4] = {-1, -1, -1, -1};
      for (int fr = 0; fr < eff_h; fr += ci.dilation_h) {
        const int r = xr0 + fr;
        if ((unsigned)r >= (unsigned)ci.in_h) continue;
        for (int fc = 0; fc < eff_w; fc += ci.dilation_w) {
          const int c = xc0 + fc;
          if ((unsigned)c >= (unsigned)ci.in_w) continue;
          const f32x4 v = *reinterpret_cast<const f32x4*>(xn + ((int64_t)r * ci.in_w + c) * ci.in_c);
#pragma unroll
          for (int e = 0; e < 4; e++)
            if (v[e] > best[e]) {
              best[e] = v[e];
              pos[e] = fr * eff_w + fc;
            }
        }
      }
      const int mine = (eff_h - 1 - wr) * eff_w + (eff_w - 1 - wc);
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (pos[e] == mine) acc[e] += d[e];
    }
  }
  if (kind != TFHIP_POOL_MAX) acc *= 1.0f / (float)(ci.filter_h * ci.filter_w);
  *reinterpret_cast<f32x4*>(dx + g * 4) = acc;
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

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

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
  float* dxf = static_cast<float*>(bdx->ptr);
  if (ch_mul == 1 && ci->stride_h == 1 && ci->stride_w == 1 && y_n > 0) {
    // stride 1: dx is the depthwise convolution of dy with the filter flipped in both spatial
    // directions and the padding filter - 1 - pad: the forward kernels do it at their speed
    Temp tflip(ctx);
    if (!tflip.get((size_t)w_n * sizeof(float))) return TFHIP_EDEVICE;
    tfhip::launch(ctx, flip_depthwise_filter_kernel, dim3((unsigned)ceil_div(w_n, 256)), dim3(256), 0, wf, static_cast<float*>(tflip.ptr), ci->filter_h, ci->filter_w,
                       ci->in_c);
    TFHIP_LAUNCH_CHECK(ctx);
    tfhip_conv2d_info back = *ci;
    back.in_h = ci->out_h; back.in_w = ci->out_w;
    back.out_h = ci->in_h; back.out_w = ci->in_w;
    back.out_c = ci->in_c;
    back.pad_top = ci->filter_h - 1 - ci->pad_top;
    back.pad_left = ci->filter_w - 1 - ci->pad_left;
    back.pad_bottom = back.pad_right = 0;   // (not read by the kernels)
    if ((rc = depthwise_forward_f32(ctx, dyf, static_cast<const float*>(tflip.ptr), dxf, &back))) return rc;
    strncat(ctx->last_kernel, "_as_der_input", sizeof ctx->last_kernel - strlen(ctx->last_kernel) - 1);
    return TFHIP_OK;
  }
  if (ch_mul == 1 && ci->in_c % 4 == 0 && aligned16(dyf) && aligned16(wf) && aligned16(dxf)) {
    const unsigned blocks = (unsigned)ceil_div(x_n / 4, 256);
    const int s = ci->stride_h == ci->stride_w && ci->stride_h <= 2 ? ci->stride_h : 0;
    ctx->name_kernel("depthwise_der_input_vec_s%d", s);
    if (s == 1)
      tfhip::launch(ctx, depthwise_der_input_vec_kernel<1>, dim3(blocks), dim3(256), 0,
                         dyf, wf, dxf, *ci);
    else if (s == 2)
      tfhip::launch(ctx, depthwise_der_input_vec_kernel<2>, dim3(blocks), dim3(256), 0,
                         dyf, wf, dxf, *ci);
    else
      tfhip::launch(ctx, depthwise_der_input_vec_kernel<0>, dim3(blocks), dim3(256), 0,
                         dyf, wf, dxf, *ci);
    TFHIP_LAUNCH_CHECK(ctx);
    return TFHIP_OK;
  }
  ctx->name_kernel("depthwise_der_input");
  tfhip::launch(ctx, depthwise_der_input_kernel, dim3(grid_for(ctx, x_n)), dim3(256), 0,
                     dyf, wf, dxf, *ci, ch_mul);
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
  const int64_t pixels = (int64_t)ci->batch * ci->out_h * ci->out_w;
  if (ch_mul == 1 && ci->filter_h == 3 && ci->filter_w == 3 && ci->in_c % 4 == 0 && aligned16(xf) &&
      aligned16(dyf) && pixels > 0) {
    const int c4 = ci->in_c / 4;
    int qpw = 1;                       // channel quads per workgroup: a power of two <= 64
    while (qpw < 64 && qpw < c4) qpw *= 2;
    const int64_t blocks_c = ceil_div(c4, qpw);
    const int subs = 256 / qpw;
    // two workgroups per CU, and at least 32 pixels per lane so that the reduction through
    // LDS and the partial sums stay a small part of the work
    int64_t slices = ceil_div((int64_t)ctx->num_cus * 2, blocks_c);
    if (slices > ceil_div(pixels, (int64_t)subs * 32)) slices = ceil_div(pixels, (int64_t)subs * 32);
    if (slices < 1) slices = 1;
    if (slices > 65535) slices = 65535;
    const int64_t per_slice = ceil_div(pixels, slices);
    if (!tpart.get((size_t)(slices * w_n) * sizeof(double))) return TFHIP_EDEVICE;
    ctx->name_kernel("depthwise3x3_der_filter");
    tfhip::launch(ctx, depthwise3x3_der_filter_partial_kernel, dim3((unsigned)blocks_c, (unsigned)slices),
                       dim3(256), (size_t)(256 * 9 * 4 * sizeof(float)), xf, dyf,
                       static_cast<double*>(tpart.ptr), *ci, qpw, per_slice);
    TFHIP_LAUNCH_CHECK(ctx);
    tfhip::launch(ctx, depthwise_der_filter_finish_kernel, dim3((unsigned)ceil_div(w_n, 256)), dim3(256),
                       0, static_cast<const double*>(tpart.ptr),
                       static_cast<float*>(bdw->ptr), w_n, (int)slices);
    TFHIP_LAUNCH_CHECK(ctx);
    return TFHIP_OK;
  }
  // enough pixel slices to fill the machine, at least 64 pixels each
  const int64_t channel_blocks = ceil_div(ci->out_c, 64);
  int64_t slices = ceil_div((int64_t)ctx->num_cus * 8, channel_blocks * taps);
  if (slices > ceil_div(pixels, 64)) slices = ceil_div(pixels, 64);
  if (slices < 1) slices = 1;
  if (slices > 65535) slices = 65535;
  const int64_t per_slice = ceil_div(pixels > 0 ? pixels : 1, slices);
  if (!tpart.get((size_t)(slices * w_n) * sizeof(double))) return TFHIP_EDEVICE;
  ctx->name_kernel("depthwise_der_filter");
  tfhip::launch(ctx, depthwise_der_filter_partial_kernel,
                     dim3((unsigned)channel_blocks, (unsigned)taps, (unsigned)slices), dim3(256), 0, xf, dyf, static_cast<double*>(tpart.ptr), *ci, ch_mul, per_slice);
  TFHIP_LAUNCH_CHECK(ctx);
  tfhip::launch(ctx, depthwise_der_filter_finish_kernel, dim3((unsigned)ceil_div(w_n, 256)), dim3(256),
                     0, static_cast<const double*>(tpart.ptr),
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
  float* dxf = static_cast<float*>(bdx->ptr);
  if (ci->in_c % 4 == 0 && aligned16(dyf) && aligned16(xf) && aligned16(dxf)) {
    ctx->name_kernel(
             kind == TFHIP_POOL_MAX ? "max_pool_backprop_vec" : "avg_pool_backprop_vec");
    tfhip::launch(ctx, pool2d_backprop_vec_kernel, dim3((unsigned)ceil_div(x_n / 4, 256)), dim3(256), 0, dyf, xf, dxf, *ci, kind);
    TFHIP_LAUNCH_CHECK(ctx);
    return TFHIP_OK;
  }
  ctx->name_kernel(
           kind == TFHIP_POOL_MAX ? "max_pool_backprop" : "avg_pool_backprop");
  tfhip::launch(ctx, pool2d_backprop_kernel, dim3(grid_for(ctx, x_n)), dim3(256), 0, dyf,
                     xf, static_cast<float*>(bdx->ptr), *ci, kind);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}
