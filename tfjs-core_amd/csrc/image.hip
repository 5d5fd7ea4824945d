// Memory-bound NHWC image kernels: depthwiseConv2D (+ folded bias / relu / relu6) and
// avg / max pooling.  Replaces backend_cpu.ts:1979-2035 and :2273-2345 of the reference.
//
// Both stream the activation tensor through HBM once.  Lanes run along the channel axis
// (4 channels = 16 bytes per lane) so every wavefront access is a run of contiguous
// 16-byte pieces; the 3x3 kernel keeps a TH x TW patch of outputs per lane in registers so
// each input vector fetched is used by up to 9 multiply-adds without going back to L2.
#include <type_traits>

#include "tfhip_internal.h"

namespace tfhip {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float dq(unsigned q, double scale, double mn) {
#pragma clang fp contract(off)
  double v = (double)q * scale;
  v = v + mn;
  return (float)v;
}

__device__ __forceinline__ float act_f(float v, int act) {
  switch (act) {
    case TFHIP_ACT_RELU: return (v > 0.f || v != v) ? v : 0.f;
    case TFHIP_ACT_RELU6: return v > 6.f ? 6.f : (v < 0.f ? 0.f : v);
    default: return v;
  }
}

// The same activations as a clamp to [lo, hi] (linear: the whole line): IEEE 754-2019 maximum /
// minimum, which gfx950 has as v_maximum3_f32 / v_minimum3_f32, return NaN when an operand is NaN,
// so NaN passes through as it does through the reference's Math.max / Math.min.
struct ActFlags {
  float lo, hi;
};
__device__ __forceinline__ ActFlags act_flags(int act) {
  ActFlags f;
  f.lo = act == TFHIP_ACT_RELU || act == TFHIP_ACT_RELU6 ? 0.f : -__builtin_inff();
  f.hi = act == TFHIP_ACT_RELU6 ? 6.f : __builtin_inff();
  return f;
}
__device__ __forceinline__ float act_fast(float v, const ActFlags& f) {
  return __builtin_elementwise_minimum(__builtin_elementwise_maximum(v, f.lo), f.hi);
}

struct DwArgs {
  const float* x;
  const void* w;
  const float* bias;
  float* y;
  tfhip_conv2d_info ci;
  int ch_mul;
  int bias_kind, act;
  int quant;
  double qscale, qmin;
  int tiles_w, tiles_h, c4;  // fast path: patch grid and channel quads
  int reverse;               // fast path: walk the rows of every XCD's run from the end
};

// 3x3, dilation 1, channel multiplier 1, C % 4 == 0, stride S.  One lane = one channel
// quad of a TH x TW output patch.  Lane order: channel quad fastest, then patch column,
// patch row, image — neighbours in a wavefront touch neighbouring addresses.
template <int S, int TH, int TW>
__global__ __launch_bounds__(256) void depthwise3x3_kernel(const DwArgs p) {
  constexpr int IH = (TH - 1) * S + 3, IW = (TW - 1) * S + 3;
  __builtin_amdgcn_s_setprio(WAVE_PRIORITY_MEMORY_BOUND);
  const tfhip_conv2d_info& ci = p.ci;
  const int64_t total = (int64_t)ci.batch * p.tiles_h * p.tiles_w * p.c4;
  // contiguous image regions per XCD: the halo rows two patch rows share are then served
  // by that XCD's L2 instead of being fetched once per XCD
  const int64_t gid =
      (int64_t)xcd_remap_dir(blockIdx.x, gridDim.x, p.reverse) * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int cq = (int)(gid % p.c4);
  int64_t t = gid / p.c4;
  const int tw = (int)(t % p.tiles_w);
  t /= p.tiles_w;
  const int th = (int)(t % p.tiles_h);
  const int n = (int)(t / p.tiles_h);
  const int c = cq * 4;
  const int C = ci.in_c;

  f32x4 w[9];
  if (p.quant) {
    const unsigned char* wq = static_cast<const unsigned char*>(p.w);
#pragma unroll
    for (int i = 0; i < 9; i++) {
      const unsigned v = *reinterpret_cast<const unsigned*>(wq + (int64_t)i * C + c);
#pragma unroll
      for (int e = 0; e < 4; e++) w[i][e] = dq((v >> (8 * e)) & 0xffu, p.qscale, p.qmin);
    }
  } else {
    const float* wf = static_cast<const float*>(p.w);
#pragma unroll
    for (int i = 0; i < 9; i++) w[i] = *reinterpret_cast<const f32x4*>(wf + (int64_t)i * C + c);
  }

  const int oh0 = th * TH, ow0 = tw * TW;
  const int ih0 = oh0 * S - ci.pad_top, iw0 = ow0 * S - ci.pad_left;
  const float* xn = p.x + (int64_t)n * ci.in_h * ci.in_w * C + c;

  f32x4 acc[TH][TW];
#pragma unroll
  for (int i = 0; i < TH; i++)
#pragma unroll
    for (int j = 0; j < TW; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Accumulation order per output is filter row, then filter column (as the reference's
  // loops, backend_cpu.ts:1996-2030), because input rows are visited in ascending order.
#pragma unroll
  for (int r = 0; r < IH; r++) {
    const int ih = ih0 + r;
    const bool row_ok = (unsigned)ih < (unsigned)ci.in_h;
    f32x4 in[IW];
#pragma unroll
    for (int q = 0; q < IW; q++) {
      const int iw = iw0 + q;
      in[q] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (row_ok && (unsigned)iw < (unsigned)ci.in_w)
        in[q] = *reinterpret_cast<const f32x4*>(xn + ((int64_t)ih * ci.in_w + iw) * C);
    }
#pragma unroll
    for (int i = 0; i < TH; i++) {
      const int kh = r - i * S;
      if (kh < 0 || kh > 2) continue;
#pragma unroll
      for (int j = 0; j < TW; j++)
#pragma unroll
        for (int kw = 0; kw < 3; kw++) acc[i][j] += in[j * S + kw] * w[kh * 3 + kw];
    }
  }

  const ActFlags af = act_flags(p.act);
  f32x4 b = {0.f, 0.f, 0.f, 0.f};
  if (p.bias_kind == TFHIP_BCAST_COLUMN) b = *reinterpret_cast<const f32x4*>(p.bias + c);
  else if (p.bias_kind == TFHIP_BCAST_SCALAR) b = f32x4{p.bias[0], p.bias[0], p.bias[0], p.bias[0]};
#pragma unroll
  for (int i = 0; i < TH; i++) {
    const int oh = oh0 + i;
    if (oh >= ci.out_h) continue;
#pragma unroll
    for (int j = 0; j < TW; j++) {
      const int ow = ow0 + j;
      if (ow >= ci.out_w) continue;
      f32x4 v = acc[i][j] + b;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = act_fast(v[e], af);
      *reinterpret_cast<f32x4*>(p.y + (((int64_t)n * ci.out_h + oh) * ci.out_w + ow) * C + c) = v;
    }
  }
}

// 3x3, stride 1, dilation 1, channel multiplier 1, C % 4 == 0, for large images: one lane =
// one channel quad of a strip TW outputs wide, walked down `rows` output rows.  Every input
// row of the strip is fetched once (TW + 2 vectors, the next PF rows already in flight) and
// feeds the three output rows it belongs to, which live in three rotating accumulator rows;
// nothing is read twice vertically, and the two halo columns are shared with the
// neighbouring lane's loads of the same moment.  Each output sums its taps in the order
// filter row, then filter column, as the patch kernel above and the reference do.
template <int TW, int PF>
__global__ __launch_bounds__(256) void depthwise3x3_rows_kernel(const DwArgs p, int rows,
                                                                int chunks, unsigned x_bytes,
                                                                unsigned y_bytes) {
  __builtin_amdgcn_s_setprio(WAVE_PRIORITY_MEMORY_BOUND);
  constexpr int IW = TW + 2;
  constexpr int NB = PF + 1;                       // row buffers: PF rows in flight + the one in use
  constexpr int PERIOD = NB % 3 == 0 ? NB : 3 * NB;  // buffers and accumulator rows take turns
  constexpr unsigned OOB = 0x80000000u;  // beyond any extent below 2 GiB: loads give 0, stores vanish
  const tfhip_conv2d_info& ci = p.ci;
  const int64_t total = (int64_t)ci.batch * chunks * p.tiles_w * p.c4;
  const int64_t gid =
      (int64_t)xcd_remap_dir(blockIdx.x, gridDim.x, p.reverse) * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int cq = (int)(gid % p.c4);
  int64_t t = gid / p.c4;
  const int tw = (int)(t % p.tiles_w);
  t /= p.tiles_w;
  const int chunk = (int)(t % chunks);
  const int n = (int)(t / chunks);
  const int c = cq * 4;
  const int C = ci.in_c;

  f32x4 w[9];
  if (p.quant) {
    const unsigned char* wq = static_cast<const unsigned char*>(p.w);
#pragma unroll
    for (int i = 0; i < 9; i++) {
      const unsigned v = *reinterpret_cast<const unsigned*>(wq + (int64_t)i * C + c);
#pragma unroll
      for (int e = 0; e < 4; e++) w[i][e] = dq((v >> (8 * e)) & 0xffu, p.qscale, p.qmin);
    }
  } else {
    const float* wf = static_cast<const float*>(p.w);
#pragma unroll
    for (int i = 0; i < 9; i++) w[i] = *reinterpret_cast<const f32x4*>(wf + (int64_t)i * C + c);
  }
  f32x4 b = {0.f, 0.f, 0.f, 0.f};
  if (p.bias_kind == TFHIP_BCAST_COLUMN) b = *reinterpret_cast<const f32x4*>(p.bias + c);
  else if (p.bias_kind == TFHIP_BCAST_SCALAR) b = f32x4{p.bias[0], p.bias[0], p.bias[0], p.bias[0]};

  // All addresses are 32-bit byte offsets into buffer descriptors over x and y: padding,
  // rows outside the chunk and columns outside the image get OOB instead of a branch.
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(p.x), (short)0, (int)x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ry =
      __builtin_amdgcn_make_buffer_rsrc(p.y, (short)0, (int)y_bytes, 0x00020000);
  const ActFlags af = act_flags(p.act);
  const int oh0 = chunk * rows;
  const int oh1 = min(ci.out_h, oh0 + rows);
  const int ow0 = tw * TW;
  const int iw0 = ow0 - ci.pad_left;
  const unsigned x_img = ((unsigned)n * ci.in_h * ci.in_w * C + c) * 4u;
  const unsigned y_img = ((unsigned)n * ci.out_h * ci.out_w * C + c) * 4u;
  const unsigned x_row = (unsigned)ci.in_w * C * 4u, y_row = (unsigned)ci.out_w * C * 4u;
  unsigned col_in[IW], col_out[TW];
#pragma unroll
  for (int q = 0; q < IW; q++)
    col_in[q] = (unsigned)(iw0 + q) < (unsigned)ci.in_w ? x_img + (unsigned)(iw0 + q) * C * 4u : OOB;
#pragma unroll
  for (int j = 0; j < TW; j++)
    col_out[j] = ow0 + j < ci.out_w ? y_img + (unsigned)(ow0 + j) * C * 4u : OOB;
  const int ih_first = oh0 - ci.pad_top;         // filter row 0 of output row oh0
  const int ih_last = oh1 - 1 - ci.pad_top + 2;  // filter row 2 of output row oh1 - 1

  auto load_row = [&](int ih, f32x4 (&in)[IW]) {
    const bool row_ok = (unsigned)ih < (unsigned)ci.in_h && ih <= ih_last;
    const unsigned at = (unsigned)ih * x_row;
#pragma unroll
    for (int q = 0; q < IW; q++)
      in[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                            rx, (int)(row_ok ? at + col_in[q] : OOB), 0, 0));
  };
  auto store_row = [&](int oh, const f32x4 (&acc)[TW]) {
    const bool row_ok = oh >= oh0 && oh < oh1;
    const unsigned at = (unsigned)oh * y_row;
#pragma unroll
    for (int j = 0; j < TW; j++) {
      f32x4 v = acc[j] + b;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = act_fast(v[e], af);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), ry,
                                             (int)(row_ok ? at + col_out[j] : OOB), 0, 0);
    }
  };
  // Input row ih is filter row kh of output row ih + pad_top - kh: `newest` starts with it
  // (kh = 0), `middle` gets its second filter row, `oldest` its last and is complete.
  auto feed = [&](const f32x4 (&in)[IW], f32x4 (&oldest)[TW], f32x4 (&middle)[TW],
                  f32x4 (&newest)[TW]) {
#pragma unroll
    for (int j = 0; j < TW; j++) {
      f32x4 a = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kw = 0; kw < 3; kw++) a += in[j + kw] * w[kw];
      newest[j] = a;
#pragma unroll
      for (int kw = 0; kw < 3; kw++) middle[j] += in[j + kw] * w[3 + kw];
#pragma unroll
      for (int kw = 0; kw < 3; kw++) oldest[j] += in[j + kw] * w[6 + kw];
    }
  };

  f32x4 acc[3][TW];
#pragma unroll
  for (int i = 0; i < 3; i++)
#pragma unroll
    for (int j = 0; j < TW; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  f32x4 buf[NB][IW];
#pragma unroll
  for (int q = 0; q < PF; q++) load_row(ih_first + q, buf[q]);
  // One step: start the loads of the row PF steps ahead, feed the current row, store the output
  // row it completes (input row ih completes output row ih + pad_top - 2).  NB row buffers and
  // three accumulator rows take turns: the pattern repeats every PERIOD rows, and with the loop
  // unrolled every buffer of a step is known at compile time.  Rows past ih_last load nothing
  // and store nothing.
  for (int ih = ih_first; ih <= ih_last; ih += PERIOD) {
#pragma unroll
    for (int s = 0; s < PERIOD; s++) {

      load_row(ih + s + PF, buf[(s + PF) % NB]);
      __builtin_amdgcn_sched_barrier(0);  // loads first, and none from a later step
      feed(buf[s % NB], acc[s % 3], acc[(s + 1) % 3], acc[(s + 2) % 3]);
      store_row(ih + s + ci.pad_top - 2, acc[s % 3]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// Any filter size, stride, dilation and channel multiplier: one lane per output element,
// output channel fastest.
__global__ void depthwise_generic_kernel(const DwArgs p) {
  const tfhip_conv2d_info& ci = p.ci;
  const int64_t total = (int64_t)ci.batch * ci.out_h * ci.out_w * ci.out_c;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total; gid += stride) {
    const int oc = (int)(gid % ci.out_c);
    int64_t t = gid / ci.out_c;
    const int ow = (int)(t % ci.out_w);
    t /= ci.out_w;
    const int oh = (int)(t % ci.out_h);
    const int n = (int)(t / ci.out_h);
    const int c = oc / p.ch_mul, q = oc - c * p.ch_mul;
    float acc = 0.f;
    for (int kh = 0; kh < ci.filter_h; kh++) {
      const int ih = oh * ci.stride_h - ci.pad_top + kh * ci.dilation_h;
      if ((unsigned)ih >= (unsigned)ci.in_h) continue;
      for (int kw = 0; kw < ci.filter_w; kw++) {
        const int iw = ow * ci.stride_w - ci.pad_left + kw * ci.dilation_w;
        if ((unsigned)iw >= (unsigned)ci.in_w) continue;
        const int64_t wi = (((int64_t)kh * ci.filter_w + kw) * ci.in_c + c) * p.ch_mul + q;
        const float wv = p.quant ? dq(static_cast<const unsigned char*>(p.w)[wi], p.qscale, p.qmin)
                                 : static_cast<const float*>(p.w)[wi];
        acc += p.x[(((int64_t)n * ci.in_h + ih) * ci.in_w + iw) * ci.in_c + c] * wv;
      }
    }
    if (p.bias_kind == TFHIP_BCAST_COLUMN) acc += p.bias[oc];
    else if (p.bias_kind == TFHIP_BCAST_SCALAR) acc += p.bias[0];
    p.y[gid] = act_f(acc, p.act);
  }
}

// avg: mean over the in-bounds part of the window (count = visited pixels,
// backend_cpu.ts:2312-2336); max: NaN never wins (`pixel > max`).  Channel fastest.
__global__ void pool2d_kernel(const float* x, float* y, const tfhip_conv2d_info ci, int kind) {
  const int eff_h = ci.filter_h + (ci.filter_h - 1) * (ci.dilation_h - 1);
  const int eff_w = ci.filter_w + (ci.filter_w - 1) * (ci.dilation_w - 1);
  const int64_t total = (int64_t)ci.batch * ci.out_h * ci.out_w * ci.out_c;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total; gid += stride) {
    const int c = (int)(gid % ci.out_c);
    int64_t t = gid / ci.out_c;
    const int ow = (int)(t % ci.out_w);
    t /= ci.out_w;
    const int oh = (int)(t % ci.out_h);
    const int n = (int)(t / ci.out_h);
    const int r0 = oh * ci.stride_h - ci.pad_top, c0 = ow * ci.stride_w - ci.pad_left;
    const int r_min = r0 > 0 ? r0 : 0, c_min = c0 > 0 ? c0 : 0;
    const int r_max = ci.in_h < eff_h + r0 ? ci.in_h : eff_h + r0;
    const int c_max = ci.in_w < eff_w + c0 ? ci.in_w : eff_w + c0;
    double sum = 0.0;
    float mx = -INFINITY;
    int count = 0;
    for (int r = r_min; r < r_max; r += ci.dilation_h)
      for (int q = c_min; q < c_max; q += ci.dilation_w) {
        const float v = x[(((int64_t)n * ci.in_h + r) * ci.in_w + q) * ci.in_c + c];
        if (kind == TFHIP_POOL_MAX) {
          if (v > mx) mx = v;
        } else {
          sum += (double)v;
          count++;
        }
      }
    y[gid] = kind == TFHIP_POOL_AVG ? (float)(sum / (double)count) : mx;
  }
}

// Global average pool (window = whole image, 'valid'): x [N, HW, C] -> y [N, C].  One lane
// per (image, channel quad); consecutive lanes read consecutive channel quads.
__global__ void global_avgpool_kernel(const float* x, float* y, int n_img, int hw, int c4) {
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= n_img * c4) return;
  const int n = gid / c4, cq = gid - n * c4;
  const f32x4* src = reinterpret_cast<const f32x4*>(x) + (int64_t)n * hw * c4 + cq;
  double s0 = 0, s1 = 0, s2 = 0, s3 = 0;
  // seven loads in flight at a time (a 7x7 window is 7 such groups); summed in pixel order
  int i = 0;
  for (; i + 7 <= hw; i += 7) {
    f32x4 v[7];
#pragma unroll
    for (int u = 0; u < 7; u++) v[u] = src[(int64_t)(i + u) * c4];
#pragma unroll
    for (int u = 0; u < 7; u++) {
      s0 += v[u][0]; s1 += v[u][1]; s2 += v[u][2]; s3 += v[u][3];
    }
  }
  for (; i < hw; i++) {
    const f32x4 v = src[(int64_t)i * c4];
    s0 += v[0]; s1 += v[1]; s2 += v[2]; s3 += v[3];
  }
  const double d = (double)hw;
  reinterpret_cast<f32x4*>(y)[gid] = f32x4{(float)(s0 / d), (float)(s1 / d), (float)(s2 / d), (float)(s3 / d)};
}

// localResponseNormalization4D (backend_cpu.ts:3211-3244): out = x * (bias + alpha * sum of
// x^2 over the channels within depth_radius of this one) ^ -beta.  One lane per element; the
// window of neighbouring lanes overlaps, so the loads come out of L1.
__global__ void lrn_kernel(const float* __restrict__ x, float* __restrict__ out, int64_t n,
                           int channels, int radius, float bias, float alpha, float beta) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int c = (int)(i % channels);
    const int64_t px = i - c;
    const int lo = c - radius > 0 ? c - radius : 0;
    const int hi = c + radius < channels - 1 ? c + radius : channels - 1;
    float sum = 0.f;
    for (int k = lo; k <= hi; k++) {
      const float z = x[px + k];
      sum += z * z;
    }
    out[i] = x[i] * powf(bias + alpha * sum, -beta);
  }
}

// LRNGrad (backend_cpu.ts:3246-3281), gathered: element k collects, from every channel o of its
// pixel whose window holds k, dy[o] * (-2 alpha beta x[k] y[o] / norm[o] + [o == k] norm[o]^-beta)
// with norm[o] = bias + alpha * sum of x^2 over the window of o.
__global__ void lrn_grad_kernel(const float* __restrict__ dy, const float* __restrict__ x,
                                const float* __restrict__ y, float* __restrict__ dx, int64_t n,
                                int channels, int radius, float bias, float alpha, float beta) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int k = (int)(i % channels);
    const int64_t px = i - k;
    const int o_lo = k - radius > 0 ? k - radius : 0;
    const int o_hi = k + radius < channels - 1 ? k + radius : channels - 1;
    const float xk = x[i];
    float acc = 0.f;
    for (int o = o_lo; o <= o_hi; o++) {
      const int lo = o - radius > 0 ? o - radius : 0;
      const int hi = o + radius < channels - 1 ? o + radius : channels - 1;
      float sum = 0.f;
      for (int q = lo; q <= hi; q++) {
        const float z = x[px + q];
        sum += z * z;
      }
      const float norm = alpha * sum + bias;
      float d = -2.f * alpha * beta * xk * y[px + o] / norm;
      if (o == k) d += powf(norm, -beta);
      acc += d * dy[px + o];
    }
    dx[i] = acc;
  }
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <int S, int TH, int TW>
static void launch_dw3x3(tfhip_ctx* ctx, DwArgs& p) {
  ctx->name_kernel("depthwise3x3_s%d_%dx%d", S, TH, TW);
  p.tiles_h = (int)ceil_div(p.ci.out_h, TH);
  p.tiles_w = (int)ceil_div(p.ci.out_w, TW);
  const int64_t total = (int64_t)p.ci.batch * p.tiles_h * p.tiles_w * p.c4;
  p.reverse = ctx->take_sweep();
  tfhip::launch(ctx, (depthwise3x3_kernel<S, TH, TW>), dim3((unsigned)ceil_div(total, 256)),
                     dim3(256), 0, p);
}

template <int TW, int PF>
static void launch_dw3x3_rows(tfhip_ctx* ctx, DwArgs& p, int rows) {
  ctx->name_kernel("depthwise3x3_s1_rows_w%d_ahead%d", TW, PF);
  const int chunks = (int)ceil_div(p.ci.out_h, rows);
  p.tiles_w = (int)ceil_div(p.ci.out_w, TW);
  const int64_t total = (int64_t)p.ci.batch * chunks * p.tiles_w * p.c4;
  p.reverse = ctx->take_sweep();
  tfhip::launch(ctx, (depthwise3x3_rows_kernel<TW, PF>), dim3((unsigned)ceil_div(total, 256)),
                     dim3(256), 0, p, rows, chunks,
                     (unsigned)((int64_t)p.ci.batch * p.ci.in_h * p.ci.in_w * p.ci.in_c * 4),
                     (unsigned)((int64_t)p.ci.batch * p.ci.out_h * p.ci.out_w * p.ci.out_c * 4));
}

static int check_geometry(tfhip_ctx* ctx, const char* op, const tfhip_conv2d_info* ci) {
  if (ci->batch < 0 || ci->in_h < 0 || ci->in_w < 0 || ci->in_c < 0 || ci->out_h < 0 ||
      ci->out_w < 0 || ci->out_c < 0 || ci->filter_h <= 0 || ci->filter_w <= 0 ||
      ci->stride_h <= 0 || ci->stride_w <= 0 || ci->dilation_h <= 0 || ci->dilation_w <= 0)
    return ctx->fail(TFHIP_EINVAL, "%s: bad geometry", op);
  return TFHIP_OK;
}

// Picks and launches the kernel for a filled-in DwArgs (p.x, p.w, p.y, bias, act, quant set).
static int dispatch_depthwise(tfhip_ctx* ctx, DwArgs& p, const tfhip_conv2d_info* ci, int ch_mul,
                              int bias_kind, int64_t x_n, int64_t o_n) {
  const bool fast = ci->filter_h == 3 && ci->filter_w == 3 && ci->dilation_h == 1 &&
                    ci->dilation_w == 1 && ch_mul == 1 && ci->in_c % 4 == 0 &&
                    ci->stride_h == ci->stride_w && (ci->stride_h == 1 || ci->stride_h == 2) &&
                    aligned16(p.x) && aligned16(p.w) && aligned16(p.y) &&
                    (bias_kind != TFHIP_BCAST_COLUMN || aligned16(p.bias));
  if (fast) {
    p.c4 = ci->in_c / 4;
    // Stride 2 streams best with one output per lane (measured on MI355X, fp32, batch 32-64).
    // Stride 1: the row-walking kernel when the image is large enough to give every SIMD a
    // few wavefronts (it fetches each input row once), else 2x2 patches.  Measured on MI355X
    // (fp32, batch 32-64): 28-row chunks stream best; halve them when that would leave a
    // second, nearly empty round of wavefronts, or too few wavefronts.
    int rows = 0;
    if (ci->stride_h == 1 && x_n * 4 < (1ll << 31) && o_n * 4 < (1ll << 31)) {
      const int64_t lanes_per_chunk = (int64_t)ci->batch * ceil_div(ci->out_w, 2) * p.c4;
      const int64_t slots = (int64_t)ctx->num_cus * 12;  // 3 wavefronts per SIMD
      auto waves = [&](int r) { return lanes_per_chunk * ceil_div(ci->out_h, r) / 64; };
      rows = ci->out_h < 28 ? ci->out_h : 28;
      while (rows > 7 && waves(rows) < slots / 2) rows = (rows + 1) / 2;
      if (rows > 7 && waves(rows) > slots && waves(rows) * 2 < slots * 3) rows = (rows + 1) / 2;
      if (waves(rows) < slots / 4) rows = 0;
    }
    if (rows > 0) {
      // Two input rows in flight per wavefront (measured in a batch-64 MobileNet step against one
      // row: [64,14,14,512] 10.6 -> 9.4 us, [64,7,7,1024] 7.5 -> 6.8, [64,28,28,256] 25.1 -> 24.6;
      // three rows in flight, 217 registers: 11.1 / 8.2 / 26.8; strips one output column wide with
      // one / two / three rows in flight: 10.0 / 10.3 / 11.5 us on the first shape)
      launch_dw3x3_rows<2, 2>(ctx, p, rows);
    } else if (ci->stride_h == 1) {
      if (ci->out_w >= 112 && ci->in_c >= 128 && ci->out_w % 8 == 0) launch_dw3x3<1, 2, 8>(ctx, p);
      else launch_dw3x3<1, 2, 2>(ctx, p);
    } else {
      launch_dw3x3<2, 1, 1>(ctx, p);
    }
  } else {
    ctx->name_kernel("depthwise_generic");
    const int64_t blocks = ceil_div(o_n, 256);
    const int64_t cap = (int64_t)ctx->num_cus * 16;
    tfhip::launch(ctx, depthwise_generic_kernel, dim3((unsigned)(blocks > cap ? cap : blocks)),
                       dim3(256), 0, p);
  }
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

// depthwiseConv2D of float32 device buffers without bias or activation: the forward kernels
// reused by depthwiseConv2DDerInput (stride 1: dx is the depthwise convolution of dy with the
// spatially flipped filter).
int depthwise_forward_f32(tfhip_ctx* ctx, const float* x, const float* w, float* y,
                          const tfhip_conv2d_info* ci) {
  DwArgs p = {};
  p.x = x;
  p.w = w;
  p.y = y;
  p.ci = *ci;
  p.ch_mul = ci->out_c / ci->in_c;
  p.bias_kind = TFHIP_BCAST_NONE;
  p.act = TFHIP_ACT_LINEAR;
  return dispatch_depthwise(ctx, p, ci, p.ch_mul, TFHIP_BCAST_NONE,
                            (int64_t)ci->batch * ci->in_h * ci->in_w * ci->in_c,
                            (int64_t)ci->batch * ci->out_h * ci->out_w * ci->out_c);
}

}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_depthwise_conv2d(tfhip_ctx* ctx, int64_t x, int64_t filter, int64_t out,
                                      const tfhip_conv2d_info* ci, int64_t bias, int bias_kind,
                                      int act, const tfhip_qparams* q) {
  if (!ctx || !ci) return TFHIP_EINVAL;
  int rc;
  if ((rc = check_geometry(ctx, "depthwiseConv2D", ci))) return rc;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bw, filter);
  TFHIP_GET(ctx, bo, out);
  if (ci->in_c <= 0 || ci->out_c % ci->in_c != 0)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2D: out channels must be a multiple of in channels");
  const int ch_mul = ci->out_c / ci->in_c;
  const int64_t x_n = (int64_t)ci->batch * ci->in_h * ci->in_w * ci->in_c;
  const int64_t w_n = (int64_t)ci->filter_h * ci->filter_w * ci->out_c;
  const int64_t o_n = (int64_t)ci->batch * ci->out_h * ci->out_w * ci->out_c;
  if (bx->numel != x_n || bw->numel != w_n || bo->numel != o_n)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2D: buffer sizes do not match the geometry");
  if (bo->dtype != TFHIP_FLOAT32)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2D: output buffer must be float32");
  if (act != TFHIP_ACT_LINEAR && act != TFHIP_ACT_RELU && act != TFHIP_ACT_RELU6)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2D: activation %d is not folded here", act);
  if (bias_kind != TFHIP_BCAST_NONE && bias_kind != TFHIP_BCAST_SCALAR &&
      bias_kind != TFHIP_BCAST_COLUMN)
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2D: bias layout %d is not folded here", bias_kind);
  const bool quant = bw->dtype == TFHIP_UINT8Q;
  if (quant != (q != nullptr))
    return ctx->fail(TFHIP_EINVAL, "depthwiseConv2D: qparams must be given exactly for a quantised filter");
  if (o_n == 0) return TFHIP_OK;

  Temp tx(ctx), tw(ctx), tb(ctx);
  DwArgs p = {};
  if ((rc = as_f32(ctx, bx, &tx, &p.x))) return rc;
  if (quant) {
    p.w = bw->ptr;
    p.quant = 1;
    p.qscale = q->scale;
    p.qmin = q->min;
  } else {
    const float* wf;
    if ((rc = as_f32(ctx, bw, &tw, &wf))) return rc;
    p.w = wf;
  }
  if (bias_kind != TFHIP_BCAST_NONE) {
    TFHIP_GET(ctx, bb, bias);
    if (bb->numel != (bias_kind == TFHIP_BCAST_SCALAR ? 1 : ci->out_c))
      return ctx->fail(TFHIP_EINVAL, "depthwiseConv2D: bias size does not match its layout");
    if ((rc = as_f32(ctx, bb, &tb, &p.bias))) return rc;
  }
  p.y = static_cast<float*>(bo->ptr);
  p.ci = *ci;
  p.ch_mul = ch_mul;
  p.bias_kind = bias_kind;
  p.act = act;

  return dispatch_depthwise(ctx, p, ci, ch_mul, bias_kind, x_n, o_n);
}

extern "C" int tfhip_pool2d(tfhip_ctx* ctx, int64_t x, int64_t out, const tfhip_conv2d_info* ci,
                            int kind) {
  if (!ctx || !ci) return TFHIP_EINVAL;
  int rc;
  if ((rc = check_geometry(ctx, "pool", ci))) return rc;
  if (kind != TFHIP_POOL_AVG && kind != TFHIP_POOL_MAX)
    return ctx->fail(TFHIP_EINVAL, "pool: unknown kind %d", kind);
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (ci->in_c != ci->out_c) return ctx->fail(TFHIP_EINVAL, "pool: channel counts differ");
  const int64_t x_n = (int64_t)ci->batch * ci->in_h * ci->in_w * ci->in_c;
  const int64_t o_n = (int64_t)ci->batch * ci->out_h * ci->out_w * ci->out_c;
  if (bx->numel != x_n || bo->numel != o_n)
    return ctx->fail(TFHIP_EINVAL, "pool: buffer sizes do not match the geometry");
  if (bo->dtype != TFHIP_FLOAT32) return ctx->fail(TFHIP_EINVAL, "pool: output must be float32");
  if (o_n == 0) return TFHIP_OK;
  Temp tx(ctx);
  const float* xf;
  if ((rc = as_f32(ctx, bx, &tx, &xf))) return rc;
  float* y = static_cast<float*>(bo->ptr);
  const bool global = kind == TFHIP_POOL_AVG && ci->out_h == 1 && ci->out_w == 1 &&
                      ci->filter_h == ci->in_h && ci->filter_w == ci->in_w && ci->pad_top == 0 &&
                      ci->pad_left == 0 && ci->dilation_h == 1 && ci->dilation_w == 1 &&
                      ci->in_c % 4 == 0 && aligned16(xf) && aligned16(y);
  if (global) {
    ctx->name_kernel("global_avgpool");
    const int items = ci->batch * (ci->in_c / 4);
    tfhip::launch(ctx, global_avgpool_kernel, dim3((unsigned)ceil_div(items, 64)), dim3(64), 0, xf, y, ci->batch, ci->in_h * ci->in_w, ci->in_c / 4);
  } else {
    const int64_t blocks = ceil_div(o_n, 256);
    const int64_t cap = (int64_t)ctx->num_cus * 16;
    ctx->name_kernel("pool2d");
    tfhip::launch(ctx, pool2d_kernel, dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(256), 0, xf, y, *ci, kind);
  }
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

static int lrn_check(tfhip_ctx* ctx, const char* op, const Buf* const* bufs, int n_bufs, int64_t pixels,
                     int channels, int radius) {
  if (pixels < 0 || channels < 0 || radius < 0) return ctx->fail(TFHIP_EINVAL, "%s: bad geometry", op);
  for (int i = 0; i < n_bufs; i++) {
    if (bufs[i]->numel != pixels * channels)
      return ctx->fail(TFHIP_EINVAL, "%s: a buffer holds %lld elements, the shape needs %lld", op,
                       (long long)bufs[i]->numel, (long long)(pixels * channels));
    if (bufs[i]->dtype != TFHIP_FLOAT32) return ctx->fail(TFHIP_EINVAL, "%s: float32 buffers only", op);
  }
  return TFHIP_OK;
}

extern "C" int tfhip_lrn(tfhip_ctx* ctx, int64_t x, int64_t out, int64_t pixels, int channels,
                         int depth_radius, float bias, float alpha, float beta) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  const Buf* bufs[] = {bx, bo};
  int rc;
  if ((rc = lrn_check(ctx, "localResponseNormalization", bufs, 2, pixels, channels, depth_radius))) return rc;
  const int64_t n = bx->numel;
  if (n == 0) return TFHIP_OK;
  const int64_t blocks = ceil_div(n, 256), cap = (int64_t)ctx->num_cus * 16;
  tfhip::launch(ctx, lrn_kernel, dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(256), 0,
                     (const float*)bx->ptr, (float*)bo->ptr, n, channels, depth_radius, bias, alpha, beta);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_lrn_grad(tfhip_ctx* ctx, int64_t dy, int64_t x, int64_t y, int64_t dx,
                              int64_t pixels, int channels, int depth_radius, float bias,
                              float alpha, float beta) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bdy, dy);
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, by, y);
  TFHIP_GET(ctx, bdx, dx);
  const Buf* bufs[] = {bdy, bx, by, bdx};
  int rc;
  if ((rc = lrn_check(ctx, "LRNGrad", bufs, 4, pixels, channels, depth_radius))) return rc;
  const int64_t n = bx->numel;
  if (n == 0) return TFHIP_OK;
  const int64_t blocks = ceil_div(n, 256), cap = (int64_t)ctx->num_cus * 16;
  tfhip::launch(ctx, lrn_grad_kernel, dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(256), 0, (const float*)bdy->ptr, (const float*)bx->ptr, (const float*)by->ptr,
                     (float*)bdx->ptr, n, channels, depth_radius, bias, alpha, beta);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}
