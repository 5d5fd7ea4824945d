/*
 * cpu_ref.c — TEST INFRASTRUCTURE, not product code.
 *
 * A plain-C restatement of the loops of tfjs-core's backend_cpu that sit on the hip
 * backend's hot path.  It exists only to check the HIP kernels (tests, smoke) and to be
 * timed as the CPU baseline; nothing in the product path may call it.
 *
 * backend_cpu computes in JavaScript numbers (IEEE double) and stores into Float32Array /
 * Int32Array, so every function below does its arithmetic in double and rounds to float
 * exactly where the reference stores to a typed array.  Each function cites the reference
 * lines it follows (paths relative to tfjs-core/src/).
 *
 * Parity pins (see tests/test_oracle_*.py): every function is checked against the
 * known-answer vectors of the reference's own *_test.ts files transcribed under
 * tests/golden/, plus float64 brute-force / closed-form checks.  One behaviour is
 * PARITY UNPINNED: depthwise convolution with asymmetric padding on non-square inputs,
 * where backend_cpu swaps padLeft/padTop (backends/cpu/backend_cpu.ts:2000,2010); no
 * reference vector covers it.  `pad_quirk` selects the backend_cpu behaviour; 0 selects
 * the TensorFlow / WebGL semantics that the hip backend implements.
 *
 * Build: gcc -O2 -fPIC -shared (see Makefile).  -ffast-math must NOT be used: the
 * float/double rounding points are the whole point.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct ref_conv2d_info { /* same field order as tfhip_conv2d_info */
  int32_t batch;
  int32_t in_h, in_w, in_c;
  int32_t out_h, out_w, out_c;
  int32_t stride_h, stride_w;
  int32_t dilation_h, dilation_w;
  int32_t filter_h, filter_w;
  int32_t pad_top, pad_left, pad_bottom, pad_right;
} ref_conv2d_info;

/* backends/cpu/backend_cpu.ts:491-540 — 48-wide blocking (blockSize, :83); products and
 * the per-block sum are doubles, `resVals[...] += sum` rounds to float once per k-block. */
void ref_batch_matmul(const float* a, const float* b, float* out, int batch, int m, int n,
                      int k, int transpose_a, int transpose_b) {
  const int bs = 48;
  const int64_t a_batch = (int64_t)m * k, b_batch = (int64_t)k * n;
  const int64_t a_outer = transpose_a ? 1 : k, a_inner = transpose_a ? m : 1;
  const int64_t b_inner = transpose_b ? 1 : n, b_outer = transpose_b ? k : 1;
  const int64_t size = (int64_t)m * n;
  memset(out, 0, sizeof(float) * (size_t)(batch * size));
  for (int bi = 0; bi < batch; bi++)
    for (int i0 = 0; i0 < m; i0 += bs)
      for (int j0 = 0; j0 < n; j0 += bs)
        for (int k0 = 0; k0 < k; k0 += bs) {
          const int i1 = i0 + bs < m ? i0 + bs : m;
          const int j1 = j0 + bs < n ? j0 + bs : n;
          const int k1 = k0 + bs < k ? k0 + bs : k;
          for (int i = i0; i < i1; i++)
            for (int j = j0; j < j1; j++) {
              double sum = 0.0;
              for (int kk = k0; kk < k1; kk++)
                sum += (double)a[bi * a_batch + i * a_outer + kk * a_inner] *
                       (double)b[kk * b_inner + j * b_outer + bi * b_batch];
              float* r = &out[bi * size + (int64_t)i * n + j];
              *r = (float)((double)*r + sum);
            }
        }
}

/* Element strides of an image tensor in either data format, as backend_cpu.ts:1565-1572 takes
 * them from x.strides / y.strides: channelsLast [b,h,w,c], channelsFirst [b,c,h,w]. */
typedef struct img_strides {
  int64_t b, row, col, ch;
} img_strides;
static img_strides strides_of(int h, int w, int c, int channels_first) {
  img_strides s;
  s.b = (int64_t)h * w * c;
  if (channels_first) {
    s.ch = (int64_t)h * w;
    s.row = w;
    s.col = 1;
  } else {
    s.row = (int64_t)w * c;
    s.col = c;
    s.ch = 1;
  }
  return s;
}

/* backends/cpu/backend_cpu.ts:1552-1616; out-of-bounds taps are skipped (:1586,:1596);
 * `yVals[...] += xVal * w` rounds to float after every MAC.  The data format only changes the
 * strides (:1565-1572), not the order of the loops. */
static void conv2d_strided(const float* x, const float* w, float* y, const ref_conv2d_info* ci,
                           int channels_first) {
  const img_strides xs = strides_of(ci->in_h, ci->in_w, ci->in_c, channels_first);
  const img_strides ys = strides_of(ci->out_h, ci->out_w, ci->out_c, channels_first);
  const int64_t w_s0 = (int64_t)ci->filter_w * ci->in_c * ci->out_c;
  const int64_t w_s1 = (int64_t)ci->in_c * ci->out_c;
  const int oc = ci->out_c;
  memset(y, 0, sizeof(float) * (size_t)(ys.b * ci->batch));
  for (int b = 0; b < ci->batch; ++b)
    for (int yr = 0; yr < ci->out_h; ++yr) {
      const int xr_corner = yr * ci->stride_h - ci->pad_top;
      for (int wr = 0; wr < ci->filter_h; ++wr) {
        const int xr = xr_corner + wr * ci->dilation_h;
        if (xr < 0 || xr >= ci->in_h) continue;
        for (int yc = 0; yc < ci->out_w; ++yc) {
          float* yp = y + b * ys.b + yr * ys.row + yc * ys.col;
          const int xc_corner = yc * ci->stride_w - ci->pad_left;
          for (int wc = 0; wc < ci->filter_w; ++wc) {
            const int xc = xc_corner + wc * ci->dilation_w;
            if (xc < 0 || xc >= ci->in_w) continue;
            const float* xp = x + b * xs.b + xr * xs.row + xc * xs.col;
            const float* wp = w + wr * w_s0 + wc * w_s1;
            for (int d1 = 0; d1 < ci->in_c; ++d1) {
              const double xv = (double)xp[d1 * xs.ch];
              for (int d2 = 0; d2 < oc; ++d2)
                yp[d2 * ys.ch] = (float)((double)yp[d2 * ys.ch] + xv * (double)wp[d2]);
              wp += oc;
            }
          }
        }
      }
    }
}
void ref_conv2d(const float* x, const float* w, float* y, const ref_conv2d_info* ci) {
  conv2d_strided(x, w, y, ci, 0);
}
/* x [b, in_c, in_h, in_w], y [b, out_c, out_h, out_w]; the filter stays [fh, fw, in_c, out_c]. */
void ref_conv2d_nchw(const float* x, const float* w, float* y, const ref_conv2d_info* ci) {
  conv2d_strided(x, w, y, ci, 1);
}

/* backends/cpu/backend_cpu.ts:1979-2035.  pad_quirk != 0 reproduces :2000 (rows offset by
 * padLeft) and :2010 (columns offset by padTop); 0 uses top for rows, left for columns. */
void ref_depthwise_conv2d(const float* x, const float* w, float* y, const ref_conv2d_info* ci,
                          int pad_quirk) {
  const int ch_mul = ci->out_c / ci->in_c;
  const int64_t x_row = (int64_t)ci->in_w * ci->in_c, x_b = x_row * ci->in_h;
  const int64_t y_row = (int64_t)ci->out_w * ci->out_c, y_b = y_row * ci->out_h;
  const int64_t w_s0 = (int64_t)ci->filter_w * ci->in_c * ch_mul;
  const int64_t w_s1 = (int64_t)ci->in_c * ch_mul;
  const int row_pad = pad_quirk ? ci->pad_left : ci->pad_top;
  const int col_pad = pad_quirk ? ci->pad_top : ci->pad_left;
  memset(y, 0, sizeof(float) * (size_t)(y_b * ci->batch));
  for (int b = 0; b < ci->batch; ++b)
    for (int yr = 0; yr < ci->out_h; ++yr) {
      const int xr_corner = yr * ci->stride_h - row_pad;
      for (int wr = 0; wr < ci->filter_h; ++wr) {
        const int xr = xr_corner + wr * ci->dilation_h;
        if (xr < 0 || xr >= ci->in_h) continue;
        for (int yc = 0; yc < ci->out_w; ++yc) {
          const int xc_corner = yc * ci->stride_w - col_pad;
          for (int wc = 0; wc < ci->filter_w; ++wc) {
            const int xc = xc_corner + wc * ci->dilation_w;
            if (xc < 0 || xc >= ci->in_w) continue;
            const float* xp = x + b * x_b + xr * x_row + (int64_t)xc * ci->in_c;
            const float* wp = w + wr * w_s0 + wc * w_s1;
            float* yp = y + b * y_b + yr * y_row + (int64_t)yc * ci->out_c;
            for (int d1 = 0; d1 < ci->in_c; ++d1) {
              const double xv = (double)xp[d1];
              for (int q = 0; q < ch_mul; ++q)
                yp[q] = (float)((double)yp[q] + xv * (double)wp[q]);
              yp += ch_mul;
              wp += ch_mul;
            }
          }
        }
      }
    }
}

/* backends/cpu/backend_cpu.ts:2273-2341 (avgPool :2869-2873, maxPool :2343-2345).
 * kind 0 = avg: double window sum over in-bounds pixels only, divided by their count.
 * kind 1 = max: starts at -inf, `pixel > max` so NaN never replaces a number; the
 * isNaN(minMaxValue) early exit (:2329) can never fire for max, kept for fidelity. */
void ref_pool2d(const float* x, float* y, const ref_conv2d_info* ci, int kind) {
  const int eff_h = ci->filter_h + (ci->filter_h - 1) * (ci->dilation_h - 1);
  const int eff_w = ci->filter_w + (ci->filter_w - 1) * (ci->dilation_w - 1);
  const int64_t x_row = (int64_t)ci->in_w * ci->in_c, x_b = x_row * ci->in_h;
  const int64_t y_row = (int64_t)ci->out_w * ci->out_c, y_b = y_row * ci->out_h;
  for (int b = 0; b < ci->batch; ++b)
    for (int d = 0; d < ci->in_c; ++d)
      for (int yr = 0; yr < ci->out_h; ++yr) {
        const int xr_corner = yr * ci->stride_h - ci->pad_top;
        const int xr_min = xr_corner > 0 ? xr_corner : 0;
        const int xr_max = ci->in_h < eff_h + xr_corner ? ci->in_h : eff_h + xr_corner;
        for (int yc = 0; yc < ci->out_w; ++yc) {
          const int xc_corner = yc * ci->stride_w - ci->pad_left;
          const int xc_min = xc_corner > 0 ? xc_corner : 0;
          const int xc_max = ci->in_w < eff_w + xc_corner ? ci->in_w : eff_w + xc_corner;
          double mm = -INFINITY, avg = 0.0;
          int count = 0;
          for (int xr = xr_min; xr < xr_max; xr += ci->dilation_h) {
            for (int xc = xc_min; xc < xc_max; xc += ci->dilation_w) {
              const double pixel = (double)x[b * x_b + xr * x_row + (int64_t)xc * ci->in_c + d];
              if (kind == 1) {
                if (pixel > mm) mm = pixel;
              } else {
                avg += pixel;
                count++;
              }
            }
            if (isnan(mm)) break;
          }
          y[b * y_b + yr * y_row + (int64_t)yc * ci->out_c + d] =
              kind == 0 ? (float)(avg / (double)count) : (float)mm;
        }
      }
}

/* ---- backward kernels --------------------------------------------------------------- */

/* backends/cpu/backend_cpu.ts:1686-1762.  The loop bounds are JavaScript numbers: yRMax =
 * min(outHeight, (filterHeight + xRCorner) / strideHeight) is fractional and compared with `<`;
 * one double dot product per dx element, stored to float once.  The data format changes the
 * strides of dx and dy only (:1698-1706). */
static void conv2d_der_input_strided(const float* dy, const float* w, float* dx,
                                     const ref_conv2d_info* ci, int channels_first) {
  const int fh = ci->filter_h, fw = ci->filter_w, ic = ci->in_c, oc = ci->out_c;
  const int top_pad = fh - 1 - ci->pad_top, left_pad = fw - 1 - ci->pad_left;
  const img_strides xs = strides_of(ci->in_h, ci->in_w, ic, channels_first);
  const img_strides ys = strides_of(ci->out_h, ci->out_w, oc, channels_first);
  const int64_t w_s0 = (int64_t)fw * ic * oc, w_s1 = (int64_t)ic * oc, w_s2 = oc;
  for (int b = 0; b < ci->batch; ++b)
    for (int d1 = 0; d1 < ic; ++d1)
      for (int xr = 0; xr < ci->in_h; ++xr) {
        const int xr_corner = xr - top_pad;
        const double yr_min = fmax(0.0, ceil((double)xr_corner / ci->stride_h));
        const double yr_max = fmin((double)ci->out_h, (double)(fh + xr_corner) / ci->stride_h);
        for (int xc = 0; xc < ci->in_w; ++xc) {
          const int xc_corner = xc - left_pad;
          const double yc_min = fmax(0.0, ceil((double)xc_corner / ci->stride_w));
          const double yc_max = fmin((double)ci->out_w, (double)(fw + xc_corner) / ci->stride_w);
          double dot = 0.0;
          for (int yr = (int)yr_min; yr < yr_max; ++yr) {
            const int wr = yr * ci->stride_h - xr_corner;
            for (int yc = (int)yc_min; yc < yc_max; ++yc) {
              const int wc = yc * ci->stride_w - xc_corner;
              const float* dyp = dy + b * ys.b + yr * ys.row + yc * ys.col;
              const float* wp = w + w_s0 * (fh - 1 - wr) + w_s1 * (fw - 1 - wc) + w_s2 * d1;
              for (int d2 = 0; d2 < oc; ++d2) dot += (double)dyp[d2 * ys.ch] * (double)wp[d2];
            }
          }
          dx[b * xs.b + xr * xs.row + xc * xs.col + d1 * xs.ch] = (float)dot;
        }
      }
}
void ref_conv2d_der_input(const float* dy, const float* w, float* dx, const ref_conv2d_info* ci) {
  conv2d_der_input_strided(dy, w, dx, ci, 0);
}
void ref_conv2d_der_input_nchw(const float* dy, const float* w, float* dx,
                               const ref_conv2d_info* ci) {
  conv2d_der_input_strided(dy, w, dx, ci, 1);
}

/* backends/cpu/backend_cpu.ts:1849-1898: per filter element one double dot product over batch,
 * output rows and columns, stored to float once; channelsFirst reads x and dy through other
 * strides (:1857-1865). */
static void conv2d_der_filter_strided(const float* x, const float* dy, float* dw,
                                      const ref_conv2d_info* ci, int channels_first) {
  const int fh = ci->filter_h, fw = ci->filter_w, ic = ci->in_c, oc = ci->out_c;
  const img_strides xs = strides_of(ci->in_h, ci->in_w, ic, channels_first);
  const img_strides ys = strides_of(ci->out_h, ci->out_w, oc, channels_first);
  for (int wr = 0; wr < fh; ++wr) {
    const double yr_min = fmax(0.0, ceil((double)(ci->pad_top - wr) / ci->stride_h));
    const double yr_max = fmin((double)ci->out_h, (double)(ci->in_h + ci->pad_top - wr) / ci->stride_h);
    for (int wc = 0; wc < fw; ++wc) {
      const double yc_min = fmax(0.0, ceil((double)(ci->pad_left - wc) / ci->stride_w));
      const double yc_max = fmin((double)ci->out_w, (double)(ci->in_w + ci->pad_left - wc) / ci->stride_w);
      for (int d1 = 0; d1 < ic; ++d1)
        for (int d2 = 0; d2 < oc; ++d2) {
          double dot = 0.0;
          for (int b = 0; b < ci->batch; ++b)
            for (int yr = (int)yr_min; yr < yr_max; ++yr) {
              const int xr = wr + yr * ci->stride_h - ci->pad_top;
              for (int yc = (int)yc_min; yc < yc_max; ++yc) {
                const int xc = wc + yc * ci->stride_w - ci->pad_left;
                dot += (double)x[b * xs.b + xr * xs.row + xc * xs.col + d1 * xs.ch] *
                       (double)dy[b * ys.b + yr * ys.row + yc * ys.col + d2 * ys.ch];
              }
            }
          dw[(((int64_t)wr * fw + wc) * ic + d1) * oc + d2] = (float)dot;
        }
    }
  }
}
void ref_conv2d_der_filter(const float* x, const float* dy, float* dw, const ref_conv2d_info* ci) {
  conv2d_der_filter_strided(x, dy, dw, ci, 0);
}
void ref_conv2d_der_filter_nchw(const float* x, const float* dy, float* dw,
                                const ref_conv2d_info* ci) {
  conv2d_der_filter_strided(x, dy, dw, ci, 1);
}

/* backends/cpu/backend_cpu.ts:2037-2103. */
void ref_depthwise_conv2d_der_input(const float* dy, const float* w, float* dx,
                                    const ref_conv2d_info* ci) {
  const int fh = ci->filter_h, fw = ci->filter_w, ic = ci->in_c, oc = ci->out_c;
  const int ch_mul = oc / ic;
  const int top_pad = fh - 1 - ci->pad_top, left_pad = fw - 1 - ci->pad_left;
  const int64_t x_row = (int64_t)ci->in_w * ic, x_b = x_row * ci->in_h;
  const int64_t y_row = (int64_t)ci->out_w * oc, y_b = y_row * ci->out_h;
  const int64_t w_s0 = (int64_t)fw * ic * ch_mul, w_s1 = (int64_t)ic * ch_mul, w_s2 = ch_mul;
  for (int b = 0; b < ci->batch; ++b)
    for (int d1 = 0; d1 < ic; ++d1)
      for (int xr = 0; xr < ci->in_h; ++xr) {
        const int xr_corner = xr - top_pad;
        const double yr_min = fmax(0.0, ceil((double)xr_corner / ci->stride_h));
        const double yr_max = fmin((double)ci->out_h, (double)(fh + xr_corner) / ci->stride_h);
        for (int xc = 0; xc < ci->in_w; ++xc) {
          const int xc_corner = xc - left_pad;
          const double yc_min = fmax(0.0, ceil((double)xc_corner / ci->stride_w));
          const double yc_max = fmin((double)ci->out_w, (double)(fw + xc_corner) / ci->stride_w);
          double dot = 0.0;
          for (int yr = (int)yr_min; yr < yr_max; ++yr) {
            const int wr = yr * ci->stride_h - xr_corner;
            for (int yc = (int)yc_min; yc < yc_max; ++yc) {
              const int wc = yc * ci->stride_w - xc_corner;
              const float* dyp = dy + b * y_b + yr * y_row + (int64_t)yc * oc;
              const float* wp = w + w_s0 * (fh - 1 - wr) + w_s1 * (fw - 1 - wc) + w_s2 * d1;
              for (int dm = 0; dm < ch_mul; ++dm)
                dot += (double)dyp[d1 * ch_mul + dm] * (double)wp[dm];
            }
          }
          dx[b * x_b + xr * x_row + (int64_t)xc * ic + d1] = (float)dot;
        }
      }
}

/* backends/cpu/backend_cpu.ts:2105-2150. */
void ref_depthwise_conv2d_der_filter(const float* x, const float* dy, float* dw,
                                     const ref_conv2d_info* ci) {
  const int fh = ci->filter_h, fw = ci->filter_w, ic = ci->in_c, oc = ci->out_c;
  const int ch_mul = oc / ic;
  const int64_t x_row = (int64_t)ci->in_w * ic, x_b = x_row * ci->in_h;
  const int64_t y_row = (int64_t)ci->out_w * oc, y_b = y_row * ci->out_h;
  for (int wr = 0; wr < fh; ++wr) {
    const double yr_min = fmax(0.0, ceil((double)(ci->pad_top - wr) / ci->stride_h));
    const double yr_max = fmin((double)ci->out_h, (double)(ci->in_h + ci->pad_top - wr) / ci->stride_h);
    for (int wc = 0; wc < fw; ++wc) {
      const double yc_min = fmax(0.0, ceil((double)(ci->pad_left - wc) / ci->stride_w));
      const double yc_max = fmin((double)ci->out_w, (double)(ci->in_w + ci->pad_left - wc) / ci->stride_w);
      for (int d2 = 0; d2 < oc; ++d2) {
        const int d1 = d2 / ch_mul, dm = d2 % ch_mul;
        double dot = 0.0;
        for (int b = 0; b < ci->batch; ++b)
          for (int yr = (int)yr_min; yr < yr_max; ++yr) {
            const int xr = wr + yr * ci->stride_h - ci->pad_top;
            for (int yc = (int)yc_min; yc < yc_max; ++yc) {
              const int xc = wc + yc * ci->stride_w - ci->pad_left;
              dot += (double)x[b * x_b + xr * x_row + (int64_t)xc * ic + d1] *
                     (double)dy[b * y_b + yr * y_row + (int64_t)yc * oc + d2];
            }
          }
        dw[(((int64_t)wr * fw + wc) * ic + d1) * ch_mul + dm] = (float)dot;
      }
    }
  }
}

/* backends/cpu/backend_cpu.ts:2347-2398: position (within the dilated window, row-major over
 * the effective filter) of the first strict maximum; -1 when nothing beats -inf. */
void ref_max_pool_positions(const float* x, int32_t* pos, const ref_conv2d_info* ci) {
  const int eff_h = ci->filter_h + (ci->filter_h - 1) * (ci->dilation_h - 1);
  const int eff_w = ci->filter_w + (ci->filter_w - 1) * (ci->dilation_w - 1);
  const int64_t x_row = (int64_t)ci->in_w * ci->in_c, x_b = x_row * ci->in_h;
  const int64_t y_row = (int64_t)ci->out_w * ci->out_c, y_b = y_row * ci->out_h;
  for (int b = 0; b < ci->batch; ++b)
    for (int d = 0; d < ci->in_c; ++d)
      for (int yr = 0; yr < ci->out_h; ++yr) {
        const int xr_corner = yr * ci->stride_h - ci->pad_top;
        int xr_min = xr_corner;
        while (xr_min < 0) xr_min += ci->dilation_h;
        const int xr_max = ci->in_h < eff_h + xr_corner ? ci->in_h : eff_h + xr_corner;
        for (int yc = 0; yc < ci->out_w; ++yc) {
          const int xc_corner = yc * ci->stride_w - ci->pad_left;
          int xc_min = xc_corner;
          while (xc_min < 0) xc_min += ci->dilation_w;
          const int xc_max = ci->in_w < eff_w + xc_corner ? ci->in_w : eff_w + xc_corner;
          double max_value = -INFINITY;
          int max_position = -1;
          for (int xr = xr_min; xr < xr_max; xr += ci->dilation_h) {
            const int wr = xr - xr_corner;
            for (int xc = xc_min; xc < xc_max; xc += ci->dilation_w) {
              const int wc = xc - xc_corner;
              const double pixel = (double)x[b * x_b + xr * x_row + (int64_t)xc * ci->in_c + d];
              if (pixel > max_value) {
                max_value = pixel;
                max_position = wr * eff_w + wc;
              }
            }
          }
          pos[b * y_b + yr * y_row + (int64_t)yc * ci->out_c + d] = max_position;
        }
      }
}

/* backends/cpu/backend_cpu.ts:2400-2457 (kind 1, needs x) and :2459-2509 (kind 0: the sum of
 * the dy that cover the pixel times 1 / (filterHeight * filterWidth), whatever part of the
 * window was inside the image). */
void ref_pool2d_backprop(const float* dy, const float* x, float* dx, const ref_conv2d_info* ci,
                         int kind) {
  const int eff_h = ci->filter_h + (ci->filter_h - 1) * (ci->dilation_h - 1);
  const int eff_w = ci->filter_w + (ci->filter_w - 1) * (ci->dilation_w - 1);
  const int pad_left = eff_w - 1 - ci->pad_left, pad_top = eff_h - 1 - ci->pad_top;
  const int64_t x_row = (int64_t)ci->in_w * ci->in_c, x_b = x_row * ci->in_h;
  const int64_t y_row = (int64_t)ci->out_w * ci->out_c, y_b = y_row * ci->out_h;
  const double avg_multiplier = 1.0 / (double)(ci->filter_h * ci->filter_w);
  int32_t* pos = NULL;
  if (kind == 1) {
    pos = (int32_t*)malloc(sizeof(int32_t) * (size_t)(y_b * ci->batch));
    ref_max_pool_positions(x, pos, ci);
  }
  for (int b = 0; b < ci->batch; ++b)
    for (int d = 0; d < ci->in_c; ++d)
      for (int dxr = 0; dxr < ci->in_h; ++dxr)
        for (int dxc = 0; dxc < ci->in_w; ++dxc) {
          const int dyr_corner = dxr - pad_top, dyc_corner = dxc - pad_left;
          double dot = 0.0;
          for (int wr = 0; wr < eff_h; wr += ci->dilation_h) {
            const int num_r = dyr_corner + wr;
            if (num_r < 0 || num_r % ci->stride_h != 0) continue;
            const int dyr = num_r / ci->stride_h;
            if (dyr >= ci->out_h) continue;
            for (int wc = 0; wc < eff_w; wc += ci->dilation_w) {
              const int num_c = dyc_corner + wc;
              if (num_c < 0 || num_c % ci->stride_w != 0) continue;
              const int dyc = num_c / ci->stride_w;
              if (dyc >= ci->out_w) continue;
              const int64_t at = b * y_b + dyr * y_row + (int64_t)dyc * ci->out_c + d;
              if (kind == 1) {
                const int max_pos = eff_h * eff_w - 1 - pos[at];
                if (max_pos != wr * eff_w + wc) continue;
              }
              dot += (double)dy[at];
            }
          }
          dx[b * x_b + dxr * x_row + (int64_t)dxc * ci->in_c + d] =
              (float)(kind == 1 ? dot : dot * avg_multiplier);
        }
  free(pos);
}

/* ---- elementwise ------------------------------------------------------------------- */
enum {
  REF_ADD = 0, REF_SUB, REF_MUL, REF_DIV, REF_PRELU, REF_MAXIMUM, REF_MINIMUM,
  REF_POW, REF_SQUARED_DIFFERENCE, REF_MOD, REF_FLOOR_DIV, REF_ATAN2, REF_ELU_DER
};

/* Math.pow of ECMAScript: a NaN exponent gives NaN (also for base 1), and (+-1) ** +-Infinity
 * is NaN; everything else is C's pow. */
static double js_pow(double a, double b) {
  if (isnan(b)) return NAN;
  if (fabs(a) == 1.0 && isinf(b)) return NAN;
  return pow(a, b);
}

static double binary_eval(int op, double a, double b) {
  switch (op) {
    case REF_ADD: return a + b;                       /* backend_cpu.ts:440-452 */
    case REF_SUB: return a - b;                       /* :469-481 */
    case REF_MUL: return a * b;                       /* :557-572 */
    case REF_DIV: return a / b;                       /* :574-580 */
    case REF_PRELU: return a < 0 ? b * a : a;         /* :1203-1209 */
    case REF_MAXIMUM: return (isnan(a) || isnan(b)) ? NAN : (a > b ? a : b); /* Math.max :931-936 */
    case REF_MINIMUM: return (isnan(a) || isnan(b)) ? NAN : (a < b ? a : b); /* Math.min :886-891 */
    case REF_POW: return js_pow(a, b);                /* :483-489 */
    case REF_SQUARED_DIFFERENCE: return (a - b) * (a - b); /* :984-991 */
    case REF_MOD: {                                   /* :893-904; % is fmod */
      const double rem = fmod(a, b);
      if ((a < 0 && b < 0) || (a >= 0 && b >= 0)) return rem;
      return fmod(rem + b, b);
    }
    case REF_FLOOR_DIV: return floor(a / b);          /* :582-588 */
    case REF_ATAN2: return atan2(a, b);               /* :1425-1431 */
    case REF_ELU_DER: return b >= 1 ? a : a * (b + 1); /* eluDer(dy, y) :1227-1242 */
  }
  return NAN;
}

/* backends/cpu/backend_cpu.ts:3515-3549 with ops/broadcast_util.ts:27-87.  Operands and
 * result are doubles here; the Python wrapper converts from / rounds to the stored dtype
 * (float32 store rounds, Int32Array store truncates).  Shapes are right-aligned. */
int ref_binary(int op, const double* a, const int32_t* a_shape, int a_rank, const double* b,
               const int32_t* b_shape, int b_rank, double* out, const int32_t* out_shape,
               int out_rank) {
  int64_t n = 1, a_len = 1, b_len = 1;
  for (int i = 0; i < out_rank; i++) n *= out_shape[i];
  for (int i = 0; i < a_rank; i++) a_len *= a_shape[i];
  for (int i = 0; i < b_rank; i++) b_len *= b_shape[i];
  /* getBroadcastDims (:27-42): dims of the operand that are 1 where the result is > 1 */
  int a_bc = 0, b_bc = 0;
  for (int i = 0; i < a_rank; i++) {
    const int dim = a_rank - 1 - i, od = out_rank - 1 - i;
    if (a_shape[dim] == 1 && out_shape[od] > 1) a_bc++;
  }
  for (int i = 0; i < b_rank; i++) {
    const int dim = b_rank - 1 - i, od = out_rank - 1 - i;
    if (b_shape[dim] == 1 && out_shape[od] > 1) b_bc++;
  }
  if (a_bc + b_bc == 0) { /* fast path :3526-3530 (what a [C] bias on [...,C] hits) */
    for (int64_t i = 0; i < n; i++) out[i] = binary_eval(op, a[i % a_len], b[i % b_len]);
    return 0;
  }
  int32_t loc[8];
  if (out_rank > 8) return 1;
  for (int64_t i = 0; i < n; i++) {
    int64_t rem = i;
    for (int d = out_rank - 1; d >= 0; d--) {
      loc[d] = (int32_t)(rem % out_shape[d]);
      rem /= out_shape[d];
    }
    int64_t ai = 0, bi = 0, stride = 1;
    for (int d = a_rank - 1; d >= 0; d--) {
      const int od = out_rank - a_rank + d;
      const int32_t c = (a_shape[d] == 1 && out_shape[od] > 1) ? 0 : loc[od];
      ai += c * stride;
      stride *= a_shape[d];
    }
    stride = 1;
    for (int d = b_rank - 1; d >= 0; d--) {
      const int od = out_rank - b_rank + d;
      const int32_t c = (b_shape[d] == 1 && out_shape[od] > 1) ? 0 : loc[od];
      bi += c * stride;
      stride *= b_shape[d];
    }
    out[i] = binary_eval(op, a[ai], b[bi]);
  }
  return 0;
}

enum {
  REF_RELU = 0, REF_CLIP, REF_EXP, REF_LOG, REF_NEG, REF_ABS, REF_SIGMOID, REF_SQRT,
  REF_SQUARE, REF_TANH, REF_RSQRT,
  REF_FLOOR, REF_CEIL, REF_ROUND, REF_SIGN, REF_EXPM1, REF_LOG1P, REF_RECIPROCAL, REF_SIN,
  REF_COS, REF_TAN, REF_ASIN, REF_ACOS, REF_ATAN, REF_SINH, REF_COSH, REF_ASINH, REF_ACOSH,
  REF_ATANH, REF_ERF, REF_ELU, REF_SELU, REF_SOFTPLUS, REF_STEP, REF_IS_NAN, REF_IS_INF,
  REF_IS_FINITE
};

/* backends/cpu/backend_cpu.ts: relu :1191-1201 (Math.max(0,x), NaN-propagating), clip
 * :1265-1275, exp :1094-1103, log :1116-1126, neg :434-438 (multiply by -1), abs
 * :1277-1285, sigmoid :1310-1318, sqrt :1140-1150, square :1164-1174, tanh (util.tanh)
 * :1455-1465, rsqrt :1152-1162.  double libm, one rounding to float at the store. */
void ref_unary(int op, const float* x, float* out, int64_t n, float p0, float p1) {
  for (int64_t i = 0; i < n; i++) {
    const double v = (double)x[i];
    double r;
    switch (op) {
      case REF_RELU: r = isnan(v) ? NAN : (v > 0 ? v : 0); break;
      case REF_CLIP: r = v > (double)p1 ? (double)p1 : (v < (double)p0 ? (double)p0 : v); break;
      case REF_EXP: r = exp(v); break;
      case REF_LOG: r = log(v); break;
      case REF_NEG: r = -v; break;
      case REF_ABS: r = fabs(v); break;
      case REF_SIGMOID: r = 1.0 / (1.0 + exp(-v)); break;
      case REF_SQRT: r = sqrt(v); break;
      case REF_SQUARE: r = v * v; break;
      case REF_TANH: r = tanh(v); break;
      case REF_RSQRT: r = 1.0 / sqrt(v); break;
      case REF_FLOOR: r = floor(v); break;            /* backend_cpu.ts:1004-1013 */
      case REF_CEIL: r = ceil(v); break;              /* :993-1002 */
      case REF_ROUND: {                               /* :1071-1092, banker's rounding */
        const double base = floor(v);
        if (v - base < 0.5) r = floor(v);
        else if (v - base > 0.5) r = ceil(v);
        else r = fmod(base, 2.0) == 0.0 ? base : base + 1.0;
        break;
      }
      case REF_SIGN: r = v < 0 ? -1 : (v > 0 ? 1 : 0); break; /* :1015-1030 */
      case REF_EXPM1: r = expm1(v); break;            /* :1105-1114 */
      case REF_LOG1P: r = log1p(v); break;            /* :1128-1138 */
      case REF_RECIPROCAL: r = 1.0 / v; break;        /* :1176-1185 */
      case REF_SIN: r = sin(v); break;                /* :1359-1368 */
      case REF_COS: r = cos(v); break;                /* :1370-1379 */
      case REF_TAN: r = tan(v); break;                /* :1381-1390 */
      case REF_ASIN: r = asin(v); break;              /* :1392-1401 */
      case REF_ACOS: r = acos(v); break;              /* :1403-1412 */
      case REF_ATAN: r = atan(v); break;              /* :1414-1423 */
      case REF_SINH: r = sinh(v); break;              /* :1433-1442 */
      case REF_COSH: r = cosh(v); break;              /* :1444-1453 */
      case REF_ASINH: r = asinh(v); break;            /* :1466-1475 */
      case REF_ACOSH: r = acosh(v); break;            /* :1477-1486 */
      case REF_ATANH: r = atanh(v); break;            /* :1488-1497 */
      case REF_ERF: {                                 /* :1499-1518, ops/erf_util.ts:18-23 */
        const double p = 0.3275911, a1 = 0.254829592, a2 = -0.284496736, a3 = 1.421413741,
                     a4 = -1.453152027, a5 = 1.061405429;
        const double t = 1.0 / (1.0 + p * v);
        r = 1.0 - (((((a5 * t + a4) * t) + a3) * t + a2) * t + a1) * t * exp(-v * v);
        break;
      }
      case REF_ELU: r = v >= 0 ? v : exp(v) - 1; break; /* :1211-1225 */
      case REF_SELU:                                  /* :1244-1263, ops/selu_util.ts:18-19 */
        r = v >= 0 ? 1.0507009873554804934193349852946 * v
                   : 1.7580993408473768599402175208123 * (exp(v) - 1);
        break;
      case REF_SOFTPLUS: {                            /* :1321-1357 */
        const double threshold = log(1.1920928955078125e-7) + 2.0;
        const double e = exp(v);
        if (v < threshold) r = e;
        else if (v > -threshold) r = v;
        else r = log(1.0 + e);
        break;
      }
      case REF_STEP: r = isnan(v) ? NAN : (v > 0 ? 1 : (double)p0); break; /* :1520-1535 */
      case REF_IS_NAN: r = isnan(v) ? 1 : 0; break;   /* :1032-1043 */
      case REF_IS_INF: r = isinf(v) ? 1 : 0; break;   /* :1045-1056 */
      case REF_IS_FINITE: r = isfinite(v) ? 1 : 0; break; /* :1058-1069 */
      default: r = NAN;
    }
    out[i] = (float)r;
  }
}

/* ---- reductions over the innermost axis ---------------------------------------------- */
enum { REF_SUM = 0, REF_MAX, REF_MIN, REF_ARGMAX, REF_ARGMIN, REF_PROD, REF_ALL, REF_ANY };

/* sum backend_cpu.ts:590-611 (double accumulator, one rounding); max :906-929 and min
 * :861-884 (seeded with element 0, strict compare, so a NaN only survives in slot 0);
 * argMax :686-712 / argMin :658-684 (first index of the strict extremum).  x is read as
 * doubles; out is double (values) — the wrapper rounds / converts. */
void ref_reduce(int op, const double* x, double* out, int64_t outer, int64_t inner) {
  for (int64_t i = 0; i < outer; i++) {
    const double* row = x + i * inner;
    /* prod :613-633 starts at 1; all :938-959 and any :961-982 start from element 0 */
    double acc = (op == REF_SUM) ? 0.0 : (op == REF_PROD) ? 1.0 : row[0];
    int64_t idx = 0;
    for (int64_t j = 0; j < inner; j++) {
      const double v = row[j];
      switch (op) {
        case REF_SUM: acc += v; break;
        case REF_MAX: if (v > acc) acc = v; break;
        case REF_MIN: if (v < acc) acc = v; break;
        case REF_ARGMAX: if (v > acc) { acc = v; idx = j; } break;
        case REF_ARGMIN: if (v < acc) { acc = v; idx = j; } break;
        case REF_PROD: acc *= v; break;
        case REF_ALL: acc = (acc != 0 && !isnan(acc)) ? v : acc; break; /* all = all && value */
        case REF_ANY: acc = (acc != 0 && !isnan(acc)) ? acc : v; break; /* any = any || value */
      }
    }
    out[i] = (op == REF_ARGMAX || op == REF_ARGMIN) ? (double)idx : acc;
  }
}

/* ops/softmax.ts:45-79 + ops/reduction_ops.ts:56-74 as backend_cpu executes them:
 * max -> sub -> exp -> sum -> log -> add -> sub -> exp, every intermediate stored as
 * float32 (the sum accumulates in double and rounds once). */
void ref_softmax_rows(const float* x, float* out, int64_t rows, int64_t cols) {
  float* tmp = (float*)malloc(sizeof(float) * (size_t)(cols > 0 ? cols : 1));
  for (int64_t r = 0; r < rows; r++) {
    const float* row = x + r * cols;
    float mx = row[0];
    for (int64_t j = 0; j < cols; j++) if (row[j] > mx) mx = row[j];
    double s = 0.0;
    for (int64_t j = 0; j < cols; j++) {
      const float a = (float)((double)row[j] - (double)mx);
      tmp[j] = (float)exp((double)a);
      s += (double)tmp[j];
    }
    const float c = (float)s;
    const float d = (float)log((double)c);
    const float lse = (float)((double)mx + (double)d);
    for (int64_t j = 0; j < cols; j++) {
      const float lr = (float)((double)row[j] - (double)lse);
      out[r * cols + j] = (float)exp((double)lr);
    }
  }
  free(tmp);
}

/* ---- data movement ------------------------------------------------------------------- */
/* backends/cpu/backend_cpu.ts:2204-2223 with x viewed as [outer, axis_dim, inner];
 * 4-byte elements copied verbatim. */
void ref_gather(const int32_t* x, const int32_t* indices, int32_t* out, int64_t outer,
                int64_t axis_dim, int64_t inner, int64_t n_idx) {
  for (int64_t o = 0; o < outer; o++)
    for (int64_t i = 0; i < n_idx; i++)
      memcpy(out + (o * n_idx + i) * inner, x + (o * axis_dim + indices[i]) * inner,
             sizeof(int32_t) * (size_t)inner);
}

/* backends/cpu/backend_cpu.ts:2178-2200: newLoc[i] = loc[perm[i]]. */
int ref_transpose(const int32_t* x, const int32_t* shape, int rank, const int32_t* perm,
                  int32_t* out) {
  int32_t new_shape[8], loc[8];
  if (rank > 8) return 1;
  int64_t n = 1;
  for (int i = 0; i < rank; i++) { new_shape[i] = shape[perm[i]]; n *= shape[i]; }
  for (int64_t i = 0; i < n; i++) {
    int64_t rem = i;
    for (int d = rank - 1; d >= 0; d--) { loc[d] = (int32_t)(rem % shape[d]); rem /= shape[d]; }
    int64_t ni = 0;
    for (int d = 0; d < rank; d++) ni = ni * new_shape[d] + loc[perm[d]];
    out[ni] = x[i];
  }
  return 0;
}

/* io/io_utils.ts:122-147, float32 branch: v*scale + min in double, one rounding. */
void ref_dequantize_u8(const uint8_t* q, float* out, int64_t n, double scale, double min) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)((double)q[i] * scale + min);
}
/* the same branch for quantization.dtype 'uint16' (io/io_utils.ts:131-136) */
void ref_dequantize_u16(const uint16_t* q, float* out, int64_t n, double scale, double min) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)((double)q[i] * scale + min);
}

/* backends/cpu/backend_cpu.ts:1299-1308: Int32Array store of a float = ToInt32 (truncate
 * toward zero, NaN/inf -> 0, wrap modulo 2^32). */
void ref_float_to_int(const float* x, int32_t* out, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    const double v = (double)x[i];
    if (isnan(v) || isinf(v)) { out[i] = 0; continue; }
    const double t = trunc(v);
    const double m = fmod(t, 4294967296.0);
    const int64_t w = (int64_t)m;
    out[i] = (int32_t)(uint32_t)(w & 0xffffffffLL);
  }
}
