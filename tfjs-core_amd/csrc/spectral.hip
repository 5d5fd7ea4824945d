// Discrete Fourier transform of rows of complex numbers: fft / ifft of the reference
// (backend.ts:618-622; backend_cpu.ts:3343-3467).  Complex tensors are float32 buffers of
// interleaved (real, imaginary) pairs, the layout the reference's readSync returns
// (backend_cpu.ts:214-223, backends/complex_util.ts:30-44).
//
// One lane per output coefficient: out[row, k] = sum_j x[row, j] * exp(-+ 2 pi i j k / n),
// accumulated in double with the twiddle angle reduced modulo n first, so the result is the
// correctly rounded transform to well within float32 for any n (the reference's radix-2 path
// rounds to float32 after every butterfly, its general path after every term).  The lanes of
// a wavefront read the same x[row, j] at the same time, so the row comes out of L1 / L2; the
// work is O(n^2) per row, which is what the reference's general path costs too.
#include "tfhip_internal.h"

namespace tfhip {

__global__ void dft_rows_kernel(const float* __restrict__ x, float* __restrict__ out, int64_t batch,
                                int64_t n, int inverse) {
  const int64_t total = batch * n;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const double sign = inverse ? 2.0 : -2.0;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
    const int64_t row = g / n, k = g - row * n;
    const float* xr = x + row * n * 2;
    double re = 0.0, im = 0.0;
    int64_t m = 0;  // (j * k) mod n, stepped instead of multiplied
    for (int64_t j = 0; j < n; j++) {
      double s, c;
      sincospi(sign * (double)m / (double)n, &s, &c);
      const double a = xr[2 * j], b = xr[2 * j + 1];
      re += a * c - b * s;
      im += a * s + b * c;
      m += k;
      if (m >= n) m -= n;
    }
    if (inverse) {
      re /= (double)n;
      im /= (double)n;
    }
    out[2 * g] = (float)re;
    out[2 * g + 1] = (float)im;
  }
}

}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_fft(tfhip_ctx* ctx, int64_t x, int64_t out, int64_t batch, int64_t n,
                         int inverse) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (batch < 0 || n < 0) return ctx->fail(TFHIP_EINVAL, "fft: bad geometry");
  if (bx->dtype != TFHIP_FLOAT32 || bo->dtype != TFHIP_FLOAT32 || bx->numel != batch * n * 2 ||
      bo->numel != batch * n * 2)
    return ctx->fail(TFHIP_EINVAL, "fft: input and result are float32 buffers of batch x n (real, imaginary) pairs");
  if (bx->ptr == bo->ptr && bo->numel) return ctx->fail(TFHIP_EINVAL, "fft: the transform is not in place");
  if (bo->numel == 0) return TFHIP_OK;
  const int64_t blocks = (batch * n + 255) / 256, cap = (int64_t)ctx->num_cus * 16;
  tfhip::launch(ctx, dft_rows_kernel, dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(256), 0,
                     (const float*)bx->ptr, (float*)bo->ptr, batch, n, inverse ? 1 : 0);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}
