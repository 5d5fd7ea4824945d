// Row reductions (sum / max / min / argMax / argMin), one-pass row softmax, gather and
// transpose.  Replaces backend_cpu.ts:590-611, 658-712, 861-929, 2178-2223 and the softmax
// composite of ops/softmax.ts:45-79 + ops/reduction_ops.ts:56-74 of the reference.
//
// A row is reduced by one wavefront: lanes stride over the row (coalesced), then combine
// with cross-lane shuffles.  The result is independent of the launch shape, so argMax /
// argMin are deterministic and bit-exact against a sequential scan.
#include "tfhip_internal.h"

namespace tfhip {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float ld(const void* p, int dt, int64_t i) {
  switch (dt) {
    case TFHIP_FLOAT32: return static_cast<const float*>(p)[i];
    case TFHIP_INT32: return (float)static_cast<const int32_t*>(p)[i];
    default: return (float)static_cast<const uint8_t*>(p)[i];
  }
}

constexpr int WAVE = 64;
constexpr int ROWS_PER_BLOCK = 4;  // 4 wavefronts per workgroup, one row each

// max / min follow backend_cpu: the accumulator starts at element 0 and only a strictly
// greater (smaller) value replaces it, so NaN survives only from slot 0.  arg* return the
// first index of the strict extremum; ties and NaN keep the earlier index.
template <typename OutT>
__global__ __launch_bounds__(WAVE* ROWS_PER_BLOCK) void reduce_rows_kernel(
    int op, const void* x, int x_dt, OutT* out, int64_t outer, int64_t inner) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  const int64_t base = row * inner;
  if (op == TFHIP_SUM) {
    double s = 0.0;
    for (int64_t j = lane; j < inner; j += WAVE) s += (double)ld(x, x_dt, base + j);
    for (int off = WAVE / 2; off > 0; off >>= 1) s += __shfl_down(s, off, WAVE);
    if (lane == 0) {
      if (std::is_same<OutT, float>::value) out[row] = (OutT)(float)s;
      else out[row] = (OutT)(int32_t)(uint32_t)(int64_t)s;
    }
    return;
  }
  if (op == TFHIP_PROD) {
    double s = 1.0;
    for (int64_t j = lane; j < inner; j += WAVE) s *= (double)ld(x, x_dt, base + j);
    for (int off = WAVE / 2; off > 0; off >>= 1) s *= __shfl_down(s, off, WAVE);
    if (lane == 0) {
      if (std::is_same<OutT, float>::value) out[row] = (OutT)(float)s;
      else out[row] = (OutT)(int32_t)(uint32_t)(int64_t)s;
    }
    return;
  }
  if (op == TFHIP_ALL || op == TFHIP_ANY) {
    int hit = 0;  // any: a non-zero element; all: a zero element
    for (int64_t j = lane; j < inner; j += WAVE) hit |= (ld(x, x_dt, base + j) != 0.f) == (op == TFHIP_ANY);
    for (int off = WAVE / 2; off > 0; off >>= 1) hit |= __shfl_down(hit, off, WAVE);
    if (lane == 0) out[row] = (OutT)(op == TFHIP_ANY ? hit : !hit);
    return;
  }
  const bool want_max = op == TFHIP_MAX || op == TFHIP_ARGMAX;
  const float first = ld(x, x_dt, base);
  float best = first;
  int64_t idx = 0;
  for (int64_t j = lane; j < inner; j += WAVE) {
    const float v = ld(x, x_dt, base + j);
    if (want_max ? v > best : v < best) {
      best = v;
      idx = j;
    }
  }
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ob = __shfl_down(best, off, WAVE);
    const int64_t oi = __shfl_down(idx, off, WAVE);
    const bool better = want_max ? ob > best : ob < best;
    if (better || (ob == best && oi < idx)) {
      best = ob;
      idx = oi;
    }
  }
  if (lane == 0) {
    if (op == TFHIP_ARGMAX || op == TFHIP_ARGMIN) out[row] = (OutT)idx;
    else if (std::is_same<OutT, float>::value) out[row] = (OutT)best;
    else out[row] = (OutT)(int32_t)best;
  }
}

// Few rows, long rows (a whole tensor summed to a scalar, a global norm, a loss): one wavefront
// per row would leave the machine idle, so every row is cut into `parts` contiguous pieces.  A
// wavefront reduces one piece exactly as reduce_rows_kernel reduces a row and leaves a partial
// result: the running sum / product (double), the any/all flag, or the extremum with the index
// of its first occurrence.  Every piece of a row starts its extremum from the row's element 0,
// as the single pass does, so NaN survives only from slot 0 here too.
__global__ __launch_bounds__(WAVE* ROWS_PER_BLOCK) void reduce_parts_kernel(
    int op, const void* x, int x_dt, double* pval, long long* pidx, int64_t outer, int64_t inner,
    int parts, int64_t seg, int vec) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t piece = (int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (piece >= outer * parts) return;
  const int64_t row = piece / parts;
  const int part = (int)(piece - row * parts);
  const int64_t base = row * inner;
  const int64_t j0 = part * seg, j1 = min(inner, j0 + seg);
  // four independent loads per lane and trip keep enough bytes in flight for the HBM rate
  constexpr int U = 4;
  if (op == TFHIP_SUM || op == TFHIP_PROD) {
    const bool sum = op == TFHIP_SUM;
    double s[U];
#pragma unroll
    for (int u = 0; u < U; u++) s[u] = sum ? 0.0 : 1.0;
    int64_t j = j0 + lane;
    if (vec) {
      // float32 rows whose pieces start on 16-byte boundaries: 16 bytes per lane and load
      const f32x4* xv = reinterpret_cast<const f32x4*>(static_cast<const float*>(x) + base);
      int64_t q = j0 / 4 + lane;
      const int64_t q1 = j1 / 4;
      for (; q + (U - 1) * WAVE < q1; q += U * WAVE) {
        f32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = xv[q + u * WAVE];
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
          for (int e = 0; e < 4; e++) s[u] = sum ? s[u] + (double)v[u][e] : s[u] * (double)v[u][e];
      }
      for (; q < q1; q += WAVE) {
        const f32x4 v = xv[q];
#pragma unroll
        for (int e = 0; e < 4; e++) s[0] = sum ? s[0] + (double)v[e] : s[0] * (double)v[e];
      }
      j = q1 * 4 + lane;  // what is left of a row whose length is no multiple of 4
    }
    for (; j + (U - 1) * WAVE < j1; j += U * WAVE) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; u++) v[u] = ld(x, x_dt, base + j + u * WAVE);
#pragma unroll
      for (int u = 0; u < U; u++) s[u] = sum ? s[u] + (double)v[u] : s[u] * (double)v[u];
    }
    for (; j < j1; j += WAVE) s[0] = sum ? s[0] + (double)ld(x, x_dt, base + j) : s[0] * (double)ld(x, x_dt, base + j);
    double t = sum ? (s[0] + s[1]) + (s[2] + s[3]) : (s[0] * s[1]) * (s[2] * s[3]);
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const double o = __shfl_down(t, off, WAVE);
      t = sum ? t + o : t * o;
    }
    if (lane == 0) pval[piece] = t;
    return;
  }
  if (op == TFHIP_ALL || op == TFHIP_ANY) {
    int hit = 0;  // any: a non-zero element; all: a zero element
    for (int64_t j = j0 + lane; j < j1; j += WAVE) hit |= (ld(x, x_dt, base + j) != 0.f) == (op == TFHIP_ANY);
    for (int off = WAVE / 2; off > 0; off >>= 1) hit |= __shfl_down(hit, off, WAVE);
    if (lane == 0) pval[piece] = (double)hit;
    return;
  }
  const bool want_max = op == TFHIP_MAX || op == TFHIP_ARGMAX;
  float best = ld(x, x_dt, base);
  int64_t idx = 0;
  int64_t j = j0 + lane;
  if (vec) {
    const f32x4* xv = reinterpret_cast<const f32x4*>(static_cast<const float*>(x) + base);
    int64_t q = j0 / 4 + lane;
    const int64_t q1 = j1 / 4;
    for (; q < q1; q += U * WAVE) {
      f32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; u++) v[u] = q + u * WAVE < q1 ? xv[q + u * WAVE] : f32x4{best, best, best, best};
      // in ascending index order within the lane, so that of equal values the first is kept
#pragma unroll
      for (int u = 0; u < U; u++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (want_max ? v[u][e] > best : v[u][e] < best) {
            best = v[u][e];
            idx = 4 * (q + u * WAVE) + e;
          }
    }
    j = q1 * 4 + lane;
  }
  for (; j + (U - 1) * WAVE < j1; j += U * WAVE) {
    float v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = ld(x, x_dt, base + j + u * WAVE);
#pragma unroll
    for (int u = 0; u < U; u++)
      if (want_max ? v[u] > best : v[u] < best) {
        best = v[u];
        idx = j + u * WAVE;
      }
  }
  for (; j < j1; j += WAVE) {
    const float v = ld(x, x_dt, base + j);
    if (want_max ? v > best : v < best) {
      best = v;
      idx = j;
    }
  }
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ob = __shfl_down(best, off, WAVE);
    const int64_t oi = __shfl_down(idx, off, WAVE);
    const bool better = want_max ? ob > best : ob < best;
    if (better || (ob == best && oi < idx)) {
      best = ob;
      idx = oi;
    }
  }
  if (lane == 0) {
    pval[piece] = (double)best;
    pidx[piece] = idx;
  }
}

// Combines the partial results of every row, one wavefront per row, with the same rules (sums
// in double; a later piece wins an extremum only when strictly better, equal values keep the
// lower index), so the result does not depend on how the row was cut.
template <typename OutT>
__global__ __launch_bounds__(WAVE* ROWS_PER_BLOCK) void reduce_finish_kernel(
    int op, const double* pval, const long long* pidx, OutT* out, int64_t outer, int parts) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= outer) return;
  const double* pv = pval + row * parts;
  if (op == TFHIP_SUM || op == TFHIP_PROD) {
    const bool sum = op == TFHIP_SUM;
    double s = sum ? 0.0 : 1.0;
    for (int k = lane; k < parts; k += WAVE) s = sum ? s + pv[k] : s * pv[k];
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const double o = __shfl_down(s, off, WAVE);
      s = sum ? s + o : s * o;
    }
    if (lane == 0) {
      if (std::is_same<OutT, float>::value) out[row] = (OutT)(float)s;
      else out[row] = (OutT)(int32_t)(uint32_t)(int64_t)s;
    }
    return;
  }
  if (op == TFHIP_ALL || op == TFHIP_ANY) {
    int hit = 0;
    for (int k = lane; k < parts; k += WAVE) hit |= pv[k] != 0.0;
    for (int off = WAVE / 2; off > 0; off >>= 1) hit |= __shfl_down(hit, off, WAVE);
    if (lane == 0) out[row] = (OutT)(op == TFHIP_ANY ? hit : !hit);
    return;
  }
  const bool want_max = op == TFHIP_MAX || op == TFHIP_ARGMAX;
  const long long* pi = pidx + row * parts;
  float best = (float)pv[0];
  int64_t idx = pi[0];
  for (int k = lane; k < parts; k += WAVE) {
    const float v = (float)pv[k];
    const int64_t vi = pi[k];
    if ((want_max ? v > best : v < best) || (v == best && vi < idx)) {
      best = v;
      idx = vi;
    }
  }
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ob = __shfl_down(best, off, WAVE);
    const int64_t oi = __shfl_down(idx, off, WAVE);
    const bool better = want_max ? ob > best : ob < best;
    if (better || (ob == best && oi < idx)) {
      best = ob;
      idx = oi;
    }
  }
  if (lane == 0) {
    if (op == TFHIP_ARGMAX || op == TFHIP_ARGMIN) out[row] = (OutT)idx;
    else if (std::is_same<OutT, float>::value) out[row] = (OutT)best;
    else out[row] = (OutT)(int32_t)best;
  }
}

// softmax over the last axis with the rounding points of the reference composite:
// m = max(x); e = exp(x - m); s = sum(e); lse = m + log(s); y = exp(x - lse).
// SLOTS > 0: the row fits SLOTS registers per lane (cols <= 64 * SLOTS): one pass over
// memory with all loads in flight.  SLOTS == 0: any length, three passes.
template <int SLOTS>
__global__ __launch_bounds__(WAVE* ROWS_PER_BLOCK) void softmax_rows_kernel(
    const float* x, float* y, int64_t rows, int64_t cols) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* xr = x + row * cols;
  float* yr = y + row * cols;
  float m = xr[0];
  if (SLOTS > 0) {
    constexpr int S = SLOTS > 0 ? SLOTS : 1;
    float v[S];
#pragma unroll
    for (int i = 0; i < S; i++) {
      const int64_t j = lane + i * WAVE;
      v[i] = xr[j < cols ? j : 0];
    }
#pragma unroll
    for (int i = 0; i < S; i++)
      if (v[i] > m) m = v[i];
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const float o = __shfl_xor(m, off, WAVE);
      if (o > m) m = o;
    }
    double s = 0.0;
#pragma unroll
    for (int i = 0; i < S; i++)
      if (lane + i * WAVE < cols) s += (double)expf(v[i] - m);
    for (int off = WAVE / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, WAVE);
    const float lse = m + logf((float)s);
#pragma unroll
    for (int i = 0; i < S; i++)
      if (lane + i * WAVE < cols) yr[lane + i * WAVE] = expf(v[i] - lse);
    return;
  }
  for (int64_t j = lane; j < cols; j += WAVE) {
    const float v = xr[j];
    if (v > m) m = v;
  }
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float o = __shfl_xor(m, off, WAVE);
    if (o > m) m = o;
  }
  // a NaN in slot 0 makes every lane's m NaN already (all start from xr[0])
  double s = 0.0;
  for (int64_t j = lane; j < cols; j += WAVE) s += (double)expf(xr[j] - m);
  for (int off = WAVE / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, WAVE);
  const float lse = m + logf((float)s);
  for (int64_t j = lane; j < cols; j += WAVE) yr[j] = expf(xr[j] - lse);
}

// cumsum along the innermost axis (backend_cpu.ts:714-745): one wavefront per row walks the row
// 64 elements at a time, a shuffle scan inside the group and a running carry between groups.
// Floats are summed in double and rounded once per element, int32 wraps like Int32Array.
template <typename OutT>
__global__ __launch_bounds__(WAVE* ROWS_PER_BLOCK) void cumsum_rows_kernel(
    const void* x, int x_dt, OutT* out, int64_t rows, int64_t cols, int exclusive, int reverse) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int64_t base = row * cols;
  double carry = 0.0;
  for (int64_t j0 = 0; j0 < cols; j0 += WAVE) {
    const int64_t j = j0 + lane;                       // position along the scan direction
    const int64_t at = base + (reverse ? cols - 1 - j : j);
    const double v = j < cols ? (double)ld(x, x_dt, at) : 0.0;
    double s = v;
    for (int off = 1; off < WAVE; off <<= 1) {
      const double o = __shfl_up(s, off, WAVE);
      if (lane >= off) s += o;
    }
    const double incl = carry + s;
    const double r = exclusive ? incl - v : incl;
    if (j < cols) {
      if (std::is_same<OutT, float>::value) out[at] = (OutT)(float)r;
      else out[at] = (OutT)(int32_t)(uint32_t)(int64_t)r;
    }
    carry = __shfl(incl, WAVE - 1, WAVE);
  }
}

// topk along the innermost axis (backends/topk_impl.ts:25-60: a stable sort by descending value,
// so equal values keep ascending index order).  One wavefront per row selects the k entries one
// after the other: entry i is the largest element that comes after entry i-1 in that order
// (smaller value, or equal value and larger index); ties go to the smallest index.  k passes over
// the row, which stays in L1/L2; NaN elements are never selected (JavaScript's comparator leaves
// their place unspecified) and rows that run out of candidates repeat index -1 / value NaN.
template <typename T>
__global__ __launch_bounds__(WAVE* ROWS_PER_BLOCK) void topk_rows_kernel(
    const T* __restrict__ x, T* __restrict__ values, int32_t* __restrict__ indices, int64_t rows,
    int64_t cols, int k) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * cols;
  bool have_prev = false;
  T prev_v = T(0);
  int64_t prev_i = -1;
  bool exhausted = false;  // (the same for every lane)
  for (int out = 0; out < k; out++) {
    bool found = false;
    T best = T(0);
    int64_t best_i = cols;
    for (int64_t j = lane; j < cols && !exhausted; j += WAVE) {
      const T v = xr[j];
      if (v != v) continue;
      if (have_prev && !(v < prev_v || (v == prev_v && j > prev_i))) continue;
      if (!found || v > best) {  // ascending j within a lane: the first of equal values stays
        best = v;
        best_i = j;
        found = true;
      }
    }
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const T ob = __shfl_xor(best, off, WAVE);
      const int64_t oi = __shfl_xor(best_i, off, WAVE);
      const int of = __shfl_xor((int)found, off, WAVE);
      if (of && (!found || ob > best || (ob == best && oi < best_i))) {
        best = ob;
        best_i = oi;
        found = true;
      }
    }
    if (lane == 0) {
      values[row * k + out] = found ? best : (T)NAN;
      indices[row * k + out] = found ? (int32_t)best_i : -1;
    }
    have_prev = true;
    prev_v = best;
    prev_i = best_i;
    exhausted = !found;
  }
}

// out[o, i, :] = x[o, indices[i], :] for 4-byte or 1-byte elements.
template <typename T>
__global__ void gather_kernel(const T* x, const int32_t* indices, T* out, int64_t outer,
                              int64_t axis_dim, int64_t inner, int64_t n_idx) {
  const int64_t total = outer * n_idx * inner;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
    const int64_t in = g % inner;
    const int64_t t = g / inner;
    const int64_t i = t % n_idx, o = t / n_idx;
    const int64_t src = indices[i];
    // an index outside the axis reads nothing (the reference would yield undefined)
    out[g] = (src >= 0 && src < axis_dim) ? x[(o * axis_dim + src) * inner + in] : T(0);
  }
}

constexpr int MAXR = 6;
struct PermArgs {
  int rank;
  int out_dim[MAXR];
  int64_t in_stride[MAXR];  // stride in x of the dimension that lands on out dim d
};

template <typename T>
__global__ void transpose_kernel(const T* x, T* out, int64_t n, PermArgs pa) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < n; g += stride) {
    int64_t rem = g, src = 0;
#pragma unroll
    for (int d = MAXR - 1; d >= 0; d--) {
      if (d < pa.rank) {
        src += (rem % pa.out_dim[d]) * pa.in_stride[d];
        rem /= pa.out_dim[d];
      }
    }
    out[g] = x[src];
  }
}

static unsigned grid_cap(tfhip_ctx* ctx, int64_t items, int block) {
  const int64_t want = ceil_div(items, block), cap = (int64_t)ctx->num_cus * 16;
  return (unsigned)(want < 1 ? 1 : (want > cap ? cap : want));
}

}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_reduce(tfhip_ctx* ctx, int op, int64_t x, int64_t out, int64_t outer,
                            int64_t inner) {
  if (!ctx) return TFHIP_EINVAL;
  if (op < TFHIP_SUM || op > TFHIP_ANY) return ctx->fail(TFHIP_EINVAL, "reduce: unknown op %d", op);
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (outer < 0 || inner < 0 || bx->numel != outer * inner || bo->numel != outer)
    return ctx->fail(TFHIP_EINVAL, "reduce: buffers hold %lld and %lld elements, need %lld and %lld",
                     (long long)bx->numel, (long long)bo->numel, (long long)(outer * inner),
                     (long long)outer);
  if (bx->dtype == TFHIP_UINT8Q) return ctx->fail(TFHIP_EINVAL, "reduce: quantised input");
  const bool arg = op == TFHIP_ARGMAX || op == TFHIP_ARGMIN;
  if (arg && bo->dtype != TFHIP_INT32)
    return ctx->fail(TFHIP_EINVAL, "reduce: argMax/argMin write int32");
  const bool logical = op == TFHIP_ALL || op == TFHIP_ANY;
  if (logical ? bo->dtype != TFHIP_BOOL : (bo->dtype != TFHIP_INT32 && bo->dtype != TFHIP_FLOAT32))
    return ctx->fail(TFHIP_EINVAL, "reduce: output must be float32 or int32 (bool for all/any)");
  if (outer == 0) return TFHIP_OK;
  if (inner == 0) {
    if (op == TFHIP_PROD) return tfhip_fill(ctx, out, 1.0);
    if (op != TFHIP_SUM) return ctx->fail(TFHIP_EINVAL, "reduce: empty axis has no extremum");
    return tfhip_fill(ctx, out, 0.0);
  }
  if (ceil_div(outer, ROWS_PER_BLOCK) > 0x7fffffffLL) return ctx->fail(TFHIP_ENOTSUP, "reduce: too many rows");
  const dim3 block(WAVE * ROWS_PER_BLOCK);
  // Fewer rows than the machine has room for wavefronts, and rows long enough to be worth a
  // second launch: cut every row into pieces, reduce the pieces, then combine them.
  const int64_t room = (int64_t)ctx->num_cus * 16;
  if (outer * 2 <= room && inner >= 16384 && !ctx->no_alloc) {
    const int64_t min_piece = 4096;
    int64_t parts = std::min<int64_t>(ceil_div(room, outer), ceil_div(inner, min_piece));
    parts = std::min<int64_t>(parts, 4096);
    const int64_t seg = ceil_div(ceil_div(inner, parts), WAVE) * WAVE;  // whole trips of a wavefront
    parts = ceil_div(inner, seg);
    if (parts > 1) {
      const int64_t pieces = outer * parts;
      Temp partial(ctx);
      if (!partial.get((size_t)pieces * 16)) return TFHIP_EDEVICE;
      // 16-byte loads: float32, every row and (seg is a multiple of 64) every piece 16-byte aligned
      const int vec = bx->dtype == TFHIP_FLOAT32 && inner % 4 == 0 &&
                      (reinterpret_cast<uintptr_t>(bx->ptr) & 15) == 0;
      double* pval = static_cast<double*>(partial.ptr);
      long long* pidx = reinterpret_cast<long long*>(pval + pieces);
      tfhip::launch(ctx, reduce_parts_kernel, dim3((unsigned)ceil_div(pieces, ROWS_PER_BLOCK)), block, 0,
                    op, bx->ptr, bx->dtype, pval, pidx, outer, inner, (int)parts, seg, vec);
      TFHIP_LAUNCH_CHECK_NAMED(ctx, "reduce_parts");
      const dim3 fgrid((unsigned)ceil_div(outer, ROWS_PER_BLOCK));
      if (bo->dtype == TFHIP_FLOAT32)
        tfhip::launch(ctx, reduce_finish_kernel<float>, fgrid, block, 0, op, pval, pidx,
                      (float*)bo->ptr, outer, (int)parts);
      else if (bo->dtype == TFHIP_BOOL)
        tfhip::launch(ctx, reduce_finish_kernel<uint8_t>, fgrid, block, 0, op, pval, pidx,
                      (uint8_t*)bo->ptr, outer, (int)parts);
      else
        tfhip::launch(ctx, reduce_finish_kernel<int32_t>, fgrid, block, 0, op, pval, pidx,
                      (int32_t*)bo->ptr, outer, (int)parts);
      TFHIP_LAUNCH_CHECK_NAMED(ctx, "reduce_finish");
      return TFHIP_OK;
    }
  }
  const dim3 grid((unsigned)ceil_div(outer, ROWS_PER_BLOCK));
  if (bo->dtype == TFHIP_FLOAT32)
    tfhip::launch(ctx, reduce_rows_kernel<float>, grid, block, 0, op, bx->ptr,
                       bx->dtype, (float*)bo->ptr, outer, inner);
  else if (bo->dtype == TFHIP_BOOL)
    tfhip::launch(ctx, reduce_rows_kernel<uint8_t>, grid, block, 0, op, bx->ptr,
                       bx->dtype, (uint8_t*)bo->ptr, outer, inner);
  else
    tfhip::launch(ctx, reduce_rows_kernel<int32_t>, grid, block, 0, op, bx->ptr,
                       bx->dtype, (int32_t*)bo->ptr, outer, inner);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_softmax_rows(tfhip_ctx* ctx, int64_t x, int64_t out, int64_t rows,
                                  int64_t cols) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (rows < 0 || cols < 0 || bx->numel != rows * cols || bo->numel != rows * cols)
    return ctx->fail(TFHIP_EINVAL, "softmax: buffer sizes do not match rows x cols");
  if (bo->dtype != TFHIP_FLOAT32) return ctx->fail(TFHIP_EINVAL, "softmax: output must be float32");
  if (rows * cols == 0) return TFHIP_OK;
  Temp tx(ctx);
  const float* xf;
  int rc;
  if ((rc = as_f32(ctx, bx, &tx, &xf))) return rc;
  const dim3 grid((unsigned)ceil_div(rows, ROWS_PER_BLOCK)), block(WAVE * ROWS_PER_BLOCK);
  float* yf = static_cast<float*>(bo->ptr);
  if (cols <= WAVE)
    tfhip::launch(ctx, softmax_rows_kernel<1>, grid, block, 0, xf, yf, rows, cols);
  else if (cols <= WAVE * 4)
    tfhip::launch(ctx, softmax_rows_kernel<4>, grid, block, 0, xf, yf, rows, cols);
  else if (cols <= WAVE * 16)
    tfhip::launch(ctx, softmax_rows_kernel<16>, grid, block, 0, xf, yf, rows, cols);
  else
    tfhip::launch(ctx, softmax_rows_kernel<0>, grid, block, 0, xf, yf, rows, cols);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_gather(tfhip_ctx* ctx, int64_t x, int64_t indices, int64_t out,
                            int64_t outer, int64_t axis_dim, int64_t inner, int64_t n_indices) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bi, indices);
  TFHIP_GET(ctx, bo, out);
  if (outer < 0 || axis_dim < 0 || inner < 0 || n_indices < 0 ||
      bx->numel != outer * axis_dim * inner || bi->numel != n_indices ||
      bo->numel != outer * n_indices * inner)
    return ctx->fail(TFHIP_EINVAL, "gather: buffer sizes do not match the shapes given");
  if (bi->dtype != TFHIP_INT32) return ctx->fail(TFHIP_EINVAL, "gather: indices must be int32");
  if (dtype_size(bx->dtype) != dtype_size(bo->dtype))
    return ctx->fail(TFHIP_EINVAL, "gather: input and output element sizes differ");
  const int64_t total = bo->numel;
  if (total == 0) return TFHIP_OK;
  const dim3 grid(grid_cap(ctx, total, 256)), block(256);
  if (dtype_size(bx->dtype) == 4)
    tfhip::launch(ctx, gather_kernel<int32_t>, grid, block, 0, (const int32_t*)bx->ptr,
                       (const int32_t*)bi->ptr, (int32_t*)bo->ptr, outer, axis_dim, inner, n_indices);
  else
    tfhip::launch(ctx, gather_kernel<uint8_t>, grid, block, 0, (const uint8_t*)bx->ptr,
                       (const int32_t*)bi->ptr, (uint8_t*)bo->ptr, outer, axis_dim, inner, n_indices);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_transpose(tfhip_ctx* ctx, int64_t x, const int32_t* x_shape, int rank,
                               const int32_t* perm, int64_t out) {
  if (!ctx) return TFHIP_EINVAL;
  if (rank < 0 || rank > MAXR) return ctx->fail(TFHIP_ENOTSUP, "transpose: rank above %d", MAXR);
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  int64_t n = 1, strides[MAXR];
  bool seen[MAXR] = {false};
  for (int i = rank - 1; i >= 0; i--) {
    strides[i] = n;
    n *= x_shape[i];
  }
  PermArgs pa = {};
  pa.rank = rank;
  for (int d = 0; d < rank; d++) {
    const int s = perm[d];
    if (s < 0 || s >= rank || seen[s]) return ctx->fail(TFHIP_EINVAL, "transpose: bad permutation");
    seen[s] = true;
    pa.out_dim[d] = x_shape[s];  // newShape[i] = x.shape[perm[i]] (backend_cpu.ts:2181-2184)
    pa.in_stride[d] = strides[s];
  }
  if (bx->numel != n || bo->numel != n || dtype_size(bx->dtype) != dtype_size(bo->dtype))
    return ctx->fail(TFHIP_EINVAL, "transpose: buffer sizes do not match the shape given");
  if (n == 0) return TFHIP_OK;
  const dim3 grid(grid_cap(ctx, n, 256)), block(256);
  if (dtype_size(bx->dtype) == 4)
    tfhip::launch(ctx, transpose_kernel<int32_t>, grid, block, 0,
                       (const int32_t*)bx->ptr, (int32_t*)bo->ptr, n, pa);
  else
    tfhip::launch(ctx, transpose_kernel<uint8_t>, grid, block, 0,
                       (const uint8_t*)bx->ptr, (uint8_t*)bo->ptr, n, pa);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_cumsum(tfhip_ctx* ctx, int64_t x, int64_t out, int64_t outer, int64_t inner,
                            int exclusive, int reverse) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bo, out);
  if (outer < 0 || inner < 0 || bx->numel != outer * inner || bo->numel != outer * inner)
    return ctx->fail(TFHIP_EINVAL, "cumsum: buffers hold %lld and %lld elements, need %lld",
                     (long long)bx->numel, (long long)bo->numel, (long long)(outer * inner));
  if (bx->dtype == TFHIP_UINT8Q || (bo->dtype != TFHIP_FLOAT32 && bo->dtype != TFHIP_INT32))
    return ctx->fail(TFHIP_EINVAL, "cumsum: output must be float32 or int32");
  if (outer * inner == 0) return TFHIP_OK;
  if (ceil_div(outer, ROWS_PER_BLOCK) > 0x7fffffffLL) return ctx->fail(TFHIP_ENOTSUP, "cumsum: too many rows");
  const dim3 grid((unsigned)ceil_div(outer, ROWS_PER_BLOCK)), block(WAVE * ROWS_PER_BLOCK);
  if (bo->dtype == TFHIP_FLOAT32)
    tfhip::launch(ctx, cumsum_rows_kernel<float>, grid, block, 0, bx->ptr, bx->dtype,
                       (float*)bo->ptr, outer, inner, exclusive, reverse);
  else
    tfhip::launch(ctx, cumsum_rows_kernel<int32_t>, grid, block, 0, bx->ptr, bx->dtype,
                       (int32_t*)bo->ptr, outer, inner, exclusive, reverse);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

extern "C" int tfhip_topk(tfhip_ctx* ctx, int64_t x, int64_t values, int64_t indices, int64_t rows,
                          int64_t cols, int k) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bv, values);
  TFHIP_GET(ctx, bi, indices);
  if (rows < 0 || cols < 0 || k < 0 || k > cols)
    return ctx->fail(TFHIP_EINVAL, "'k' passed to topk() must be <= the last dimension (%lld) but got %d",
                     (long long)cols, k);
  if (bx->numel != rows * cols || bv->numel != rows * k || bi->numel != rows * k)
    return ctx->fail(TFHIP_EINVAL, "topk: buffer sizes do not match rows x cols and rows x k");
  if ((bx->dtype != TFHIP_FLOAT32 && bx->dtype != TFHIP_INT32) || bv->dtype != bx->dtype ||
      bi->dtype != TFHIP_INT32)
    return ctx->fail(TFHIP_EINVAL, "topk: values keep x's dtype (float32 or int32), indices are int32");
  if (rows * k == 0) return TFHIP_OK;
  if (ceil_div(rows, ROWS_PER_BLOCK) > 0x7fffffffLL) return ctx->fail(TFHIP_ENOTSUP, "topk: too many rows");
  const dim3 grid((unsigned)ceil_div(rows, ROWS_PER_BLOCK)), block(WAVE * ROWS_PER_BLOCK);
  if (bx->dtype == TFHIP_FLOAT32)
    tfhip::launch(ctx, topk_rows_kernel<float>, grid, block, 0, (const float*)bx->ptr,
                       (float*)bv->ptr, (int32_t*)bi->ptr, rows, cols, k);
  else
    tfhip::launch(ctx, topk_rows_kernel<int32_t>, grid, block, 0, (const int32_t*)bx->ptr,
                       (int32_t*)bv->ptr, (int32_t*)bi->ptr, rows, cols, k);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}
