// Dense contractions on the fp32 matrix cores of gfx950: batchMatMul / fusedBatchMatMul
// and conv2d / fusedConv2d (implicit GEMM over NHWC), with bias + activation in the
// epilogue and optional uint8 affine-quantised weights dequantised while the B tile is
// staged.  Replaces backend_cpu.ts:491-555 and :1536-1616 of the reference.
//
// Kernel shape.  A workgroup of WAVES_M x WAVES_N wavefronts (64 lanes each) owns a
// BM x BN tile of the result, BM = WAVES_M*TM*32, BN = WAVES_N*TN*32; every wavefront
// holds TM x TN accumulators of v_mfma_f32_32x32x2f32 (16 VGPRs each).  The K loop walks
// BK = 16 columns at a time through two LDS buffers: while the matrix cores work on tile
// t out of LDS, the global loads of tile t+1 are in flight into registers, and one barrier
// per step hands the buffers over.
//
// LDS layout.  A is kept [row][k] with a row pitch of BK+4 floats so that a lane fetches
// four consecutive k of its row with one 16-byte read; B is kept [k][col].  The MFMA
// wants lane l to supply k = l/32, so within a group of 8 k the lanes 0..31 take
// k = 0..3 and lanes 32..63 take k = 4..7, and MFMA number r of the group multiplies
// k = r (low half) with k = 4+r (high half): a permutation of the summation order only.
// Likewise lane j of accumulator tile tj owns column TN*j + tj, so a lane reads its TN B
// values with one access and writes TN adjacent results.
#include <type_traits>

#include "tfhip_internal.h"

namespace tfhip {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { A_ROWMAJOR = 0, A_TRANSPOSED = 1, A_IM2COL = 2 };
enum { B_ROWMAJOR = 0, B_TRANSPOSED = 1, B_UINT8 = 2 };

struct GemmArgs {
  const float* A;
  const void* B;
  float* C;
  const float* bias;
  const float* prelu;
  int M, N, K;
  int lda, ldb;
  long long strideA, strideB, strideC;  // per-batch element strides
  int bias_kind, prelu_kind, act;
  int a_vec, b_vec;  // operands allow aligned 4-element accesses
  // implicit-GEMM geometry (A_IM2COL): rows are (n, oh, ow), k is (kh, kw, c)
  int H, W, Cin, OH, OW, KH, KW, sh, sw, dh, dw, pt, pl;
  double qscale, qmin;
  int tiles_m, tiles_n;
};

constexpr int BK = 16;
constexpr int LDA_S = BK + 4;
constexpr int TILES_PER_KBLOCK = 48 / BK;

// w = q*scale + min evaluated in double, rounded once (io/io_utils.ts:133-136).
__device__ __forceinline__ float dequant(unsigned q, double scale, double mn) {
#pragma clang fp contract(off)
  double v = (double)q * scale;
  v = v + mn;
  return (float)v;
}

// Activation of the reference (backend_cpu.ts:50-62) with JavaScript's NaN behaviour:
// Math.max(0, NaN) is NaN (:1191-1201), clip keeps NaN (:1265-1275).
__device__ __forceinline__ float activate(float v, int act, float alpha) {
  switch (act) {
    case TFHIP_ACT_RELU: return (v > 0.f || v != v) ? v : 0.f;
    case TFHIP_ACT_RELU6: return v > 6.f ? 6.f : (v < 0.f ? 0.f : v);
    case TFHIP_ACT_PRELU: return v < 0.f ? alpha * v : v;
    default: return v;
  }
}

// Workgroups are handed to the 8 XCDs round-robin by linear id; remap so that each XCD
// (own L2) receives a contiguous run of tiles, i.e. neighbours that share A rows / B
// columns hit the same L2.
__device__ __forceinline__ int xcd_remap(int bid, int total) {
  constexpr int XCDS = 8;
  const int per = total / XCDS, rem = total % XCDS;
  const int x = bid % XCDS, i = bid / XCDS;
  // XCD x owns `per` tiles (+1 for the first `rem` XCDs)
  const int start = x * per + (x < rem ? x : rem);
  return start + i;
}

template <int WAVES_M, int WAVES_N, int TM, int TN, int AMODE, int BMODE, bool KBLOCKED>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_kernel(const GemmArgs p) {
  constexpr int THREADS = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * TM * 32;
  constexpr int BN = WAVES_N * TN * 32;
  constexpr int LDB_S = BN + 4;
  constexpr int A_ITEMS = BM * BK / 4;  // 4-element groups per A tile
  constexpr int B_ITEMS = BK * BN / 4;
  constexpr int A_PER = (A_ITEMS + THREADS - 1) / THREADS;
  constexpr int B_PER = (B_ITEMS + THREADS - 1) / THREADS;

  __shared__ __attribute__((aligned(16))) float As[2][BM * LDA_S];
  __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB_S];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l32 = lane & 31, g = lane >> 5;

  const int tile = xcd_remap(blockIdx.x, p.tiles_m * p.tiles_n);
  const int bm0 = (tile / p.tiles_n) * BM;
  const int bn0 = (tile % p.tiles_n) * BN;
  const int batch = blockIdx.z;

  const float* __restrict__ A = p.A + batch * p.strideA;
  const float* __restrict__ Bf = static_cast<const float*>(p.B) + batch * p.strideB;
  const unsigned char* __restrict__ Bq =
      static_cast<const unsigned char*>(p.B) + batch * p.strideB;
  float* __restrict__ C = p.C + batch * p.strideC;

  // ---- per-thread description of the A items it stages (fixed over the K loop) ----
  // A_ROWMAJOR / A_IM2COL: item = (row, k-quad); A_TRANSPOSED: item = (k, row-quad).
  int a_row[A_PER], a_kq[A_PER];
  long long a_base[A_PER];  // row-major: row*lda ; im2col: n*H*W*Cin
  int a_ih0[A_PER], a_iw0[A_PER];
  bool a_ok[A_PER];
#pragma unroll
  for (int i = 0; i < A_PER; i++) {
    const int item = tid + i * THREADS;
    a_ok[i] = item < A_ITEMS;
    if (AMODE == A_TRANSPOSED) {
      a_kq[i] = item / (BM / 4);           // k within the tile
      a_row[i] = (item % (BM / 4)) * 4;    // first of 4 rows
      a_base[i] = 0;
    } else {
      a_row[i] = item / (BK / 4);
      a_kq[i] = (item % (BK / 4)) * 4;
      const int m = bm0 + a_row[i];
      if (m >= p.M) a_ok[i] = false;
      if (AMODE == A_ROWMAJOR) {
        a_base[i] = (long long)m * p.lda;
      } else {
        const int ow = m % p.OW, t = m / p.OW;
        const int oh = t % p.OH, n = t / p.OH;
        a_base[i] = (long long)n * p.H * p.W * p.Cin;
        a_ih0[i] = oh * p.sh - p.pt;
        a_iw0[i] = ow * p.sw - p.pl;
      }
    }
  }

  auto load_a = [&](int k0, f32x4 (&reg)[A_PER]) {
#pragma unroll
    for (int i = 0; i < A_PER; i++) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (a_ok[i]) {
        if (AMODE == A_ROWMAJOR) {
          const int k = k0 + a_kq[i];
          const float* src = A + a_base[i] + k;
          if (p.a_vec && k + 3 < p.K) {
            v = *reinterpret_cast<const f32x4*>(src);
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (k + e < p.K) v[e] = src[e];
          }
        } else if (AMODE == A_TRANSPOSED) {
          const int k = k0 + a_kq[i];
          const int m = bm0 + a_row[i];
          if (k < p.K) {
            const float* src = A + (long long)k * p.lda + m;
            if (p.a_vec && m + 3 < p.M) {
              v = *reinterpret_cast<const f32x4*>(src);
            } else {
#pragma unroll
              for (int e = 0; e < 4; e++)
                if (m + e < p.M) v[e] = src[e];
            }
          }
        } else {  // A_IM2COL
          const int k = k0 + a_kq[i];
          if (p.a_vec) {  // Cin % 4 == 0: the 4 elements share one filter tap
            if (k < p.K) {
              const int tap = k / p.Cin, c = k - tap * p.Cin;
              const int kh = tap / p.KW, kw = tap - kh * p.KW;
              const int ih = a_ih0[i] + kh * p.dh, iw = a_iw0[i] + kw * p.dw;
              if ((unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W)
                v = *reinterpret_cast<const f32x4*>(
                    A + a_base[i] + ((long long)ih * p.W + iw) * p.Cin + c);
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const int ke = k + e;
              if (ke < p.K) {
                const int tap = ke / p.Cin, c = ke - tap * p.Cin;
                const int kh = tap / p.KW, kw = tap - kh * p.KW;
                const int ih = a_ih0[i] + kh * p.dh, iw = a_iw0[i] + kw * p.dw;
                if ((unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W)
                  v[e] = A[a_base[i] + ((long long)ih * p.W + iw) * p.Cin + c];
              }
            }
          }
        }
      }
      reg[i] = v;
    }
  };

  auto store_a = [&](float* as, const f32x4 (&reg)[A_PER]) {
#pragma unroll
    for (int i = 0; i < A_PER; i++) {
      const int item = tid + i * THREADS;
      if (item < A_ITEMS) {
        if (AMODE == A_TRANSPOSED) {
#pragma unroll
          for (int e = 0; e < 4; e++) as[(a_row[i] + e) * LDA_S + a_kq[i]] = reg[i][e];
        } else {
          *reinterpret_cast<f32x4*>(&as[a_row[i] * LDA_S + a_kq[i]]) = reg[i];
        }
      }
    }
  };

  // B items: B_ROWMAJOR / B_UINT8: (k, col-quad); B_TRANSPOSED: (col, k-quad)
  auto load_b = [&](int k0, f32x4 (&reg)[B_PER]) {
#pragma unroll
    for (int i = 0; i < B_PER; i++) {
      const int item = tid + i * THREADS;
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (item < B_ITEMS) {
        if (BMODE == B_TRANSPOSED) {
          const int n = bn0 + item / (BK / 4);
          const int k = k0 + (item % (BK / 4)) * 4;
          if (n < p.N) {
            const float* src = Bf + (long long)n * p.ldb + k;
            if (p.b_vec && k + 3 < p.K) {
              v = *reinterpret_cast<const f32x4*>(src);
            } else {
#pragma unroll
              for (int e = 0; e < 4; e++)
                if (k + e < p.K) v[e] = src[e];
            }
          }
        } else {
          const int k = k0 + item / (BN / 4);
          const int n = bn0 + (item % (BN / 4)) * 4;
          if (k < p.K && n < p.N) {
            const long long off = (long long)k * p.ldb + n;
            if (BMODE == B_ROWMAJOR) {
              if (p.b_vec && n + 3 < p.N) {
                v = *reinterpret_cast<const f32x4*>(Bf + off);
              } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                  if (n + e < p.N) v[e] = Bf[off + e];
              }
            } else {  // B_UINT8
              if (p.b_vec && n + 3 < p.N) {
                const unsigned w = *reinterpret_cast<const unsigned*>(Bq + off);
#pragma unroll
                for (int e = 0; e < 4; e++)
                  v[e] = dequant((w >> (8 * e)) & 0xffu, p.qscale, p.qmin);
              } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                  if (n + e < p.N) v[e] = dequant(Bq[off + e], p.qscale, p.qmin);
              }
            }
          }
        }
      }
      reg[i] = v;
    }
  };

  auto store_b = [&](float* bs, const f32x4 (&reg)[B_PER]) {
#pragma unroll
    for (int i = 0; i < B_PER; i++) {
      const int item = tid + i * THREADS;
      if (item < B_ITEMS) {
        if (BMODE == B_TRANSPOSED) {
          const int nn = item / (BK / 4), kq = (item % (BK / 4)) * 4;
#pragma unroll
          for (int e = 0; e < 4; e++) bs[(kq + e) * LDB_S + nn] = reg[i][e];
        } else {
          const int kk = item / (BN / 4), nq = (item % (BN / 4)) * 4;
          *reinterpret_cast<f32x4*>(&bs[kk * LDB_S + nq]) = reg[i];
        }
      }
    }
  };

  // KBLOCKED (matMul): two-level accumulation.  The matrix cores sum 48 consecutive k into
  // `blk`, which is then added to `acc` — the block structure of the reference's matmul
  // (backend_cpu.ts:83, 516-535: 48-wide k blocks, one float32 rounding per block).  It
  // keeps float32 round-off from growing with K: partial sums stay small inside a block.
  // Convolutions accumulate straight through, as the reference's conv2d does (:1601-1604).
  f32x16 acc[TM][TN], blk[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        acc[i][j][r] = 0.f;
        blk[i][j][r] = 0.f;
      }

  f32x4 a_reg[A_PER], b_reg[B_PER];
  const int k_tiles = (p.K + BK - 1) / BK;

  load_a(0, a_reg);
  load_b(0, b_reg);
  store_a(As[0], a_reg);
  store_b(Bs[0], b_reg);
  __syncthreads();

  // One tile step: prefetch tile kt+1 into registers, run the matrix cores on tile kt out
  // of LDS, park the prefetched tile in the other LDS buffer.  `fresh` (compile time) makes
  // the first MFMA of each accumulator start from zero instead of from `blk`.
  auto tile_step = [&](int kt, auto fresh_tag) {
    constexpr bool fresh = decltype(fresh_tag)::value;
    const int cur = kt & 1;
    if (kt + 1 < k_tiles) {
      load_a((kt + 1) * BK, a_reg);
      load_b((kt + 1) * BK, b_reg);
    }
    const float* as = As[cur] + (wm * TM * 32 + l32) * LDA_S + g * 4;
    const float* bs = Bs[cur] + g * 4 * LDB_S + wn * TN * 32 + TN * l32;
#pragma unroll
    for (int kc = 0; kc < BK; kc += 8) {
      f32x4 a[TM];
      float b[4][TN];
#pragma unroll
      for (int i = 0; i < TM; i++)
        a[i] = *reinterpret_cast<const f32x4*>(as + i * 32 * LDA_S + kc);
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const float* src = bs + (kc + r) * LDB_S;
        if (TN == 2) {
          const f32x2 t = *reinterpret_cast<const f32x2*>(src);
          b[r][0] = t[0];
          b[r][TN - 1] = t[1];
        } else if (TN == 4) {
          const f32x4 t = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
          for (int j = 0; j < TN; j++) b[r][j] = t[j];
        } else {
#pragma unroll
          for (int j = 0; j < TN; j++) b[r][j] = src[j];
        }
      }
#pragma unroll
      for (int r = 0; r < 4; r++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++) {
            if (fresh && kc == 0 && r == 0) {
              const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f,
                                   0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
              blk[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][r], b[r][j], zero, 0, 0, 0);
            } else {
              blk[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][r], b[r][j], blk[i][j], 0, 0, 0);
            }
          }
    }
    if (kt + 1 < k_tiles) {
      store_a(As[cur ^ 1], a_reg);
      store_b(Bs[cur ^ 1], b_reg);
    }
    __syncthreads();
  };

  if (KBLOCKED) {
    for (int kt = 0; kt < k_tiles; kt += TILES_PER_KBLOCK) {
      tile_step(kt, std::true_type{});
#pragma unroll
      for (int t = 1; t < TILES_PER_KBLOCK; t++)
        if (kt + t < k_tiles) tile_step(kt + t, std::false_type{});
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] += blk[i][j];
    }
  } else {
    for (int kt = 0; kt < k_tiles; kt++) tile_step(kt, std::false_type{});
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) acc[i][j] = blk[i][j];
  }

  // ---- epilogue: bias, activation, store.  Accumulator register r of a 32x32 tile holds
  // row 8*(r/4) + 4*(lane/32) + r%4, column lane%32.
  const int col0 = bn0 + wn * TN * 32 + TN * l32;
  float bias_c[TN], alpha_c[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int c = col0 + j;
    bias_c[j] = 0.f;
    alpha_c[j] = 0.f;
    if (p.bias_kind == TFHIP_BCAST_SCALAR) bias_c[j] = p.bias[0];
    if (p.bias_kind == TFHIP_BCAST_COLUMN && c < p.N) bias_c[j] = p.bias[c];
    if (p.prelu_kind == TFHIP_BCAST_SCALAR) alpha_c[j] = p.prelu[0];
    if (p.prelu_kind == TFHIP_BCAST_COLUMN && c < p.N) alpha_c[j] = p.prelu[c];
  }
  const bool full_bias = p.bias_kind == TFHIP_BCAST_FULL;
  const bool full_alpha = p.prelu_kind == TFHIP_BCAST_FULL;
  const bool vec_store = (TN == 2 || TN == 4) && (p.N % TN == 0);
#pragma unroll
  for (int i = 0; i < TM; i++) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int row = bm0 + wm * TM * 32 + i * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
      if (row >= p.M) continue;
      const long long base = (long long)row * p.N + col0;
      float out[TN];
#pragma unroll
      for (int j = 0; j < TN; j++) {
        float v = acc[i][j][r];
        const bool in = col0 + j < p.N;
        if (full_bias) {
          if (in) v += p.bias[batch * p.strideC + base + j];
        } else {
          v += bias_c[j];
        }
        float al = alpha_c[j];
        if (full_alpha && in) al = p.prelu[batch * p.strideC + base + j];
        out[j] = activate(v, p.act, al);
      }
      if (vec_store && col0 + TN - 1 < p.N) {
        if (TN == 2) {
          f32x2 t = {out[0], out[TN - 1]};
          *reinterpret_cast<f32x2*>(C + base) = t;
        } else {
          f32x4 t;
#pragma unroll
          for (int j = 0; j < TN; j++) t[j] = out[j];
          *reinterpret_cast<f32x4*>(C + base) = t;
        }
      } else {
#pragma unroll
        for (int j = 0; j < TN; j++)
          if (col0 + j < p.N) C[base + j] = out[j];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
template <int WM_, int WN_, int TM_, int TN_>
struct TileCfg {
  static constexpr int WM = WM_, WN = WN_, TM = TM_, TN = TN_;
  static constexpr int BM = WM_ * TM_ * 32, BN = WN_ * TN_ * 32;
};

template <class T, int AMODE, int BMODE, bool KBLOCKED>
static void launch_cfg(tfhip_ctx* ctx, GemmArgs& p, int batch) {
  static const char* const a_names[] = {"rowmajor", "transposed", "im2col"};
  static const char* const b_names[] = {"f32", "f32t", "u8"};
  snprintf(ctx->last_kernel, sizeof ctx->last_kernel, "gemm_%dx%d_%s_%s%s", T::BM, T::BN,
           a_names[AMODE], b_names[BMODE], KBLOCKED ? "_kb48" : "");
  hipStream_t s = ctx->stream;
  p.tiles_m = (p.M + T::BM - 1) / T::BM;
  p.tiles_n = (p.N + T::BN - 1) / T::BN;
  dim3 grid(p.tiles_m * p.tiles_n, 1, batch);
  hipLaunchKernelGGL((gemm_kernel<T::WM, T::WN, T::TM, T::TN, AMODE, BMODE, KBLOCKED>), grid,
                     dim3(T::WM * T::WN * 64), 0, s, p);
}

// Tile choice: the widest tile whose grid still gives every CU work; narrow-N tiles for
// the early MobileNet layers (N = 32/64) so no matrix-core columns are wasted.
template <int AMODE, int BMODE, bool KBLOCKED>
static void launch_mode(tfhip_ctx* ctx, GemmArgs& p, int batch) {
  using Big = TileCfg<2, 2, 2, 2>;     // 128 x 128
  using Mid = TileCfg<2, 2, 2, 1>;     // 128 x 64
  using Thin = TileCfg<4, 1, 2, 1>;    // 256 x 32
  using Small = TileCfg<2, 2, 1, 1>;   // 64 x 64
  const long long cus = ctx->num_cus;
  auto blocks = [&](int bm, int bn) {
    return (long long)ceil_div(p.M, bm) * ceil_div(p.N, bn) * batch;
  };
  if (p.N <= 32) {
    launch_cfg<Thin, AMODE, BMODE, KBLOCKED>(ctx, p, batch);
  } else if (p.N <= 64) {
    if (blocks(128, 64) >= cus) launch_cfg<Mid, AMODE, BMODE, KBLOCKED>(ctx, p, batch);
    else launch_cfg<Small, AMODE, BMODE, KBLOCKED>(ctx, p, batch);
  } else if (blocks(128, 128) >= 2 * cus) {
    launch_cfg<Big, AMODE, BMODE, KBLOCKED>(ctx, p, batch);
  } else if (blocks(128, 64) >= 2 * cus) {
    launch_cfg<Mid, AMODE, BMODE, KBLOCKED>(ctx, p, batch);
  } else {
    launch_cfg<Small, AMODE, BMODE, KBLOCKED>(ctx, p, batch);
  }
}

static int launch_gemm(tfhip_ctx* ctx, GemmArgs& p, int batch, int amode, int bmode,
                       bool kblocked) {
#define TFHIP_CASE(AM, BM_, KB)                                  \
  if (amode == AM && bmode == BM_ && kblocked == KB) {           \
    launch_mode<AM, BM_, KB>(ctx, p, batch);                     \
    TFHIP_LAUNCH_CHECK(ctx);                                     \
    return TFHIP_OK;                                             \
  }
  TFHIP_CASE(A_ROWMAJOR, B_ROWMAJOR, true)
  TFHIP_CASE(A_ROWMAJOR, B_TRANSPOSED, true)
  TFHIP_CASE(A_ROWMAJOR, B_UINT8, true)
  TFHIP_CASE(A_TRANSPOSED, B_ROWMAJOR, true)
  TFHIP_CASE(A_TRANSPOSED, B_TRANSPOSED, true)
  TFHIP_CASE(A_ROWMAJOR, B_ROWMAJOR, false)
  TFHIP_CASE(A_ROWMAJOR, B_UINT8, false)
  TFHIP_CASE(A_IM2COL, B_ROWMAJOR, false)
  TFHIP_CASE(A_IM2COL, B_UINT8, false)
#undef TFHIP_CASE
  return ctx->fail(TFHIP_ENOTSUP, "matmul: operand layout combination not built "
                                  "(transposed A with quantised B)");
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Resolves a bias / prelu operand of a dense kernel: checks the element count its kind
// promises and converts int32/bool storage to float.
static int epilogue_operand(tfhip_ctx* ctx, const char* what, int64_t id, int kind,
                            int64_t n_cols, int64_t n_full, Temp* tmp, const float** out) {
  *out = nullptr;
  if (kind == TFHIP_BCAST_NONE) return TFHIP_OK;
  TFHIP_GET(ctx, b, id);
  const int64_t want = kind == TFHIP_BCAST_SCALAR ? 1 : kind == TFHIP_BCAST_COLUMN ? n_cols
                     : kind == TFHIP_BCAST_FULL ? n_full : -1;
  if (want < 0) return ctx->fail(TFHIP_EINVAL, "%s: unknown broadcast kind %d", what, kind);
  if (b->numel != want)
    return ctx->fail(TFHIP_EINVAL, "%s holds %lld elements, its layout needs %lld", what,
                     (long long)b->numel, (long long)want);
  return as_f32(ctx, b, tmp, out);
}

}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_matmul(tfhip_ctx* ctx, int64_t a, int64_t b, int64_t out, int batch,
                            int m, int n, int k, int transpose_a, int transpose_b,
                            int64_t bias, int bias_kind, int act, int64_t prelu,
                            int prelu_kind, const tfhip_qparams* q) {
  if (!ctx) return TFHIP_EINVAL;
  TFHIP_GET(ctx, ba, a);
  TFHIP_GET(ctx, bb, b);
  TFHIP_GET(ctx, bo, out);
  if (batch < 0 || m < 0 || n < 0 || k < 0)
    return ctx->fail(TFHIP_EINVAL, "matmul: negative dimension");
  if (ba->numel != (int64_t)batch * m * k || bb->numel != (int64_t)batch * k * n ||
      bo->numel != (int64_t)batch * m * n)
    return ctx->fail(TFHIP_EINVAL,
                     "matmul: buffers hold %lld, %lld, %lld elements; batch=%d m=%d n=%d k=%d "
                     "need %lld, %lld, %lld",
                     (long long)ba->numel, (long long)bb->numel, (long long)bo->numel, batch, m,
                     n, k, (long long)batch * m * k, (long long)batch * k * n,
                     (long long)batch * m * n);
  if (bo->dtype != TFHIP_FLOAT32)
    return ctx->fail(TFHIP_EINVAL, "matmul: output buffer must be float32");
  if (act < TFHIP_ACT_LINEAR || act > TFHIP_ACT_RELU6)
    return ctx->fail(TFHIP_EINVAL, "Activation %d has not been implemented for the HIP backend.",
                     act);
  if (act == TFHIP_ACT_PRELU && prelu_kind == TFHIP_BCAST_NONE)
    return ctx->fail(TFHIP_EINVAL, "matmul: prelu activation without prelu weights");
  const bool quant = bb->dtype == TFHIP_UINT8Q;
  if (quant != (q != nullptr))
    return ctx->fail(TFHIP_EINVAL, "matmul: qparams must be given exactly for a quantised b");
  if (bo->numel == 0) return TFHIP_OK;  // zero-sized result: nothing to launch

  Temp ta(ctx), tb(ctx), tbias(ctx), tprelu(ctx);
  GemmArgs p = {};
  int rc;
  if ((rc = as_f32(ctx, ba, &ta, &p.A))) return rc;
  if (quant) {
    p.B = bb->ptr;
    p.qscale = q->scale;
    p.qmin = q->min;
  } else {
    const float* bf;
    if ((rc = as_f32(ctx, bb, &tb, &bf))) return rc;
    p.B = bf;
  }
  p.C = static_cast<float*>(bo->ptr);
  const int64_t full = (int64_t)batch * m * n;
  if ((rc = epilogue_operand(ctx, "matmul: bias", bias, bias_kind, n, full, &tbias, &p.bias)))
    return rc;
  if ((rc = epilogue_operand(ctx, "matmul: prelu weights", prelu,
                             act == TFHIP_ACT_PRELU ? prelu_kind : TFHIP_BCAST_NONE, n, full,
                             &tprelu, &p.prelu)))
    return rc;
  p.bias_kind = bias_kind;
  p.prelu_kind = act == TFHIP_ACT_PRELU ? prelu_kind : TFHIP_BCAST_NONE;
  p.act = act;
  p.M = m;
  p.N = n;
  p.K = k;
  p.lda = transpose_a ? m : k;
  p.ldb = transpose_b ? k : n;
  p.strideA = (long long)m * k;
  p.strideB = (long long)k * n;
  p.strideC = (long long)m * n;
  if (k == 0) {
    // empty contraction: the result is bias/activation applied to zeros; K loop runs 0 times
  }
  const int amode = transpose_a ? A_TRANSPOSED : A_ROWMAJOR;
  const int bmode = quant ? (transpose_b ? -1 : B_UINT8) : (transpose_b ? B_TRANSPOSED : B_ROWMAJOR);
  if (bmode < 0)
    return ctx->fail(TFHIP_ENOTSUP, "matmul: transposed quantised b is not built");
  p.a_vec = aligned16(p.A) && (p.lda % 4 == 0) && (p.strideA % 4 == 0);
  p.b_vec = aligned16(p.B) && (p.ldb % 4 == 0) && (p.strideB % 4 == 0);
  return launch_gemm(ctx, p, batch, amode, bmode, /*kblocked=*/true);
}

extern "C" int tfhip_conv2d(tfhip_ctx* ctx, int64_t x, int64_t filter, int64_t out,
                            const tfhip_conv2d_info* ci, int64_t bias, int bias_kind, int act,
                            int64_t prelu, int prelu_kind, const tfhip_qparams* q) {
  if (!ctx || !ci) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bw, filter);
  TFHIP_GET(ctx, bo, out);
  if (ci->batch < 0 || ci->in_h < 0 || ci->in_w < 0 || ci->in_c < 0 || ci->out_h < 0 ||
      ci->out_w < 0 || ci->out_c < 0 || ci->filter_h <= 0 || ci->filter_w <= 0 ||
      ci->stride_h <= 0 || ci->stride_w <= 0 || ci->dilation_h <= 0 || ci->dilation_w <= 0)
    return ctx->fail(TFHIP_EINVAL, "conv2d: bad geometry");
  const int64_t x_n = (int64_t)ci->batch * ci->in_h * ci->in_w * ci->in_c;
  const int64_t w_n = (int64_t)ci->filter_h * ci->filter_w * ci->in_c * ci->out_c;
  const int64_t o_n = (int64_t)ci->batch * ci->out_h * ci->out_w * ci->out_c;
  if (bx->numel != x_n || bw->numel != w_n || bo->numel != o_n)
    return ctx->fail(TFHIP_EINVAL,
                     "conv2d: buffers hold %lld, %lld, %lld elements, geometry needs %lld, %lld, %lld",
                     (long long)bx->numel, (long long)bw->numel, (long long)bo->numel,
                     (long long)x_n, (long long)w_n, (long long)o_n);
  // every output pixel must read a window that the padding accounts for
  if ((int64_t)(ci->out_h - 1) * ci->stride_h - ci->pad_top >= ci->in_h ||
      (int64_t)(ci->out_w - 1) * ci->stride_w - ci->pad_left >= ci->in_w)
    return ctx->fail(TFHIP_EINVAL, "conv2d: output extent does not fit the input");
  if (bo->dtype != TFHIP_FLOAT32)
    return ctx->fail(TFHIP_EINVAL, "conv2d: output buffer must be float32");
  if (act < TFHIP_ACT_LINEAR || act > TFHIP_ACT_RELU6)
    return ctx->fail(TFHIP_EINVAL, "Activation %d has not been implemented for the HIP backend.",
                     act);
  if (act == TFHIP_ACT_PRELU && prelu_kind == TFHIP_BCAST_NONE)
    return ctx->fail(TFHIP_EINVAL, "conv2d: prelu activation without prelu weights");
  const bool quant = bw->dtype == TFHIP_UINT8Q;
  if (quant != (q != nullptr))
    return ctx->fail(TFHIP_EINVAL, "conv2d: qparams must be given exactly for a quantised filter");
  if (o_n == 0) return TFHIP_OK;
  if ((int64_t)ci->batch * ci->out_h * ci->out_w > 0x7fffffffLL || x_n > (1LL << 40))
    return ctx->fail(TFHIP_ENOTSUP, "conv2d: more than 2^31 output pixels");

  Temp tx(ctx), tw(ctx), tbias(ctx), tprelu(ctx);
  GemmArgs p = {};
  int rc;
  if ((rc = as_f32(ctx, bx, &tx, &p.A))) return rc;
  if (quant) {
    p.B = bw->ptr;
    p.qscale = q->scale;
    p.qmin = q->min;
  } else {
    const float* wf;
    if ((rc = as_f32(ctx, bw, &tw, &wf))) return rc;
    p.B = wf;
  }
  p.C = static_cast<float*>(bo->ptr);
  if ((rc = epilogue_operand(ctx, "conv2d: bias", bias, bias_kind, ci->out_c, o_n, &tbias,
                             &p.bias)))
    return rc;
  if ((rc = epilogue_operand(ctx, "conv2d: prelu weights", prelu,
                             act == TFHIP_ACT_PRELU ? prelu_kind : TFHIP_BCAST_NONE, ci->out_c,
                             o_n, &tprelu, &p.prelu)))
    return rc;
  p.bias_kind = bias_kind;
  p.prelu_kind = act == TFHIP_ACT_PRELU ? prelu_kind : TFHIP_BCAST_NONE;
  p.act = act;
  p.M = ci->batch * ci->out_h * ci->out_w;
  p.N = ci->out_c;
  p.K = ci->filter_h * ci->filter_w * ci->in_c;
  p.ldb = ci->out_c;
  p.b_vec = aligned16(p.B) && (p.ldb % 4 == 0);
  const bool pointwise = ci->filter_h == 1 && ci->filter_w == 1 && ci->stride_h == 1 &&
                         ci->stride_w == 1 && ci->pad_top == 0 && ci->pad_left == 0 &&
                         ci->out_h == ci->in_h && ci->out_w == ci->in_w;
  int amode;
  if (pointwise) {  // 1x1 stride-1 convolution is a plain [N*H*W, Cin] x [Cin, Cout] product
    amode = A_ROWMAJOR;
    p.lda = ci->in_c;
    p.a_vec = aligned16(p.A) && (p.lda % 4 == 0);
  } else {
    amode = A_IM2COL;
    p.H = ci->in_h; p.W = ci->in_w; p.Cin = ci->in_c;
    p.OH = ci->out_h; p.OW = ci->out_w;
    p.KH = ci->filter_h; p.KW = ci->filter_w;
    p.sh = ci->stride_h; p.sw = ci->stride_w;
    p.dh = ci->dilation_h; p.dw = ci->dilation_w;
    p.pt = ci->pad_top; p.pl = ci->pad_left;
    p.a_vec = aligned16(p.A) && (ci->in_c % 4 == 0);
  }
  return launch_gemm(ctx, p, 1, amode, quant ? B_UINT8 : B_ROWMAJOR, /*kblocked=*/false);
}
