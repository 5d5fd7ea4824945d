// Depthwise 3x3 convolution and the pointwise (1x1) convolution that follows it, as one kernel:
// the block a depthwise-separable network repeats (separableConv2d of the reference,
// ops/conv.ts:588-660, composes depthwiseConv2d and conv2d at op level; backend_cpu.ts:1979-2035
// and :1552-1616 run them), with the bias + activation that follows each of the two folded in.
//
// Why one kernel.  For the first blocks of such a network both halves are bound by HBM: the
// depthwise kernel writes an activation that the pointwise product reads right back.  Here the
// depthwise result never leaves the CU: a wavefront computes it for 32 output pixels into its
// own panel in LDS and multiplies the panel by the pointwise filter on the matrix cores.
// HBM sees the block's input once and its output once.
//
// Shape.  A workgroup is 8 wavefronts: 4 depthwise wavefronts that only load, and 4 pointwise
// wavefronts that only store (a wavefront that does both waits for the acknowledgements of its
// stores whenever it waits for a load: the two share one counter).  Each depthwise wavefront takes
// a strip of SW output columns of one image and walks down a chunk of output rows; what it
// produces goes to a panel [32 pixels][K] in LDS, two panels per depthwise wavefront, one barrier
// per panel: panel i + 1 is filled while panel i is multiplied.
//   depthwise stage: lanes run along the channels (a lane owns one quad of 4 channels and TW
//     neighbouring output columns, so a wavefront access is a run of 16-byte pieces).  Every
//     input row of the strip is fetched once (buffer loads whose offsets fall outside the
//     descriptor where the padding is; PD rows in flight) and feeds the output rows it belongs
//     to, which live in rotating accumulators; taps are summed in the order filter row, filter
//     column, as the reference does.  A finished row gets its bias and activation and goes to
//     the panel; RB rows fill the panel's 32 pixels.
//   pointwise stage: lane = pixel of the panel (16-byte LDS reads of 4 consecutive k; lanes
//     0-31 take k = 0..3 and lanes 32-63 k = 4..7 of each group of 8), v_mfma_f32_32x32x2f32,
//     bias + activation, dword stores of 128-byte runs.  Two forms:
//     - the pointwise filter [K, N] lies in LDS in operand order (K * N * 4 <= 32 KiB beside the
//       panels); pointwise wavefront i multiplies the panels of depthwise wavefront i by all N
//       columns;
//     - COLS (K = N = 128: the filter would take 64 KiB): pointwise wavefront j keeps the filter's
//       columns 32j..32j+31 in registers and multiplies the panels of all four depthwise
//       wavefronts by them; LDS holds panels only.
#include <type_traits>

#include "tfhip_internal.h"
#include "tfhip_device.h"

namespace tfhip {

struct SepArgs {
  const float* x;
  const void* dw;    // [3][3][K] float32 or uint8
  const float* dwb;  // depthwise bias: nullptr, 1 element or K elements
  const void* pw;    // [K][N] float32 or uint8
  const float* pwb;  // pointwise bias: nullptr, 1 element or N elements
  float* y;
  int batch, H, W, OH, OW, pt, pl;
  int dwb_kind, pwb_kind, dw_act, pw_act;
  int dw_quant, pw_quant;
  double dw_scale, dw_min, pw_scale, pw_min;
  unsigned x_bytes, y_bytes;
  int rh;      // output rows of a unit (a multiple of the panel's rows)
  int chunks;  // units per strip of an image: ceil(OH / rh)
  int strips;  // ceil(OW / SW)
  int units;   // batch * chunks * strips
  int reverse;
};

template <int KQ, int NJ, int S, int PD, int OCC, bool COLS>
__global__ __launch_bounds__(512, OCC) void separable_kernel(const SepArgs p) {
  constexpr int K = 8 * KQ, N = 32 * NJ;
  // COLS: the pointwise filter does not fit LDS beside the panels (K = N = 128: 64 KiB).  Then it
  // lives in registers instead: pointwise wavefront j keeps rows 0..K-1 of columns 32j..32j+31 in
  // operand order (K / 2 registers) and multiplies every panel of the workgroup by them, so LDS
  // holds panels only and all four matrix pipes of the CU work on each panel.
  static_assert(!COLS || NJ % 4 == 0, "every pointwise wavefront takes NJ / 4 blocks of 32 output columns");
  constexpr int CB = COLS ? NJ / 4 : 1;  // column blocks of a pointwise wavefront (COLS)
  constexpr int FILTER_FLOATS = COLS ? 0 : K * N;
  constexpr int QN = K / 4;            // channel quads = lanes side by side along the channels
  constexpr int PX = 64 / QN;          // pixel slots of a wavefront
  constexpr int TW = S == 1 ? 2 : 1;   // output columns of a lane
  constexpr int SW = PX * TW;          // output columns of a strip
  constexpr int RB = 32 / SW;          // output rows that fill a panel
  constexpr int NV = (TW - 1) * S + 3; // input vectors of a lane per input row
  constexpr int PITCH = K + 4;         // floats per panel row: 16-byte reads of a lane stay conflict-free
  constexpr int LEAD = 3 - S;          // input rows of a unit before the first one that completes an output row
  static_assert(QN <= 64 && 64 % QN == 0 && 32 % SW == 0, "a wavefront covers whole pixels and rows");
  static_assert(LEAD <= PD && (PD % ((S * RB) % PD ? (S * RB) % PD : 1) == 0) && PD / ((S * RB) % PD ? (S * RB) % PD : PD) <= 4,
                "row buffers take turns with a period of at most four panels");
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* bl = lds;  // pointwise filter as [K / 4][N][4] = (k / 4, col, k % 4)
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  __builtin_amdgcn_s_setprio(WAVE_PRIORITY_MEMORY_BOUND);
  const bool producer = wave < 4;
  const int pair = wave & 3;
  const int l32 = lane & 31, g = lane >> 5;
  float* const panels0 = lds + FILTER_FLOATS;                // two panels per pair
  float* panels = panels0 + pair * (2 * 32 * PITCH);         // this pair's

  if constexpr (!COLS) {
    // the pointwise filter into operand order: an item is 4 consecutive k of one column
    constexpr int PER = (K / 4 * N + 511) / 512;
    auto fill = [&](auto quant_tag) {
      f32x4 w[PER];
#pragma unroll
      for (int u = 0; u < PER; u++) {
        const int item = tid + 512 * u;
        const int k4 = item / N, col = item - k4 * N;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int at = (4 * k4 + e) * N + col;
          if (decltype(quant_tag)::value)
            w[u][e] = dequant(static_cast<const unsigned char*>(p.pw)[at], p.pw_scale, p.pw_min);
          else
            w[u][e] = static_cast<const float*>(p.pw)[at];
        }
      }
#pragma unroll
      for (int u = 0; u < PER; u++)
        *reinterpret_cast<f32x4*>(&bl[(tid + 512 * u) * 4]) = w[u];
    };
    static_assert(K / 4 * N % 512 == 0, "whole passes");
    if (p.pw_quant) fill(std::true_type{});
    else fill(std::false_type{});
  }

  // The units (image, chunk of rows, strip; strip fastest) are cut into 8 runs, one per XCD
  // (workgroup b runs on XCD b % 8; the grid is a multiple of 8): the kernels before and after
  // this one cut their rows the same way, so what an XCD leaves in its L2 is what it reads next.
  // Within its run a workgroup takes four neighbouring units (they share their halo columns),
  // one per pair of wavefronts, then the four `stride` further on, ...  With the filter in LDS
  // (EVEN) what is left of the run after the whole trips is dealt evenly, `deal` <= 4
  // neighbouring units to every workgroup, so that no workgroup (and no CU) gets a whole trip
  // more than another.  (With the filter in registers the same dealing measured 1.3 us slower on
  // [64,56,56,128] -> 128, whose units fill whole trips anyway.)
  constexpr bool EVEN = !COLS;
  const int xcd = (int)blockIdx.x & 7;
  const int per = p.units >> 3, rem = p.units & 7;
  const int run0 = xcd * per + (xcd < rem ? xcd : rem);
  const int run1 = run0 + per + (xcd < rem ? 1 : 0);
  const int wgs = (int)gridDim.x >> 3, wg = (int)blockIdx.x >> 3;
  const int stride = wgs * 4;
  const int wg_first = run0 + wg * 4;
  const int full = EVEN ? (run1 - run0) / stride : 0;  // trips in which every workgroup has four units
  const int left = (run1 - run0) - full * stride;      // units of the last, partial trip
  const int deal = (left + wgs - 1) / wgs;
  const int mine = min(deal, max(0, left - wg * deal)); // units of this workgroup in that trip
  const int last_u = run0 + full * stride + wg * deal;
  const int trips = EVEN ? full + (mine > 0 ? 1 : 0)
                         : (wg_first < run1 ? (run1 - wg_first + stride - 1) / stride : 0);
  const int iters = (p.rh + RB - 1) / RB;  // panels of a unit
  const int total = trips * iters;
  struct Unit {
    bool live;
    int n, o0, rows, strip;
  };
  auto unit_of = [&](int trip, int pr) {
    Unit un;
    int u;
    if (EVEN) {
      const bool whole = trip < full;
      u = (whole ? wg_first + trip * stride : last_u) + pr;
      un.live = whole || pr < mine;
    } else {
      u = wg_first + trip * stride + pr;
      un.live = u < run1;
    }
    const int unit = p.reverse ? run0 + run1 - 1 - u : u;
    un.strip = unit % p.strips;
    const int rest = unit / p.strips;
    const int chunk = rest % p.chunks;
    un.n = rest / p.chunks;
    un.o0 = chunk * p.rh;
    un.rows = min(p.rh, p.OH - un.o0);
    return un;
  };

  if (producer) {
    // ---- depthwise wavefronts: input rows -> panel -------------------------------------------
    const int quad = lane % QN, slot = lane / QN;
    f32x4 w[9], dwb = {0.f, 0.f, 0.f, 0.f};
    if (p.dw_quant) {
      const unsigned char* wq = static_cast<const unsigned char*>(p.dw);
#pragma unroll
      for (int i = 0; i < 9; i++) {
        const unsigned v = *reinterpret_cast<const unsigned*>(wq + i * K + 4 * quad);
#pragma unroll
        for (int e = 0; e < 4; e++) w[i][e] = dequant((v >> (8 * e)) & 0xffu, p.dw_scale, p.dw_min);
      }
    } else {
      const float* wf = static_cast<const float*>(p.dw);
#pragma unroll
      for (int i = 0; i < 9; i++) w[i] = *reinterpret_cast<const f32x4*>(wf + i * K + 4 * quad);
    }
    if (p.dwb_kind == TFHIP_BCAST_COLUMN) {
#pragma unroll
      for (int e = 0; e < 4; e++) dwb[e] = p.dwb[4 * quad + e];
    } else if (p.dwb_kind == TFHIP_BCAST_SCALAR) {
      dwb = f32x4{p.dwb[0], p.dwb[0], p.dwb[0], p.dwb[0]};
    }
    const Clamp dact = clamp_of(p.dw_act);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(p.x, p.x_bytes);
    const unsigned x_row = (unsigned)(p.W * K * 4);
    float* const panel_w = panels + (slot * TW) * PITCH + 4 * quad;  // where this lane writes
    __syncthreads();

    // Input row t of a unit (counted from the top of the padding, ih = t - pt) is filter row kh
    // of output row (t - kh) / S.  The unit consumes rows t0 .. t_last in turn; rows in the
    // padding and beyond t_last are read through an offset outside the descriptor (zeros).
    unsigned col_in[NV];
    unsigned x_img = 0;
    int t0 = 0, t_last = -1;
    // (the row's own offset is the same for the whole wavefront: it rides in the scalar offset of
    // the loads, and a row that is not there is read through a descriptor of length 0, so that a
    // row costs no vector instruction but its loads)
    const __amdgpu_buffer_rsrc_t rx_none = make_rsrc(p.x, 0);
    auto load_row = [&](int t, f32x4 (&in)[NV]) {
      const int ih = t - p.pt;
      const bool row_ok = (unsigned)ih < (unsigned)p.H && t <= t_last;
      if constexpr (COLS && S == 1) {
        // (measured: the 128 -> 128 block is 3 us faster with the offset added per lane)
        const unsigned at = x_img + (unsigned)ih * x_row;
#pragma unroll
        for (int v = 0; v < NV; v++) in[v] = buffer_load_f32x4(rx, row_ok ? at + col_in[v] : OOB_OFFSET);
      } else {
        const int at = __builtin_amdgcn_readfirstlane(row_ok ? (int)(x_img + (unsigned)ih * x_row) : 0);
        const __amdgpu_buffer_rsrc_t r = row_ok ? rx : rx_none;
#pragma unroll
        for (int v = 0; v < NV; v++)
          in[v] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)col_in[v], at, 0));
      }
    };
    auto taps = [&](f32x4& acc, const f32x4 (&in)[NV], int j, int kh) {
#pragma unroll
      for (int kw = 0; kw < 3; kw++) acc += in[j * S + kw] * w[kh * 3 + kw];
    };
    // a finished output row of the strip: bias, activation, into row `rb` of the panel
    auto emit = [&](float* panel, int rb, const f32x4 (&acc)[TW]) {
#pragma unroll
      for (int j = 0; j < TW; j++) {
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = clamp(acc[j][e] + dwb[e], dact);
        *reinterpret_cast<f32x4*>(panel + (rb * SW + j) * PITCH) = v;
      }
    };
    f32x4 buf[PD][NV];
    f32x4 A[TW], B[TW], C[TW];  // output rows in the making, oldest first (stride 2 has A only)
    int trip = 0, blk = 0;
    for (int it = 0; it <= total; it++) {
      if (it < total) {
        if (blk == 0) {
          // a new unit: its offsets, the first PD rows, the rows before the first output row
          const Unit un = unit_of(trip, pair);
          t0 = un.o0 * S;
          t_last = un.live ? (un.o0 + un.rows - 1) * S + 2 : t0 - 1;
          const int iw0 = (un.strip * SW + slot * TW) * S - p.pl;
#pragma unroll
          for (int v = 0; v < NV; v++)
            col_in[v] = (unsigned)(iw0 + v) < (unsigned)p.W ? (unsigned)(((iw0 + v) * K + 4 * quad) * 4)
                                                            : OOB_OFFSET;
          x_img = (unsigned)un.n * (unsigned)p.H * x_row;
#pragma unroll
          for (int i = 0; i < PD; i++) load_row(t0 + i, buf[i]);
          if (S == 1) {
#pragma unroll
            for (int j = 0; j < TW; j++) {
              B[j] = f32x4{0.f, 0.f, 0.f, 0.f};
              taps(B[j], buf[0], j, 0);
            }
            load_row(t0 + PD, buf[0]);
#pragma unroll
            for (int j = 0; j < TW; j++) {
              A[j] = B[j];
              taps(A[j], buf[1 % PD], j, 1);
              B[j] = f32x4{0.f, 0.f, 0.f, 0.f};
              taps(B[j], buf[1 % PD], j, 0);
            }
            load_row(t0 + 1 + PD, buf[1 % PD]);
          } else {
#pragma unroll
            for (int j = 0; j < TW; j++) {
              A[j] = f32x4{0.f, 0.f, 0.f, 0.f};
              taps(A[j], buf[0], j, 0);
            }
            load_row(t0 + PD, buf[0]);
          }
        }
        float* const panel = panel_w + (it & 1) * (32 * PITCH);
        const int i0 = LEAD + blk * RB * S;  // index (from t0) of the first row consumed here
        // Row i of the unit lives in buffer i % PD; PH = (i0 - LEAD) % PD picks the copy of the
        // steps whose buffer numbers are compile-time constants.
        auto steps = [&](auto phase_tag) {
          constexpr int PH = decltype(phase_tag)::value;
#pragma unroll
          for (int rb = 0; rb < RB; rb++) {
            if (S == 1) {
              f32x4 (&in)[NV] = buf[(LEAD + PH + rb) % PD];
#pragma unroll
              for (int j = 0; j < TW; j++) {
                C[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                taps(C[j], in, j, 0);
                taps(B[j], in, j, 1);
                taps(A[j], in, j, 2);
              }
              emit(panel, rb, A);
#pragma unroll
              for (int j = 0; j < TW; j++) {
                A[j] = B[j];
                B[j] = C[j];
              }
              load_row(t0 + i0 + rb + PD, in);
            } else {
              f32x4 (&in1)[NV] = buf[(LEAD + PH + 2 * rb) % PD];
              f32x4 (&in2)[NV] = buf[(LEAD + PH + 2 * rb + 1) % PD];
#pragma unroll
              for (int j = 0; j < TW; j++) {
                taps(A[j], in1, j, 1);
                taps(A[j], in2, j, 2);
              }
              emit(panel, rb, A);
#pragma unroll
              for (int j = 0; j < TW; j++) {
                A[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                taps(A[j], in2, j, 0);
              }
              load_row(t0 + i0 + 2 * rb + PD, in1);
              load_row(t0 + i0 + 2 * rb + 1 + PD, in2);
            }
          }
        };
        constexpr int STEP = (S * RB) % PD;  // how far a panel moves the phase
        if (STEP == 0) {
          steps(std::integral_constant<int, 0>{});
        } else {
          static_assert(STEP == 0 || PD % STEP == 0, "the phases repeat");
          const int phase = (blk * RB * S) % PD;
          if (PD / (STEP ? STEP : 1) == 2) {
            if (phase == 0) steps(std::integral_constant<int, 0>{});
            else steps(std::integral_constant<int, STEP>{});
          } else {
            if (phase == 0) steps(std::integral_constant<int, 0>{});
            else if (phase == STEP) steps(std::integral_constant<int, STEP>{});
            else if (phase == 2 * STEP) steps(std::integral_constant<int, (2 * STEP) % PD>{});
            else steps(std::integral_constant<int, (3 * STEP) % PD>{});
          }
        }
        if (++blk == iters) {
          blk = 0;
          trip++;
        }
      }
      __syncthreads();  // the panel is complete; the other one has been multiplied
    }
  } else if constexpr (COLS) {
    // ---- pointwise wavefronts, each with CB blocks of 32 output columns: every panel x its columns ----
    const int col0 = 32 * CB * pair + l32;  // this lane's column in its first block
    float b[CB][KQ][4];  // filter rows k = 8q + 4g + e of columns col0 + 32 c
#pragma unroll
    for (int c = 0; c < CB; c++)
#pragma unroll
      for (int q = 0; q < KQ; q++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int at = (8 * q + 4 * g + e) * N + col0 + 32 * c;
          b[c][q][e] = p.pw_quant
                           ? dequant(static_cast<const unsigned char*>(p.pw)[at], p.pw_scale, p.pw_min)
                           : static_cast<const float*>(p.pw)[at];
        }
    float bias_c[CB];
#pragma unroll
    for (int c = 0; c < CB; c++)
      bias_c[c] = p.pwb_kind == TFHIP_BCAST_COLUMN ? p.pwb[col0 + 32 * c]
                : p.pwb_kind == TFHIP_BCAST_SCALAR ? p.pwb[0] : 0.f;
    const Clamp pact = clamp_of(p.pw_act);
    const __amdgpu_buffer_rsrc_t ry = make_rsrc(p.y, p.y_bytes);
    const unsigned y_row = (unsigned)(p.OW * N * 4);
    // what the lane adds to the address of accumulator register r of a block: its column, and the
    // 4 pixels that the upper half of the wavefront lies further on (columns, or rows when the
    // strip is narrower than 8)
    const unsigned lane_at = (unsigned)(l32 * 4) +
                             (SW >= 8 ? (unsigned)(4 * g * N * 4) : (unsigned)(g * (4 / SW)) * y_row);
    // ... and with the register's own pixel (row m / SW, column m % SW of the block): the offset of
    // accumulator register r from the block's first pixel, the same for every block of the kernel
    unsigned reg_at[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int mc = 8 * (r >> 2) + (r & 3);
      reg_at[r] = lane_at + (unsigned)(mc / SW) * y_row + (unsigned)((mc % SW) * N * 4);
    }
    const float* const panel_r = panels0 + l32 * PITCH + 4 * g;  // this lane's operand in pair 0's first panel
    __syncthreads();

    int trip = 0, blk = 0;
    for (int it = 0; it <= total; it++) {
      if (it > 0) {
        // the four panels filled during the previous step: block `blk` of the pairs' units
#pragma nounroll
        for (int pr = 0; pr < 4; pr++) {
          const Unit un = unit_of(trip, pr);
          const int rows_left = un.rows - blk * RB;
          if (!un.live || rows_left <= 0) continue;  // (the same for the whole wavefront)
          const float* const panel = panel_r + pr * (2 * 32 * PITCH) + ((it - 1) & 1) * (32 * PITCH);
          f32x16 acc[CB];
          f32x4 a[2];
          a[0] = *reinterpret_cast<const f32x4*>(panel);
#pragma unroll
          for (int q = 0; q < KQ; q++) {
            if (q + 1 < KQ) a[(q + 1) & 1] = *reinterpret_cast<const f32x4*>(panel + 8 * (q + 1));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
              for (int c = 0; c < CB; c++) {
                const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f,
                                     0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                acc[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q & 1][e], b[c][q][e],
                                                              q == 0 && e == 0 ? zero : acc[c], 0, 0, 0);
              }
            __builtin_amdgcn_sched_barrier(0);
          }
          // accumulator register r: pixel m = 8*(r/4) + 4*(lane/32) + r%4 of the panel, column l32.
          // The block's own offset is the same for the whole wavefront and rides in the scalar
          // offset of the stores, what register r and the lane add to it (reg_at, fixed for the
          // kernel) in the vector offset: a whole block is stored without a vector instruction for
          // its addresses.
          const int orow = un.o0 + blk * RB, ocol = un.strip * SW;
          const unsigned y_blk = (unsigned)((un.n * p.OH + orow) * p.OW + ocol) * (unsigned)(N * 4) +
                                 (unsigned)(32 * CB * pair * 4);
          const int cols_left = p.OW - ocol;
          const bool whole = rows_left >= RB && cols_left >= SW;
          if (whole) {
            const int s_blk = __builtin_amdgcn_readfirstlane((int)y_blk);
#pragma unroll
            for (int r = 0; r < 16; r++) {
#pragma unroll
              for (int c = 0; c < CB; c++) {
                const float val = clamp(acc[c][r] + bias_c[c], pact);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, val), ry,
                                                      (int)(reg_at[r] + (unsigned)(32 * c * 4)), s_blk, STORE_WRITE_THROUGH);
              }
            }
          } else {
#pragma unroll
            for (int r = 0; r < 16; r++) {
              const int mc = 8 * (r >> 2) + (r & 3);  // + 4 * g
              int row, col;
              if (SW >= 8) {
                row = mc / SW;
                col = mc % SW + 4 * g;
              } else if (SW == 4) {
                row = mc / SW + g;
                col = mc % SW;
              } else {  // SW == 2: 4 * g pixels further on is 2 rows further down
                row = mc / SW + 2 * g;
                col = mc % SW;
              }
              const unsigned at = y_blk + (unsigned)row * y_row + (unsigned)(col * N * 4) + (unsigned)(l32 * 4);
              const bool ok = row < rows_left && col < cols_left;
#pragma unroll
              for (int c = 0; c < CB; c++) {
                const float val = clamp(acc[c][r] + bias_c[c], pact);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, val), ry,
                                                      (int)(ok ? at + (unsigned)(32 * c * 4) : OOB_OFFSET), 0, STORE_WRITE_THROUGH);
              }
            }
          }
        }
        if (++blk == iters) {
          blk = 0;
          trip++;
        }
      }
      __syncthreads();  // the next panels are complete; these may be overwritten
    }
  } else {
    // ---- pointwise wavefronts: panel x filter -> output --------------------------------------
    float bias_c[NJ];  // pointwise bias of column 32j + l32
#pragma unroll
    for (int j = 0; j < NJ; j++)
      bias_c[j] = p.pwb_kind == TFHIP_BCAST_COLUMN ? p.pwb[32 * j + l32]
                : p.pwb_kind == TFHIP_BCAST_SCALAR ? p.pwb[0] : 0.f;
    const Clamp pact = clamp_of(p.pw_act);
    const __amdgpu_buffer_rsrc_t ry = make_rsrc(p.y, p.y_bytes);
    const unsigned y_row = (unsigned)(p.OW * N * 4);
    const float* const panel_r = panels + l32 * PITCH + 4 * g;  // where this lane reads its operand
    __syncthreads();

    int trip = 0, blk = 0;
    Unit un = unit_of(0, pair);
    for (int it = 0; it <= total; it++) {
      // the panel filled during the previous step: block `blk` of unit `un` (a pair without a
      // unit in this trip has no panel to multiply)
      if (it > 0 && un.live) {
        const float* const panel = panel_r + ((it - 1) & 1) * (32 * PITCH);
        f32x16 acc[NJ];
        // operands of group q + 1 are read while group q is multiplied; the order is pinned so
        // that no more than two groups of them are ever live
        f32x4 a[2], b[2][NJ];
        auto read_ops = [&](int q, f32x4& ao, f32x4 (&bo)[NJ]) {
          ao = *reinterpret_cast<const f32x4*>(panel + 8 * q);
#pragma unroll
          for (int j = 0; j < NJ; j++)
            bo[j] = *reinterpret_cast<const f32x4*>(&bl[((q * 2 + g) * N + 32 * j + l32) * 4]);
        };
        read_ops(0, a[0], b[0]);
#pragma unroll
        for (int q = 0; q < KQ; q++) {
          if (q + 1 < KQ) read_ops(q + 1, a[(q + 1) & 1], b[(q + 1) & 1]);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int e = 0; e < 4; e++)
#pragma unroll
            for (int j = 0; j < NJ; j++) {
              // the very first product of a column block starts from the inline zero
              const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f,
                                   0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
              acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q & 1][e], b[q & 1][j][e],
                                                            q == 0 && e == 0 ? zero : acc[j], 0, 0, 0);
            }
          __builtin_amdgcn_sched_barrier(0);
        }

        // Accumulator register r holds pixel m = 8*(r/4) + 4*(lane/32) + r%4 of the panel,
        // column l32 of column block j; pixel m is row m / SW, column m % SW of the block.  A
        // store writes two runs of 32 consecutive floats.
        const int orow = un.o0 + blk * RB, ocol = un.strip * SW;
        const unsigned y_blk = (unsigned)((un.n * p.OH + orow) * p.OW + ocol) * (unsigned)(N * 4);
        const int rows_left = un.rows - blk * RB, cols_left = p.OW - ocol;
        auto store = [&](auto whole_tag) {
          constexpr bool whole = decltype(whole_tag)::value;
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int mc = 8 * (r >> 2) + (r & 3);  // + 4 * g
            int row, col;                            // of the pixel, the lane's part included
            unsigned at;
            if (SW >= 8) {
              row = mc / SW;
              col = mc % SW + 4 * g;
              at = y_blk + (unsigned)row * y_row + (unsigned)((mc % SW) * N * 4) +
                   (unsigned)((4 * g * N + l32) * 4);
            } else {
              row = mc / SW + g * (4 / SW);
              col = mc % SW;
              at = y_blk + (unsigned)(mc / SW) * y_row + (unsigned)(g * (4 / SW)) * y_row +
                   (unsigned)((mc % SW) * N * 4) + (unsigned)(l32 * 4);
            }
            const bool ok = whole || (row < rows_left && col < cols_left);
#pragma unroll
            for (int j = 0; j < NJ; j++) {
              const float val = clamp(acc[j][r] + bias_c[j], pact);
              __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, val), ry,
                                                    (int)(ok ? at + (unsigned)(32 * j * 4) : OOB_OFFSET), 0, 0);
            }
          }
        };
        // (made of the unit's own numbers, so the whole wavefront takes the same branch)
        if (rows_left >= RB && cols_left >= SW) store(std::true_type{});
        else if (rows_left > 0) store(std::false_type{});
      }
      if (it > 0 && ++blk == iters) {
        blk = 0;
        trip++;
        un = unit_of(trip, pair);
      }
      __syncthreads();  // the next panel is complete; this one may be overwritten
    }
  }
}

template <int KQ, int NJ, int S, int PD, int OCC, bool COLS = false>
static int launch_separable(tfhip_ctx* ctx, SepArgs& p) {
  auto kernel = separable_kernel<KQ, NJ, S, PD, OCC, COLS>;
  constexpr int K = 8 * KQ, N = 32 * NJ;
  constexpr int SW = 64 / (K / 4) * (S == 1 ? 2 : 1), RB = 32 / SW;
  const size_t lds = ((size_t)(COLS ? 0 : K * N) + 8 * 32 * (K + 4)) * sizeof(float);
  static int per_cu = 0;
  if (!per_cu) {
    if (lds > 48 * 1024)
      (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 512, lds) != hipSuccess || n < 1) {
      (void)hipGetLastError();
      n = 1;
    }
    per_cu = n;
  }
  p.strips = (int)ceil_div(p.OW, SW);
  // Chunk height: whole panels.  A chunk reads two input rows beyond its own (stride 1), so
  // chunks are as tall as they can be while every second pair of wavefronts that fits on the
  // machine still gets a unit.
  const long long slots = (long long)ctx->num_cus * per_cu * 4;
  int rh = (int)ceil_div(p.OH, RB) * RB;
  while (rh > RB && (long long)p.batch * p.strips * ceil_div(p.OH, rh) < slots / 2)
    rh = (int)ceil_div(ceil_div(rh, 2), RB) * RB;
  // Chunk height and grid together: with that height or half of it, and a grid of exactly the
  // workgroups the units fill or of whole workgroups per CU, which pair leaves the busiest CU the
  // fewest panels?  A workgroup takes its units four at a time, so a CU's work is (workgroups on
  // it) x (units of a workgroup) x (panels of a unit); every unit costs a start (its first rows
  // give no output) and re-reads the rows above and below it.  [64,112,112,32] -> 64: 1792 units
  // of 14 panels are 448 workgroups, two on 192 CUs and one on 64, 112 panels on the busiest; 3584
  // units of 7 panels on 512 workgroups are 7 units each, 98 panels on every CU: 76.4 -> 67.2 us
  // in a batch-64 MobileNet step.  (The 128 -> 128 block, one workgroup per CU, 896 units of 7
  // panels on 224 of 256 CUs, was measured with its strips cut in two on 256: 75 -> 81 us.)
  const long long resident = (long long)ctx->num_cus * per_cu / 8 * 8;  // a multiple of the XCD count
  const int cus = ctx->num_cus;
  long long grid = 0;
  double best_cost = 0;
  int best_rh = rh;
  const int half = (int)ceil_div(ceil_div(rh, 2), RB) * RB;
  for (int cand : {rh, half}) {
    if (cand < RB || (cand == half && half == rh)) continue;
    const long long units = (long long)p.batch * p.strips * ceil_div(p.OH, cand);
    const double per_unit = (double)ceil_div(cand, RB) + 0.3;
    const double halo = 1.0 + (S == 1 ? 2.0 : 0.5) / cand;
    auto consider = [&](long long g) {
      // (at least two workgroups on most CUs where that many fit: one alone, two wavefronts per
      // SIMD, hides too little latency -- [64,112,112,32] -> 64 on 256 workgroups 75.5 us)
      if (g < 8 || g > resident || g * 8 < (long long)cus * (per_cu < 2 ? per_cu : 2) * 7) return;
      // (units of the busiest workgroup: dealt evenly, or four per trip with the filter in registers)
      const double units_wg = COLS ? 4.0 * (double)ceil_div(units, 4 * g) : (double)ceil_div(units, g);
      const double c = (double)ceil_div(g, cus) * units_wg * per_unit * halo;
      if (grid == 0 || c < best_cost * 0.999) {
        grid = g;
        best_cost = c;
        best_rh = cand;
      }
    };
    consider(ceil_div(ceil_div(units, 8), 4) * 8);
    for (int k = 1; k <= per_cu; k++) consider((long long)cus * k / 8 * 8);
  }
  if (grid == 0)  // (a machine of fewer than 8 CUs: one workgroup per four units)
    grid = resident >= 8 ? resident
                         : ceil_div(ceil_div((long long)p.batch * p.strips * ceil_div(p.OH, rh), 8), 4) * 8;
  rh = best_rh;
  p.rh = rh;
  p.chunks = (int)ceil_div(p.OH, rh);
  p.units = p.batch * p.chunks * p.strips;
  ctx->name_kernel("separable_s%d_k%dxn%d_%s", S, K, N, p.pw_quant ? "u8" : "f32");
  p.reverse = ctx->take_sweep();
  tfhip::launch(ctx, kernel, dim3((unsigned)grid), dim3(512), lds, p);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// The same pair for a small problem (the layers of a network from 28 x 28 pixels down for one or
// two images): the tiled kernels above need thousands of panels to fill the machine, and as two
// launches the pair costs two kernels of 4 to 6 us each that are all latency.  Here a workgroup of
// 8 wavefronts owns a tile of 16 pixels x 64 output columns:
//   1. all 512 lanes compute the depthwise result of the 16 pixels over all K channels (an item
//      is one pixel x 4 channels: 9 range-checked 16-byte loads, taps summed in the order filter
//      row, filter column, bias, activation) into a panel [16][K + 4] in LDS.  The N / 64
//      workgroups of a pixel tile each do this again: 9 x 16 x K multiply-adds, next to nothing;
//   2. wavefront w multiplies columns k_per * w .. of the panel by the matching rows of the
//      pointwise filter, which it reads straight from memory, 16 bytes per lane = the lane's
//      column in each of the tile's four blocks (block c holds columns n0 + 4 j + c), with
//      v_mfma_f32_16x16x4f32 into two accumulator chains per block;
//   3. the 8 partial tiles meet in LDS and are added in wavefront order (fixed, so the result
//      does not depend on scheduling), then bias, activation and a 16-byte store per lane.
// K is shared by the wavefronts exactly as the one-launch kernel for small products shares it,
// so the result has the bits of the two-kernel form.
struct SepSmallArgs {
  const float* x;
  const float* dw;   // [3][3][K]
  const float* dwb;
  const float* pw;   // [K][N]
  const float* pwb;
  float* y;
  int H, W, OH, OW, K, N, S, pt, pl;
  int M;             // batch * OH * OW pixels
  int tiles_m, tiles_n, k_per, by_columns;
  int dwb_kind, pwb_kind, dw_act, pw_act;
  unsigned x_bytes, pw_bytes;
};

__global__ __launch_bounds__(512) void separable_small_kernel(const SepSmallArgs p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];  // the panel, then the partial tiles
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kq = lane >> 4;
  const int K = p.K, N = p.N, PITCH = K + 4;
  // Workgroup b runs on XCD b % 8.  by_columns (at least 8 tile columns): an XCD takes every
  // eighth tile column with all its pixel tiles, so that a line of the filter enters one L2.
  int tm = (int)blockIdx.x / p.tiles_n, tn = (int)blockIdx.x % p.tiles_n;
  if (p.by_columns) {
    const int xcd = (int)blockIdx.x & 7, j = (int)blockIdx.x >> 3;
    tn = xcd + 8 * (j / p.tiles_m);
    tm = j % p.tiles_m;
    if (tn >= p.tiles_n) return;
  }
  const int m0 = tm * 16, n0 = tn * 64;

  // ---- 1. depthwise: 16 pixels x K channels into the panel ----
  {
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(p.x, p.x_bytes);
    const Clamp dact = clamp_of(p.dw_act);
    const int QN = K >> 2;
    auto filter_of = [&](int quad, f32x4 (&w)[9], f32x4& b) {
#pragma unroll
      for (int t = 0; t < 9; t++) w[t] = *reinterpret_cast<const f32x4*>(p.dw + t * K + 4 * quad);
      b = f32x4{0.f, 0.f, 0.f, 0.f};
      if (p.dwb_kind == TFHIP_BCAST_COLUMN) b = *reinterpret_cast<const f32x4*>(p.dwb + 4 * quad);
      else if (p.dwb_kind == TFHIP_BCAST_SCALAR) b = f32x4{p.dwb[0], p.dwb[0], p.dwb[0], p.dwb[0]};
    };
    auto pixel = [&](int px, int quad, const f32x4 (&w)[9], const f32x4& b) {
      const int m = m0 + px;
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (m < p.M) {
        const int ow = m % p.OW, r = m / p.OW;
        const int oh = r % p.OH, n = r / p.OH;
        const int ih0 = oh * p.S - p.pt, iw0 = ow * p.S - p.pl;
        f32x4 in[9];
#pragma unroll
        for (int t = 0; t < 9; t++) {
          const int ih = ih0 + t / 3, iw = iw0 + t % 3;
          const bool ok = (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
          in[t] = buffer_load_f32x4(rx, ok ? (unsigned)((((n * p.H + ih) * p.W + iw) * K + 4 * quad) * 4) : OOB_OFFSET);
        }
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 9; t++) acc += in[t] * w[t];
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = clamp(acc[e] + b[e], dact);
      }
      *reinterpret_cast<f32x4*>(lds + px * PITCH + 4 * quad) = v;
    };
    f32x4 w[9], b;
    if (512 % QN == 0) {
      // every item of a lane has the lane's channel quad: its nine filter taps are read once
      const int quad = tid % QN, step = 512 / QN;
      filter_of(quad, w, b);
      for (int px = tid / QN; px < 16; px += step) pixel(px, quad, w, b);
    } else {
      for (int item = tid; item < 16 * QN; item += 512) {
        const int px = item / QN, quad = item - px * QN;
        filter_of(quad, w, b);
        pixel(px, quad, w, b);
      }
    }
  }
  __syncthreads();

  // ---- 2. pointwise: this wavefront's share of K ----
  constexpr int G = 2;
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.pw, p.pw_bytes);
  const unsigned b_at = n0 + 4 * l16 < N ? (unsigned)((4 * kq * N + n0 + 4 * l16) * 4) : OOB_OFFSET;
  const float* const a_at = lds + l16 * PITCH + 4 * kq;
  const int k_begin = wave * p.k_per;
  const int k_end = min(K, k_begin + p.k_per);
  const int groups = k_end > k_begin ? (k_end - k_begin + 15) >> 4 : 0;
  struct Operands {
    f32x4 a[G];
    f32x4 b[G][4];  // [e]: row k0 + 4 kq + e of the filter, the lane's column in blocks 0..3
  };
  auto load = [&](int q0, Operands& o) {
#pragma unroll
    for (int u = 0; u < G; u++) {
      if (q0 + u >= groups) break;
      const int k0 = k_begin + 16 * (q0 + u);
      const bool in = k0 + 4 * kq < k_end;  // (whole groups of 4: K is a multiple of 4)
      o.a[u] = in ? *reinterpret_cast<const f32x4*>(a_at + k0) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int e = 0; e < 4; e++)
        o.b[u][e] = buffer_load_f32x4(rb, in ? b_at + (unsigned)((k0 + e) * N) * 4 : OOB_OFFSET);
    }
  };
  f32x4 acc[4][2];
#pragma unroll
  for (int c = 0; c < 4; c++) acc[c][0] = acc[c][1] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto multiply = [&](int q0, const Operands& o) {
#pragma unroll
    for (int u = 0; u < G; u++) {
      if (q0 + u >= groups) break;
#pragma unroll
      for (int e = 0; e < 4; e++)
#pragma unroll
        for (int c = 0; c < 4; c++)
          acc[c][e & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(o.a[u][e], o.b[u][e][c], acc[c][e & 1], 0, 0, 0);
    }
  };
  Operands o0, o1;
  load(0, o0);
  for (int q0 = 0; q0 < groups; q0 += 2 * G) {
    load(q0 + G, o1);
    multiply(q0, o0);
    load(q0 + 2 * G, o0);
    multiply(q0 + G, o1);
  }
  __syncthreads();  // every wavefront has read its part of the panel: the partial tiles take its place

  // ---- 3. partial tiles, epilogue ----
#pragma unroll
  for (int c = 0; c < 4; c++)
#pragma unroll
    for (int r = 0; r < 4; r++) lds[((wave * 4 + c) * 4 + r) * 64 + lane] = acc[c][0][r] + acc[c][1][r];
  __syncthreads();
  if (tid >= 256) return;
  // accumulator register r of lane l is pixel 4 * (l / 16) + r, column 4 * (l % 16) + c of block c
  const int r = tid >> 6;
  const int row = m0 + 4 * kq + r, col = n0 + 4 * l16;
  f32x4 v;
#pragma unroll
  for (int c = 0; c < 4; c++) {
    float s = lds[(c * 4 + r) * 64 + lane];
#pragma unroll
    for (int w = 1; w < 8; w++) s += lds[((w * 4 + c) * 4 + r) * 64 + lane];
    v[c] = s;
  }
  if (row >= p.M || col >= N) return;
  const Clamp pact = clamp_of(p.pw_act);
#pragma unroll
  for (int c = 0; c < 4; c++) {
    float b = 0.f;
    if (p.pwb_kind == TFHIP_BCAST_COLUMN) b = p.pwb[col + c];
    else if (p.pwb_kind == TFHIP_BCAST_SCALAR) b = p.pwb[0];
    v[c] = clamp(v[c] + b, pact);
  }
  *reinterpret_cast<f32x4*>(p.y + (long long)row * N + col) = v;
}

// Whether and how the small kernel takes the pair; -1 when it does not.
static int launch_separable_small(tfhip_ctx* ctx, SepSmallArgs& p) {
  if (p.K < 32 || p.K > 1024 || (p.K & 3) || (p.N & 3)) return -1;
  const long long tiles = ceil_div(p.M, 16) * ceil_div(p.N, 64);
  // Where it pays (measured against the two-kernel form, the layers of MobileNet for 1, 2, 4 and 8
  // images): up to two workgroups per CU: one image 64 -> 128 at 112 x 112 stride 2 6.0 us against
  // 9.0, 128 -> 128 at 56 x 56 7.3 against 10.9, 256 -> 256 at 28 x 28 6.6 against 11.6, 512 -> 512
  // at 14 x 14 9.7 against 10.8; four images 512 -> 512 15.8 against 18.5, 1024 -> 1024 at 7 x 7 15.6
  // against 21.4; with more workgroups the tiled product wins (two images 128 -> 128 at 56 x 56:
  // 784 workgroups, 12.4 against 11.3).  Every one of the N / 64 workgroups of a pixel tile repeats
  // the tile's depthwise half, K channels of it: with few pixel tiles and K x N / 64 beyond 4096
  // that costs more than the second launch (one image 1024 -> 1024 at 7 x 7: 14.2 against 10.9).
  if (tiles > 2 * ctx->num_cus) return -1;
  if (tiles < ctx->num_cus / 2 && (long long)p.K * ceil_div(p.N, 64) > 4096) return -1;
  p.tiles_m = (int)ceil_div(p.M, 16);
  p.tiles_n = (int)ceil_div(p.N, 64);
  p.k_per = (int)ceil_div(ceil_div(p.K, 8), 16) * 16;
  p.by_columns = p.tiles_n >= 8;
  const long long grid = p.by_columns ? 8 * ceil_div(p.tiles_n, 8) * p.tiles_m : (long long)p.tiles_m * p.tiles_n;
  const size_t panel = (size_t)16 * (p.K + 4) * sizeof(float), parts = (size_t)8 * 4 * 4 * 64 * sizeof(float);
  const size_t lds = panel > parts ? panel : parts;
  static bool large_lds_allowed = false;
  if (lds > 48 * 1024 && !large_lds_allowed) {
    if (hipFuncSetAttribute((const void*)separable_small_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)((size_t)16 * (1024 + 4) * sizeof(float))) != hipSuccess) {
      (void)hipGetLastError();
      return -1;
    }
    large_lds_allowed = true;
  }
  ctx->name_kernel("separable_small_s%d_f32", p.S);
  tfhip::launch(ctx, separable_small_kernel, dim3((unsigned)grid), dim3(512), lds, p);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

}  // namespace tfhip

using namespace tfhip;

// Ids of the intermediate tensor of the two-kernel form: outside any range a host hands out.
static int64_t g_scratch_id = INT64_MIN / 2;

extern "C" int tfhip_separable_conv2d(tfhip_ctx* ctx, int64_t x, int64_t dw_filter,
                                      int64_t pw_filter, int64_t out,
                                      const tfhip_conv2d_info* dwi, int64_t dw_bias,
                                      int dw_bias_kind, int dw_act, int64_t pw_bias,
                                      int pw_bias_kind, int pw_act, const tfhip_qparams* dw_q,
                                      const tfhip_qparams* pw_q) {
  if (!ctx || !dwi) return TFHIP_EINVAL;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bdw, dw_filter);
  TFHIP_GET(ctx, bpw, pw_filter);
  TFHIP_GET(ctx, bo, out);
  if (dwi->batch < 0 || dwi->out_h < 0 || dwi->out_w < 0 || dwi->in_c <= 0 || dwi->out_c <= 0 ||
      dwi->out_c % dwi->in_c != 0)
    return ctx->fail(TFHIP_EINVAL, "separableConv2d: bad geometry");
  const int64_t mid_c = dwi->out_c;
  const int64_t pixels = (int64_t)dwi->batch * dwi->out_h * dwi->out_w;
  if (bpw->numel % mid_c != 0 || mid_c == 0)
    return ctx->fail(TFHIP_EINVAL, "separableConv2d: the pointwise filter holds %lld elements, "
                                   "not a multiple of the %lld depthwise output channels",
                     (long long)bpw->numel, (long long)mid_c);
  const int64_t out_c = bpw->numel / mid_c;
  if (bo->numel != pixels * out_c)
    return ctx->fail(TFHIP_EINVAL, "separableConv2d: the result holds %lld elements, the geometry "
                                   "needs %lld", (long long)bo->numel, (long long)(pixels * out_c));
  for (int act : {dw_act, pw_act})
    if (act != TFHIP_ACT_LINEAR && act != TFHIP_ACT_RELU && act != TFHIP_ACT_RELU6)
      return ctx->fail(TFHIP_EINVAL, "separableConv2d: activation %d is not folded here", act);
  for (int kind : {dw_bias_kind, pw_bias_kind})
    if (kind != TFHIP_BCAST_NONE && kind != TFHIP_BCAST_SCALAR && kind != TFHIP_BCAST_COLUMN)
      return ctx->fail(TFHIP_EINVAL, "separableConv2d: bias layout %d is not folded here", kind);
  if ((bdw->dtype == TFHIP_UINT8Q) != (dw_q != nullptr) || (bpw->dtype == TFHIP_UINT8Q) != (pw_q != nullptr))
    return ctx->fail(TFHIP_EINVAL, "separableConv2d: qparams must be given exactly for a quantised filter");

  // One kernel when the shapes are the ones it is built for; anything else runs as the two
  // kernels it stands for, with the intermediate in a pool block.
  const Buf* bdb = nullptr;
  const Buf* bpb = nullptr;
  if (dw_bias_kind != TFHIP_BCAST_NONE && !(bdb = ctx->find(dw_bias))) return TFHIP_ENOENT;
  if (pw_bias_kind != TFHIP_BCAST_NONE && !(bpb = ctx->find(pw_bias))) return TFHIP_ENOENT;
  const int K = dwi->in_c, N = (int)out_c, S = dwi->stride_h;
  const int64_t x_n = (int64_t)dwi->batch * dwi->in_h * dwi->in_w * dwi->in_c;
  bool one = dwi->filter_h == 3 && dwi->filter_w == 3 && dwi->dilation_h == 1 &&
             dwi->dilation_w == 1 && dwi->out_c == dwi->in_c && dwi->stride_h == dwi->stride_w &&
             (S == 1 || S == 2) && dwi->out_w >= 16 && bx->dtype == TFHIP_FLOAT32 &&
             bo->dtype == TFHIP_FLOAT32 && bx->numel == x_n && bdw->numel == 9 * (int64_t)K &&
             x_n * 4 < (1ll << 31) && pixels * N * 4 < (1ll << 31) && pixels > 0 &&
             (!bdb || (bdb->dtype == TFHIP_FLOAT32 &&
                       bdb->numel == (dw_bias_kind == TFHIP_BCAST_COLUMN ? K : 1))) &&
             (!bpb || (bpb->dtype == TFHIP_FLOAT32 &&
                       bpb->numel == (pw_bias_kind == TFHIP_BCAST_COLUMN ? N : 1))) &&
             (bdw->dtype == TFHIP_FLOAT32 || bdw->dtype == TFHIP_UINT8Q) &&
             (bpw->dtype == TFHIP_FLOAT32 || bpw->dtype == TFHIP_UINT8Q) && aligned16(bx->ptr) &&
             aligned16(bo->ptr);
  int variant = -1;
  if (one) {
    // enough 32-pixel panels to give every depthwise wavefront of a full machine several
    const int64_t several = (int64_t)ctx->num_cus * 8 * 32 * 3;
    if (K == 32 && N == 64 && S == 1 && pixels >= several) variant = 0;
    else if (K == 64 && N == 128 && S == 2 && pixels >= several) variant = 1;
    else if (K == 128 && N == 128 && S == 1 && pixels >= several) variant = 2;
    // (128 -> 256 at stride 2, two column blocks per pointwise wavefront, was built and measured
    // at [64,56,56,128]: 56 us against 21 + 34 us for the two kernels.  Its 1568 panels are two
    // rounds of a machine of 1024 depthwise wavefronts, the second three quarters full, and the
    // first round's loads and the last round's products overlap with nothing.)
  }
  if (variant >= 0 && !ctx->separable_off) {
    SepArgs p = {};
    p.x = static_cast<const float*>(bx->ptr);
    p.dw = bdw->ptr;
    p.pw = bpw->ptr;
    p.y = static_cast<float*>(bo->ptr);
    p.dwb = bdb ? static_cast<const float*>(bdb->ptr) : nullptr;
    p.pwb = bpb ? static_cast<const float*>(bpb->ptr) : nullptr;
    p.batch = dwi->batch;
    p.H = dwi->in_h;
    p.W = dwi->in_w;
    p.OH = dwi->out_h;
    p.OW = dwi->out_w;
    p.pt = dwi->pad_top;
    p.pl = dwi->pad_left;
    p.dwb_kind = dw_bias_kind;
    p.pwb_kind = pw_bias_kind;
    p.dw_act = dw_act;
    p.pw_act = pw_act;
    p.dw_quant = dw_q != nullptr;
    p.pw_quant = pw_q != nullptr;
    if (dw_q) p.dw_scale = dw_q->scale, p.dw_min = dw_q->min;
    if (pw_q) p.pw_scale = pw_q->scale, p.pw_min = pw_q->min;
    p.x_bytes = (unsigned)(x_n * 4);
    p.y_bytes = (unsigned)(pixels * N * 4);
    switch (variant) {
      case 0: return launch_separable<4, 2, 1, 2, 4>(ctx, p);
      // (measured at [64,112,112,64] -> 128, stride 2: the filter in registers, 4 rows in flight and
      // two workgroups per CU 75.2 us; the filter in LDS, 8 rows in flight, one workgroup 76.8)
      case 1: return launch_separable<8, 4, 2, 4, 4, true>(ctx, p);
      // (measured at [64,56,56,128] -> 128: 4 rows in flight 82 us, 2 rows 85, 8 rows 83; chunks
      // of 32 / 16 / 8 output rows instead of whole strips 87 / 91 / 89)
      case 2: return launch_separable<16, 4, 1, 4, 2, true>(ctx, p);
      default: break;
    }
  }

  // a small problem: one workgroup per 16 pixels x 64 output columns
  const bool small = dwi->filter_h == 3 && dwi->filter_w == 3 && dwi->dilation_h == 1 &&
                     dwi->dilation_w == 1 && dwi->out_c == dwi->in_c && dwi->stride_h == dwi->stride_w &&
                     (S == 1 || S == 2) && bx->dtype == TFHIP_FLOAT32 && bo->dtype == TFHIP_FLOAT32 &&
                     bdw->dtype == TFHIP_FLOAT32 && bpw->dtype == TFHIP_FLOAT32 && bx->numel == x_n &&
                     bdw->numel == 9 * (int64_t)K && x_n * 4 < (1ll << 31) && pixels * N * 4 < (1ll << 31) &&
                     (int64_t)K * N * 4 < (1ll << 31) && pixels > 0 && pixels < (1ll << 24) &&
                     (!bdb || (bdb->dtype == TFHIP_FLOAT32 &&
                               bdb->numel == (dw_bias_kind == TFHIP_BCAST_COLUMN ? K : 1) && aligned16(bdb->ptr))) &&
                     (!bpb || (bpb->dtype == TFHIP_FLOAT32 &&
                               bpb->numel == (pw_bias_kind == TFHIP_BCAST_COLUMN ? N : 1))) &&
                     aligned16(bx->ptr) && aligned16(bdw->ptr) && aligned16(bpw->ptr) && aligned16(bo->ptr);
  if (small && !ctx->separable_off) {
    SepSmallArgs q = {};
    q.x = static_cast<const float*>(bx->ptr);
    q.dw = static_cast<const float*>(bdw->ptr);
    q.pw = static_cast<const float*>(bpw->ptr);
    q.y = static_cast<float*>(bo->ptr);
    q.dwb = bdb ? static_cast<const float*>(bdb->ptr) : nullptr;
    q.pwb = bpb ? static_cast<const float*>(bpb->ptr) : nullptr;
    q.H = dwi->in_h;
    q.W = dwi->in_w;
    q.OH = dwi->out_h;
    q.OW = dwi->out_w;
    q.K = K;
    q.N = N;
    q.S = S;
    q.pt = dwi->pad_top;
    q.pl = dwi->pad_left;
    q.M = (int)pixels;
    q.dwb_kind = dw_bias_kind;
    q.pwb_kind = pw_bias_kind;
    q.dw_act = dw_act;
    q.pw_act = pw_act;
    q.x_bytes = (unsigned)(x_n * 4);
    q.pw_bytes = (unsigned)((int64_t)K * N * 4);
    const int rc = launch_separable_small(ctx, q);
    if (rc >= 0) return rc;
  }

  // the two-kernel form
  const int64_t mid = g_scratch_id++;
  const int32_t mid_shape[4] = {dwi->batch, dwi->out_h, dwi->out_w, dwi->out_c};
  int rc = tfhip_register(ctx, mid, mid_shape, 4, TFHIP_FLOAT32);
  if (rc) return rc;
  rc = tfhip_depthwise_conv2d(ctx, x, dw_filter, mid, dwi, dw_bias, dw_bias_kind, dw_act, dw_q);
  if (!rc) {
    tfhip_conv2d_info pwi = {};
    pwi.batch = dwi->batch;
    pwi.in_h = pwi.out_h = dwi->out_h;
    pwi.in_w = pwi.out_w = dwi->out_w;
    pwi.in_c = dwi->out_c;
    pwi.out_c = (int32_t)out_c;
    pwi.stride_h = pwi.stride_w = pwi.dilation_h = pwi.dilation_w = 1;
    pwi.filter_h = pwi.filter_w = 1;
    rc = tfhip_conv2d(ctx, mid, pw_filter, out, &pwi, pw_bias, pw_bias_kind, pw_act, -1,
                      TFHIP_BCAST_NONE, pw_q);
  }
  std::string keep = ctx->err;  // the message of the failing call, not of the clean-up
  (void)tfhip_dispose(ctx, mid);
  if (rc) ctx->err = keep;
  return rc;
}

// enable = 0 switches the single-kernel forms off (every call then runs its two kernels), any
// other value switches them on again: tests and measurements compare the two forms on the same
// operands.
extern "C" int tfhip_separable_single_kernel(tfhip_ctx* ctx, int enable) {
  if (!ctx) return TFHIP_EINVAL;
  ctx->separable_off = !enable;
  return TFHIP_OK;
}
