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
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "tfhip_internal.h"
#include "tfhip_device.h"

namespace tfhip {

// A_IM2COL_UP: the gather of conv2dDerInput (rows are input pixels, k is (filter row, filter
// column, output channel) of the flipped filter; the image gathered from is dy, stretched by
// the forward stride).  A_IM2COL_T: the gather of conv2dDerFilter (rows are (filter row,
// filter column, input channel), k runs over the output pixels (n, oh, ow)).
enum { A_ROWMAJOR = 0, A_TRANSPOSED = 1, A_IM2COL = 2, A_IM2COL_UP = 3, A_IM2COL_T = 4 };
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
  int up_h, up_w;  // A_IM2COL_UP: forward strides (dy is read at row / up_h when divisible)
  double qscale, qmin;
  // schedule (see work_item)
  int tiles_m, tiles_n, k_tiles, full_tiles, tail_tiles, splits, kt_per;
  int tiles_n_shift;  // log2(tiles_n) when that is a power of two, else -1 (a division on the vector ALU)
  // col_groups > 1 (unbatched products without a split along K): the tiles are numbered column
  // group by column group, a group being 1 << cg_shift tile columns of every tile row, so that an
  // XCD's run of tiles lies inside one group: its L2 then reads 1 / col_groups of B and
  // col_groups / 8 of A instead of all of B and an eighth of A (see choose_col_groups).
  int col_groups, cg_shift;
  float* partials;  // [tail_tiles * splits][BM * BN] partial tiles when splits > 1
  // minis > 0: the tail tiles are not split along K over workgroups but cut into `minis` tiles
  // of 16 x 16 each, one per workgroup, whose wavefronts take mini_k_per of K each (kwaves_tile)
  int minis, mini_k_per;
  unsigned a_bytes, b_bytes;  // per-batch byte extents of A and B (buffer-load range check)
  int reverse;  // walk the tiles / row blocks of every XCD's run from the end
};

constexpr int BK = 16;
constexpr int LDA_S = BK + 4;
constexpr int TILES_PER_KBLOCK = 48 / BK;
constexpr int NBUF = 2;  // LDS double buffer (the pipeline below relies on exactly two)

// The work of one workgroup: a whole output tile, or (when tiles are split along K to fill
// the machine) the k range [kt0, kt1) of one, written to a partial slot.
struct WorkItem {
  int tile;     // linear tile index over (batch, tile row, tile column); -1 = none
  int kt0, kt1;
  int slot;     // partial slot, -1 = finish the tile here
};

// Schedule: the first `full_tiles` workgroups take one whole tile each (ids remapped per
// XCD); the remaining tail_tiles * splits workgroups take k range h % splits of tail tile
// h / splits.  The tail workgroups are dispatched last and in hardware order, so the short
// items spread over all XCDs and CUs.
__device__ __forceinline__ WorkItem work_item(const GemmArgs& p, int block) {
  WorkItem w = {-1, 0, 0, -1};
  if (block < p.full_tiles) {
    w.tile = xcd_remap_dir(block, p.full_tiles, p.reverse);
    w.kt1 = p.k_tiles;
  } else if (block - p.full_tiles < p.tail_tiles * p.splits) {
    const int h = block - p.full_tiles;
    w.tile = p.full_tiles + h / p.splits;
    const int s = h % p.splits;
    w.kt0 = s * p.kt_per;
    w.kt1 = min(p.k_tiles, w.kt0 + p.kt_per);
    if (p.splits > 1) w.slot = h;
  }
  return w;
}

// Tile row and tile column of tile t of an unbatched product (t counts row by row, or column
// group by column group).  t is the same for the whole workgroup.
__device__ __forceinline__ void tile_row_col(const GemmArgs& p, int t, int& tm, int& tn) {
  if (p.col_groups > 1) {
    const int per = p.tiles_m << p.cg_shift;  // tiles of a column group
    int g = 0;
    while (t >= per) {  // (at most col_groups - 1 times)
      t -= per;
      g++;
    }
    tm = t >> p.cg_shift;
    tn = (g << p.cg_shift) + (t - (tm << p.cg_shift));
  } else {
    tm = p.tiles_n_shift >= 0 ? t >> p.tiles_n_shift : t / p.tiles_n;
    tn = t - tm * p.tiles_n;
  }
}

// Small products with a long contraction (a [256, 512] x [512, 256] matMul, the 14 x 14 and
// 7 x 7 pointwise layers of a single image, a classifier's last layer): too few tiles to fill
// the machine, and cutting them along K over workgroups costs a second kernel that adds the
// pieces.  Here the cut is made inside the workgroup: its WAVES wavefronts each take a share of
// K for the same 16 x 16 output tile (v_mfma_f32_16x16x4f32), load their operands straight from
// memory into the registers the matrix instruction reads, and the partial tiles meet in LDS,
// where they are added in wavefront order (a fixed order: the result does not depend on
// timing).  One launch, no partial sums in memory.  Lane l supplies row / column l % 16 and
// k = l / 16 of a group of 4; a lane loads 4 consecutive k of its row at once, so MFMA e of a
// group of 16 multiplies k = 16q + 4(l/16) + e.  G groups of 16 k make one set of operand
// registers; two sets are in flight.  `part` is WAVES x 4 x 64 floats of LDS.
template <int WAVES, int G, bool QUANT>
__device__ __forceinline__ void kwaves_tile(const GemmArgs& p, int m0, int n0, int k_per,
                                            float* part, int tid) {
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kq = lane >> 4;
  const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.A, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.B, p.b_bytes);
  constexpr int B_EL = QUANT ? 1 : 4;
  // rows beyond M and columns beyond N read as zeros: their offsets are out of range
  const unsigned a_at = m0 + l16 < p.M ? (unsigned)(((m0 + l16) * p.lda + 4 * kq) * 4) : OOB_OFFSET;
  const unsigned b_at = n0 + l16 < p.N ? (unsigned)((4 * kq * p.ldb + n0 + l16) * B_EL) : OOB_OFFSET;
  const int k_begin = wave * k_per;
  const int k_end = min(p.K, k_begin + k_per);
  const int groups = k_end > k_begin ? (k_end - k_begin + 15) >> 4 : 0;

  struct Operands {
    f32x4 a[G];
    float b[G][4];
  };
  // group q of this wavefront; k at or beyond K (whole groups of 4: K is a multiple of 4) is
  // turned out of range
  auto load = [&](int q0, Operands& o) {
#pragma unroll
    for (int u = 0; u < G; u++) {
      if (q0 + u >= groups) break;
      const int k0 = k_begin + 16 * (q0 + u);
      const bool in = k0 + 4 * kq < k_end;
      o.a[u] = buffer_load_f32x4(ra, in ? a_at + (unsigned)k0 * 4 : OOB_OFFSET);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const unsigned at = in ? b_at + (unsigned)((k0 + e) * p.ldb) * B_EL : OOB_OFFSET;
        if (QUANT) {
          const unsigned w = __builtin_amdgcn_raw_buffer_load_b8(rb, (int)at, 0, 0);
          o.b[u][e] = __builtin_bit_cast(float, w);
        } else {
          o.b[u][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rb, (int)at, 0, 0));
        }
      }
    }
  };
  f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  auto multiply = [&](int q0, const Operands& o) {
#pragma unroll
    for (int u = 0; u < G; u++) {
      if (q0 + u >= groups) break;
      const int k0 = k_begin + 16 * (q0 + u);
      const bool in = k0 + 4 * kq < k_end;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        float b = o.b[u][e];
        // (a byte that was not read is 0, which stands for the weight `min`: drop it)
        if (QUANT) b = in && n0 + l16 < p.N ? dequant(__builtin_bit_cast(unsigned, b), p.qscale, p.qmin) : 0.f;
        acc[e & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(o.a[u][e], b, acc[e & 1], 0, 0, 0);
      }
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
#pragma unroll
  for (int r = 0; r < 4; r++) part[(wave * 4 + r) * 64 + lane] = acc[0][r] + acc[1][r];
  __syncthreads();
  if (tid >= 256) return;
  // accumulator register r of lane l is row 4 * (l / 16) + r, column l % 16 of the tile
  const int r = tid >> 6;
  const int row = m0 + 4 * kq + r, col = n0 + l16;
  float v = part[r * 64 + lane];
#pragma unroll
  for (int w = 1; w < WAVES; w++) v += part[(w * 4 + r) * 64 + lane];
  if (row >= p.M || col >= p.N) return;
  const long long at = (long long)row * p.N + col;
  if (p.bias_kind == TFHIP_BCAST_SCALAR) v += p.bias[0];
  else if (p.bias_kind == TFHIP_BCAST_COLUMN) v += p.bias[col];
  else if (p.bias_kind == TFHIP_BCAST_FULL) v += p.bias[at];
  float al = 0.f;
  if (p.prelu_kind == TFHIP_BCAST_SCALAR) al = p.prelu[0];
  else if (p.prelu_kind == TFHIP_BCAST_COLUMN) al = p.prelu[col];
  else if (p.prelu_kind == TFHIP_BCAST_FULL) al = p.prelu[at];
  p.C[at] = activate(v, act_cfg(p.act), al);
}

// One 16 x 16 tile per workgroup of 8 wavefronts.  Workgroup b runs on XCD b % 8.  by_columns
// (at least 8 pairs of tile columns): an XCD takes every eighth pair of tile columns (a pair
// shares the 128-byte lines of B's rows) with all their tile rows, so that a line of B is
// fetched into one L2 only; the grid is 8 x (pairs per XCD, rounded up) x 2 x tile rows, and
// workgroups past the last column leave at once.  Otherwise (few columns: A is the large
// operand, and a tile row reads its rows of A alone) the tiles are taken in row-major order.
template <bool QUANT>
__global__ __launch_bounds__(512) void gemm_kwaves_kernel(const GemmArgs p, int k_per,
                                                          int by_columns) {
  __shared__ float part[8 * 4 * 64];
  int tm = (int)blockIdx.x / p.tiles_n, tn = (int)blockIdx.x % p.tiles_n;
  if (by_columns) {
    const int xcd = (int)blockIdx.x & 7, j = (int)blockIdx.x >> 3;
    const int per_pair = 2 * p.tiles_m;
    const int pair = xcd + 8 * (j / per_pair), rem = j % per_pair;
    tn = 2 * pair + (rem & 1);
    tm = rem >> 1;
    if (tn >= p.tiles_n) return;
  }
  kwaves_tile<8, 4, QUANT>(p, tm * 16, tn * 16, k_per, part, threadIdx.x);
}

template <int WAVES_M, int WAVES_N, int TM, int TN, int AMODE, int BMODE, bool KBLOCKED, bool FAST>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_kernel(const GemmArgs p) {
  constexpr int THREADS = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * TM * 32;
  constexpr int BN = WAVES_N * TN * 32;
  constexpr int LDB_S = BN + 4;
  constexpr int A_ITEMS = BM * BK / 4;  // 4-element groups per A tile
  constexpr int B_ITEMS = BK * BN / 4;
  constexpr int A_PER = (A_ITEMS + THREADS - 1) / THREADS;
  constexpr int B_PER = (B_ITEMS + THREADS - 1) / THREADS;

  // One LDS block: the A and B double buffers of the k loop, reused after the loop as the
  // staging area of the output tile (tiles with one accumulator column per wavefront).
  constexpr int A_FLOATS = NBUF * BM * LDA_S, B_FLOATS = NBUF * BK * LDB_S;
  constexpr bool STAGED_STORE = TN == 1;
  constexpr int LDC_S = BN + 4;
  constexpr int C_FLOATS = STAGED_STORE ? BM * LDC_S : 0;
  constexpr int LDS_FLOATS = A_FLOATS + B_FLOATS > C_FLOATS ? A_FLOATS + B_FLOATS : C_FLOATS;
  __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
  // uint8 weights: the 256 values a byte can stand for, each computed once per workgroup exactly
  // as dequant() does; a weight then costs a bit-field extract and an LDS read instead of four
  // double-precision instructions on the pipe the matrix instructions need
  __shared__ float lut[BMODE == B_UINT8 ? 256 : 1];
  float (*As)[BM * LDA_S] = reinterpret_cast<float (*)[BM * LDA_S]>(lds);
  float (*Bs)[BK * LDB_S] = reinterpret_cast<float (*)[BK * LDB_S]>(lds + A_FLOATS);

  const int tid = threadIdx.x;
  __builtin_assume(tid >= 0 && tid < THREADS);
  if (BMODE == B_UINT8 && FAST) {
    static_assert(THREADS >= 256, "one table entry per thread");
    if (tid < 256) lut[tid] = dequant((unsigned)tid, p.qscale, p.qmin);
    __syncthreads();  // (the prologue of the k loop converts weights right away)
  }
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l32 = lane & 31, g = lane >> 5;
  const int tiles_per_batch = p.tiles_m * p.tiles_n;

  // ---- per-tile description of the A/B items this thread stages ----
  // A_ROWMAJOR / A_IM2COL: item = (row, k-quad); A_TRANSPOSED: item = (k, row-quad).
  struct Loader {
    const float* A;
    const float* Bf;
    const unsigned char* Bq;
    int bm0, bn0, batch;
    int a_row[A_PER], a_kq[A_PER];
    long long a_base[A_PER];  // row-major: row*lda ; im2col: n*H*W*Cin
    int a_ih0[A_PER], a_iw0[A_PER];
    bool a_ok[A_PER];
    // FAST loaders whose k offset is the same for every lane (row-major A, every B): the byte
    // offset of the item inside a tile that lies wholly below K, and inside the one tile that K
    // cuts (items at or beyond K out of range).  The tile's own offset rides in the scalar
    // offset of the load, so a k step costs no address arithmetic on the vector ALU, which the
    // matrix instructions share.
    unsigned a_voff[A_PER], a_voff_cut[A_PER];
    unsigned b_voff[B_PER], b_voff_cut[B_PER];
  };
  constexpr bool A_UNIFORM_K = FAST && AMODE == A_ROWMAJOR;

  auto setup = [&](Loader& L, int tile) {
    // (integer division runs on the vector ALU, which the matrix instructions share: none for an
    // unbatched product, a shift for a power-of-two number of tile columns)
    const int batch = tile < tiles_per_batch ? 0 : tile / tiles_per_batch;
    const int t = tile - batch * tiles_per_batch;
    int tm, tn;
    tile_row_col(p, t, tm, tn);
    L.bm0 = tm * BM;
    L.bn0 = tn * BN;
    L.batch = batch;
    L.A = p.A + batch * p.strideA;
    L.Bf = static_cast<const float*>(p.B) + batch * p.strideB;
    L.Bq = static_cast<const unsigned char*>(p.B) + batch * p.strideB;
#pragma unroll
    for (int i = 0; i < A_PER; i++) {
      const int item = tid + i * THREADS;
      L.a_ok[i] = item < A_ITEMS;
      L.a_base[i] = 0;
      L.a_ih0[i] = L.a_iw0[i] = 0;
      if (AMODE == A_TRANSPOSED) {
        L.a_kq[i] = item / (BM / 4);           // k within the tile
        L.a_row[i] = (item % (BM / 4)) * 4;    // first of 4 rows
      } else if (AMODE == A_IM2COL_T) {
        L.a_kq[i] = item / (BM / 4);
        L.a_row[i] = (item % (BM / 4)) * 4;
        const int m = L.bm0 + L.a_row[i];      // (filter row, filter column, channel)
        if (m >= p.M) L.a_ok[i] = false;
        const int tap = m / p.Cin, c = m - tap * p.Cin;
        const int kh = tap / p.KW, kw = tap - kh * p.KW;
        L.a_base[i] = c;
        L.a_ih0[i] = kh * p.dh - p.pt;
        L.a_iw0[i] = kw * p.dw - p.pl;
      } else {
        L.a_row[i] = item / (BK / 4);
        L.a_kq[i] = (item % (BK / 4)) * 4;
        const int m = L.bm0 + L.a_row[i];
        if (m >= p.M) L.a_ok[i] = false;
        if (AMODE == A_ROWMAJOR) {
          L.a_base[i] = (long long)m * p.lda;
        } else {
          const int ow = m % p.OW, r = m / p.OW;
          const int oh = r % p.OH, n = r / p.OH;
          L.a_base[i] = (long long)n * p.H * p.W * p.Cin;
          L.a_ih0[i] = oh * p.sh - p.pt;
          L.a_iw0[i] = ow * p.sw - p.pl;
        }
      }
    }
    if (FAST) {
      const int k_cut = p.K / BK * BK;  // first k of the tile that K cuts (if K % BK != 0)
      if (A_UNIFORM_K) {
#pragma unroll
        for (int i = 0; i < A_PER; i++) {
          const unsigned at = ((unsigned)L.a_base[i] + (unsigned)L.a_kq[i]) * 4u;
          L.a_voff[i] = L.a_ok[i] ? at : OOB_OFFSET;
          L.a_voff_cut[i] = L.a_ok[i] && k_cut + L.a_kq[i] < p.K ? at : OOB_OFFSET;
        }
      }
#pragma unroll
      for (int i = 0; i < B_PER; i++) {
        const int item = tid + i * THREADS;
        int kk, n;
        unsigned at;
        if (BMODE == B_TRANSPOSED) {
          n = L.bn0 + item / (BK / 4);
          kk = (item % (BK / 4)) * 4;
          at = ((unsigned)n * p.ldb + kk) * 4u;
        } else {
          kk = item / (BN / 4);
          n = L.bn0 + (item % (BN / 4)) * 4;
          at = ((unsigned)kk * p.ldb + n) * (BMODE == B_UINT8 ? 1u : 4u);
        }
        const bool ok = item < B_ITEMS && n < p.N;
        L.b_voff[i] = ok ? at : OOB_OFFSET;
        L.b_voff_cut[i] = ok && k_cut + kk < p.K ? at : OOB_OFFSET;
      }
    }
  };

  // FAST: both operands allow aligned 16-byte accesses (K, N, Cin multiples of 4) and span
  // less than 2 GiB per batch entry.  The loaders are then straight-line buffer loads with
  // 32-bit offsets — an item that is out of range gets OOB_OFFSET and reads as zero — so the
  // loads of a step are issued back to back and nothing touches their result until the
  // matrix cores are done with the step.
  __amdgpu_buffer_rsrc_t rsrc_a, rsrc_b, rsrc_a_none, rsrc_b_none;
  // A tile that starts at k0 lies wholly below K, is cut by K, or lies beyond it (a load issued
  // ahead of the last step): the same for all lanes, so the choice between the two offset sets
  // is one select and a tile beyond K reads through the descriptor of length 0.
  auto load_a = [&](Loader& L, int k0_, f32x4 (&reg)[A_PER]) {
    // (k0 is the same for the whole workgroup; saying so keeps the descriptor and the scalar
    // offset in scalar registers wherever the compiler cannot see it)
    const int k0 = FAST ? __builtin_amdgcn_readfirstlane(k0_) : k0_;
    if (A_UNIFORM_K) {
      const bool cut = k0 + BK > p.K;
      const __amdgpu_buffer_rsrc_t r = k0 < p.K ? rsrc_a : rsrc_a_none;
      // (the steps of a workgroup go up in k, so once a tile is cut every later one is cut or
      // beyond K: the cut set replaces the other for good, under a branch that is the same for
      // the whole workgroup.  A select per item would run on the vector ALU, which shares its
      // pipe with the matrix cores, in every k step; the empty asm keeps the compiler from
      // turning the branch back into that select.)
      if (cut) {
#pragma unroll
        for (int i = 0; i < A_PER; i++) {
          unsigned v = L.a_voff_cut[i];
          asm volatile("" : "+v"(v));
          L.a_voff[i] = v;
        }
      }
#pragma unroll
      for (int i = 0; i < A_PER; i++)
        reg[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                     r, (int)L.a_voff[i], k0 * 4, 0));
      return;
    }
    if (FAST) {
#pragma unroll
      for (int i = 0; i < A_PER; i++) {
        const int k = k0 + L.a_kq[i];
        bool ok = L.a_ok[i] && k < p.K;
        unsigned off;
        if (AMODE == A_ROWMAJOR) {
          off = (unsigned)L.a_base[i] + k;
        } else if (AMODE == A_TRANSPOSED) {
          const int m = L.bm0 + L.a_row[i];
          ok = ok && m < p.M;  // M % 4 == 0: the quad is inside or outside as a whole
          off = (unsigned)k * p.lda + m;
        } else if (AMODE == A_IM2COL_T) {
          // k is an output pixel (n, oh, ow); the item's tap and channel quad are fixed
          const int ow = k % p.OW, r = k / p.OW;
          const int oh = r % p.OH, n = r / p.OH;
          const int ih = L.a_ih0[i] + oh * p.sh, iw = L.a_iw0[i] + ow * p.sw;
          ok = ok && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
          off = (unsigned)((n * p.H + ih) * p.W + iw) * p.Cin + (unsigned)L.a_base[i];
        } else {
          const int tap = k / p.Cin, c = k - tap * p.Cin;
          const int kh = tap / p.KW, kw = tap - kh * p.KW;
          int ih = L.a_ih0[i] + kh * p.dh, iw = L.a_iw0[i] + kw * p.dw;
          if (AMODE == A_IM2COL_UP) {
            ok = ok && ih >= 0 && iw >= 0 && ih % p.up_h == 0 && iw % p.up_w == 0;
            ih /= p.up_h;
            iw /= p.up_w;
          }
          ok = ok && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
          off = (unsigned)L.a_base[i] + (unsigned)(ih * p.W + iw) * p.Cin + c;
        }
        reg[i] = buffer_load_f32x4(rsrc_a, ok ? off * 4u : OOB_OFFSET);
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < A_PER; i++) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (L.a_ok[i]) {
        if (AMODE == A_ROWMAJOR) {
          const int k = k0 + L.a_kq[i];
          const float* src = L.A + L.a_base[i] + k;
          if (p.a_vec && k + 3 < p.K) {
            v = *reinterpret_cast<const f32x4*>(src);
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (k + e < p.K) v[e] = src[e];
          }
        } else if (AMODE == A_TRANSPOSED) {
          const int k = k0 + L.a_kq[i];
          const int m = L.bm0 + L.a_row[i];
          if (k < p.K) {
            const float* src = L.A + (long long)k * p.lda + m;
            if (p.a_vec && m + 3 < p.M) {
              v = *reinterpret_cast<const f32x4*>(src);
            } else {
#pragma unroll
              for (int e = 0; e < 4; e++)
                if (m + e < p.M) v[e] = src[e];
            }
          }
        } else if (AMODE == A_IM2COL_T) {
          const int k = k0 + L.a_kq[i];
          if (k < p.K) {
            const int ow = k % p.OW, r = k / p.OW;
            const int oh = r % p.OH, n = r / p.OH;
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const int m = L.bm0 + L.a_row[i] + e;
              if (m < p.M) {
                const int tap = m / p.Cin, c = m - tap * p.Cin;
                const int kh = tap / p.KW, kw = tap - kh * p.KW;
                const int ih = kh * p.dh - p.pt + oh * p.sh, iw = kw * p.dw - p.pl + ow * p.sw;
                if ((unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W)
                  v[e] = L.A[(((long long)n * p.H + ih) * p.W + iw) * p.Cin + c];
              }
            }
          }
        } else {  // A_IM2COL, A_IM2COL_UP
          const int k = k0 + L.a_kq[i];
          // dy row / column of a tap: stretched by the forward stride for A_IM2COL_UP
          auto source = [&](int kh, int kw, int& ih, int& iw) {
            ih = L.a_ih0[i] + kh * p.dh;
            iw = L.a_iw0[i] + kw * p.dw;
            if (AMODE == A_IM2COL_UP) {
              if (ih < 0 || iw < 0 || ih % p.up_h != 0 || iw % p.up_w != 0) return false;
              ih /= p.up_h;
              iw /= p.up_w;
            }
            return (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
          };
          if (p.a_vec) {  // Cin % 4 == 0: the 4 elements share one filter tap
            if (k < p.K) {
              const int tap = k / p.Cin, c = k - tap * p.Cin;
              const int kh = tap / p.KW, kw = tap - kh * p.KW;
              int ih, iw;
              if (source(kh, kw, ih, iw))
                v = *reinterpret_cast<const f32x4*>(
                    L.A + L.a_base[i] + ((long long)ih * p.W + iw) * p.Cin + c);
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const int ke = k + e;
              if (ke < p.K) {
                const int tap = ke / p.Cin, c = ke - tap * p.Cin;
                const int kh = tap / p.KW, kw = tap - kh * p.KW;
                int ih, iw;
                if (source(kh, kw, ih, iw))
                  v[e] = L.A[L.a_base[i] + ((long long)ih * p.W + iw) * p.Cin + c];
              }
            }
          }
        }
      }
      reg[i] = v;
    }
  };

  auto store_a = [&](const Loader& L, float* as, const f32x4 (&reg)[A_PER]) {
#pragma unroll
    for (int i = 0; i < A_PER; i++) {
      const int item = tid + i * THREADS;
      if (item < A_ITEMS) {
        if (AMODE == A_TRANSPOSED || AMODE == A_IM2COL_T) {
#pragma unroll
          for (int e = 0; e < 4; e++) as[(L.a_row[i] + e) * LDA_S + L.a_kq[i]] = reg[i][e];
        } else {
          *reinterpret_cast<f32x4*>(&as[L.a_row[i] * LDA_S + L.a_kq[i]]) = reg[i];
        }
      }
    }
  };

  // B items: B_ROWMAJOR / B_UINT8: (k, col-quad); B_TRANSPOSED: (col, k-quad)
  auto load_b = [&](Loader& L, int k0_, f32x4 (&reg)[B_PER]) {
    const int k0 = FAST ? __builtin_amdgcn_readfirstlane(k0_) : k0_;
    if (FAST) {
      const bool cut = k0 + BK > p.K;
      const __amdgpu_buffer_rsrc_t r = k0 < p.K ? rsrc_b : rsrc_b_none;
      const int soff = BMODE == B_TRANSPOSED ? k0 * 4 : BMODE == B_UINT8 ? k0 * p.ldb : k0 * p.ldb * 4;
      // (a row-major B needs no second set: its rows at or beyond K lie beyond the descriptor's
      // range by themselves, (k * ldb + n) * size >= K * ldb * size >= b_bytes — gfx950 checks the
      // sum of the vector and the scalar offset against the range, as a probe with a 64-byte
      // descriptor shows; a transposed one switches sets for good like A)
      if (BMODE == B_TRANSPOSED && cut) {
#pragma unroll
        for (int i = 0; i < B_PER; i++) {
          unsigned v = L.b_voff_cut[i];
          asm volatile("" : "+v"(v));
          L.b_voff[i] = v;
        }
      }
#pragma unroll
      for (int i = 0; i < B_PER; i++) {
        const unsigned voff = L.b_voff[i];
        if (BMODE == B_UINT8) {
          // The four bytes stay as they are until store_b turns them into floats on their way
          // into LDS, so nothing waits for this load here.  An item out of range reads 0 and
          // becomes the (finite) value of byte 0: every A loader zeroes the items at or beyond
          // K, so such a weight is multiplied by 0, and columns at or beyond N are never stored.
          const unsigned w = __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, soff, 0);
          reg[i][0] = __builtin_bit_cast(float, w);
        } else {
          reg[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, soff, 0));
        }
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < B_PER; i++) {
      const int item = tid + i * THREADS;
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (item < B_ITEMS) {
        if (BMODE == B_TRANSPOSED) {
          const int n = L.bn0 + item / (BK / 4);
          const int k = k0 + (item % (BK / 4)) * 4;
          if (n < p.N) {
            const float* src = L.Bf + (long long)n * p.ldb + k;
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
          const int n = L.bn0 + (item % (BN / 4)) * 4;
          if (k < p.K && n < p.N) {
            const long long off = (long long)k * p.ldb + n;
            if (BMODE == B_ROWMAJOR) {
              if (p.b_vec && n + 3 < p.N) {
                v = *reinterpret_cast<const f32x4*>(L.Bf + off);
              } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                  if (n + e < p.N) v[e] = L.Bf[off + e];
              }
            } else {  // B_UINT8
              if (p.b_vec && n + 3 < p.N) {
                const unsigned w = *reinterpret_cast<const unsigned*>(L.Bq + off);
#pragma unroll
                for (int e = 0; e < 4; e++)
                  v[e] = dequant((w >> (8 * e)) & 0xffu, p.qscale, p.qmin);
              } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                  if (n + e < p.N) v[e] = dequant(L.Bq[off + e], p.qscale, p.qmin);
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
          f32x4 v = reg[i];
          if (BMODE == B_UINT8 && FAST) {
            const unsigned w = __builtin_bit_cast(unsigned, reg[i][0]);
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = lut[(w >> (8 * e)) & 0xffu];
          }
          *reinterpret_cast<f32x4*>(&bs[kk * LDB_S + nq]) = v;
        }
      }
    }
  };

  if constexpr (FAST && AMODE == A_ROWMAJOR && BMODE != B_TRANSPOSED) {
    // a 16 x 16 piece of a tail tile (the planner sets minis only for unbatched products)
    if (p.minis > 0 && (int)blockIdx.x >= p.full_tiles) {
      // All pieces of a tail tile go to one XCD (workgroup b runs on XCD b % 8; full_tiles is a
      // multiple of the CU count), so that the tile's rows of A and columns of B are fetched
      // into one L2 only; the tail tiles take the XCDs in turn.
      const int h = (int)blockIdx.x - p.full_tiles;
      const int j = h >> 3;
      const int tt = (h & 7) + 8 * (j / p.minis), mini = j % p.minis;
      const int t = p.full_tiles + tt;
      int tm, tn;
      tile_row_col(p, t, tm, tn);
      const int m0 = tm * BM + (mini / (BN / 16)) * 16;
      const int n0 = tn * BN + (mini % (BN / 16)) * 16;
      if (tt >= p.tail_tiles || m0 >= p.M || n0 >= p.N) return;
      kwaves_tile<WAVES_M * WAVES_N, 2, BMODE == B_UINT8>(p, m0, n0, p.mini_k_per, lds, tid);
      return;
    }
  }
  Loader L;
  const WorkItem cur = work_item(p, blockIdx.x);
  if (cur.tile < 0) return;
  setup(L, cur.tile);
  const int n_steps = cur.kt1 - cur.kt0;
  rsrc_a = make_rsrc(L.A, p.a_bytes);
  rsrc_b = make_rsrc(BMODE == B_UINT8 ? (const void*)L.Bq : (const void*)L.Bf, p.b_bytes);
  rsrc_a_none = make_rsrc(L.A, 0u);
  rsrc_b_none = make_rsrc(BMODE == B_UINT8 ? (const void*)L.Bq : (const void*)L.Bf, 0u);

  // KBLOCKED (matMul): two-level accumulation.  The matrix cores sum 48 consecutive k into
  // `blk` (its first MFMA starts from the inline zero), which is then added to `acc` — the
  // block structure of the reference's matmul (backend_cpu.ts:83, 516-535: 48-wide k
  // blocks, one float32 rounding per block).  It keeps float32 round-off from growing with
  // K.  Convolutions accumulate straight through, as the reference conv does (:1601-1604).
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

  // The operands of 8 consecutive k of a step, as one wavefront feeds them to the matrix
  // cores: a[ii] = 4 k of this lane's row of accumulator row ii, b[r][j] = k r of its column.
  struct Frag {
    f32x4 a[TM];
    float b[4][TN];
  };
  auto read_frag = [&](int buf, int kc, Frag& f) {
    const float* as = As[buf] + (wm * TM * 32 + l32) * LDA_S + g * 4 + kc;
    const float* bs = Bs[buf] + (g * 4 + kc) * LDB_S + wn * TN * 32 + TN * l32;
#pragma unroll
    for (int ii = 0; ii < TM; ii++)
      f.a[ii] = *reinterpret_cast<const f32x4*>(as + ii * 32 * LDA_S);
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const float* src = bs + r * LDB_S;
      if (TN == 2) {
        const f32x2 t = *reinterpret_cast<const f32x2*>(src);
        f.b[r][0] = t[0];
        f.b[r][TN - 1] = t[1];
      } else if (TN == 4) {
        const f32x4 t = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
        for (int j = 0; j < TN; j++) f.b[r][j] = t[j];
      } else {
#pragma unroll
        for (int j = 0; j < TN; j++) f.b[r][j] = src[j];
      }
    }
  };
  // MFMAs r0..r1-1 of a fragment; with `fresh` the very first one starts `blk` from zero.
  auto mfma_rows = [&](const Frag& f, int r0, int r1, bool fresh) {
#pragma unroll
    for (int r = r0; r < r1; r++)
#pragma unroll
      for (int ii = 0; ii < TM; ii++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
          if (fresh && r == r0) {
            const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f,
                                 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            blk[ii][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[ii][r], f.b[r][j], zero, 0, 0, 0);
          } else {
            blk[ii][j] =
                __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[ii][r], f.b[r][j], blk[ii][j], 0, 0, 0);
          }
        }
  };

  // Software pipeline over the k steps (BK = 16 = two fragments of 8 k each).  In flight at
  // any time: the matrix cores on tile i out of LDS buffer i&1, tile i+1 on its way from
  // registers into the other LDS buffer, and the global loads of tile i+2 into registers.
  // One step, for tile i:
  //   read fragment 1 of tile i          (LDS latency hidden by the next MFMAs)
  //   MFMAs of fragment 0, first half
  //   park tile i+1 in the other LDS buffer; issue the global loads of tile i+2
  //   MFMAs of fragment 0, second half
  //   barrier                            (tile i+1 visible, buffer i&1 free next step)
  //   read fragment 0 of tile i+1        (latency hidden by the MFMAs of fragment 1)
  //   MFMAs of fragment 1
  // sched_barrier(0) pins that order: left alone, the scheduler sinks the global loads next
  // to their LDS stores and every step pays their latency in full.  With FAST loaders the
  // loads past the last tile are range-checked to zero and parked in an unused buffer, so
  // the loop body has no branches.
  // Staging registers.  Convolutions (not KBLOCKED) keep two sets and run the global loads
  // three tiles ahead of the matrix cores instead of two: a step of a lone wavefront is
  // shorter than a trip to HBM.
  constexpr int AHEAD = KBLOCKED ? 2 : 3;
  f32x4 a_reg[2][A_PER], b_reg[2][B_PER];
  Frag f0, f1;
  load_a(L, cur.kt0 * BK, a_reg[0]);
  load_b(L, cur.kt0 * BK, b_reg[0]);
  store_a(L, As[0], a_reg[0]);
  store_b(Bs[0], b_reg[0]);
  // tile 1 goes to set 1 (set 0 when there is one set), tile 2 to set 0
  constexpr int SET1 = AHEAD == 3 ? 1 : 0;
  if (FAST || 1 < n_steps) {
    load_a(L, (cur.kt0 + 1) * BK, a_reg[SET1]);
    load_b(L, (cur.kt0 + 1) * BK, b_reg[SET1]);
  }
  if (AHEAD == 3 && (FAST || 2 < n_steps)) {
    load_a(L, (cur.kt0 + 2) * BK, a_reg[0]);
    load_b(L, (cur.kt0 + 2) * BK, b_reg[0]);
  }
  __syncthreads();
  read_frag(0, 0, f0);

  // step i: `set` holds tile i+1 on entry and receives tile i+AHEAD
  auto step = [&](int i, int buf, f32x4 (&ar)[A_PER], f32x4 (&br)[B_PER], auto fresh_tag) {
    constexpr bool fresh = decltype(fresh_tag)::value;
    read_frag(buf, 8, f1);
    __builtin_amdgcn_sched_barrier(0);
    mfma_rows(f0, 0, 2, fresh);
    __builtin_amdgcn_sched_barrier(0);
    if (FAST || i + 1 < n_steps) {
      store_a(L, As[buf ^ 1], ar);
      store_b(Bs[buf ^ 1], br);
    }
    if (FAST || i + AHEAD < n_steps) {
      load_a(L, (cur.kt0 + i + AHEAD) * BK, ar);
      load_b(L, (cur.kt0 + i + AHEAD) * BK, br);
    }
    __builtin_amdgcn_sched_barrier(0);
    mfma_rows(f0, 2, 4, false);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    read_frag(buf ^ 1, 0, f0);
    __builtin_amdgcn_sched_barrier(0);
    mfma_rows(f1, 0, 4, false);
    __builtin_amdgcn_sched_barrier(0);
  };

  auto flush = [&]() {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) acc[i][j] += blk[i][j];
  };

  if (KBLOCKED) {
    int buf = 0;
    for (int i = 0; i < n_steps; i += TILES_PER_KBLOCK) {
      step(i, buf, a_reg[0], b_reg[0], std::true_type{});
      buf ^= 1;
#pragma unroll
      for (int t = 1; t < TILES_PER_KBLOCK; t++)
        if (i + t < n_steps) {
          step(i + t, buf, a_reg[0], b_reg[0], std::false_type{});
          buf ^= 1;
        }
      flush();
    }
  } else {
    for (int i = 0; i < n_steps; i += 2) {
      step(i, 0, a_reg[1], b_reg[1], std::false_type{});
      if (i + 1 < n_steps) step(i + 1, 1, a_reg[0], b_reg[0], std::false_type{});
    }
  }
  f32x16(&res)[TM][TN] = KBLOCKED ? acc : blk;

  // ---- store.  Accumulator register r of a 32x32 tile holds row
  // 8*(r/4) + 4*(lane/32) + r%4, column lane%32.
  const int bm0 = L.bm0, bn0 = L.bn0;
  const int batch = L.batch;
  const int col0 = bn0 + wn * TN * 32 + TN * l32;
  if (cur.slot >= 0) {
    // partial sum of a k range: raw accumulators into the tile-shaped slot
    float* slot = p.partials + (long long)cur.slot * (BM * BN);
    const int lc = wn * TN * 32 + TN * l32;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int lr = wm * TM * 32 + i * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
#pragma unroll
        for (int j = 0; j < TN; j++) slot[lr * BN + lc + j] = res[i][j][r];
      }
    return;
  }
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
  const ActCfg act = act_cfg(p.act);
  const Clamp cl = clamp_of(p.act);
  const bool prelu = p.act == TFHIP_ACT_PRELU;  // takes the FULL path: it alone needs a product
  // FULL: bias or prelu weights with one value per output element (rare) are read here.
  // INTERIOR: the whole tile lies inside the matrix, so no store needs a bounds check.
  // Addresses are a tile base that is the same for the whole wavefront plus a 32-bit offset.
  const int lrow0 = wm * TM * 32 + 4 * g;        // this lane's first row within the tile
  const int lcol0 = wn * TN * 32 + TN * l32;     // its first column within the tile
  const long long tile_at = batch * p.strideC + (long long)bm0 * p.N + bn0;
  float* __restrict__ Ct = p.C + tile_at;
  auto store = [&](auto full_tag, auto interior_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    constexpr bool INTERIOR = decltype(interior_tag)::value;
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int lrow = lrow0 + i * 32 + 8 * (r >> 2) + (r & 3);
        if (!INTERIOR && bm0 + lrow >= p.M) continue;
        const int at = lrow * p.N + lcol0;
        float out[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) {
          float bv = bias_c[j], al = alpha_c[j];
          if (FULL) {
            const bool in = col0 + j < p.N;
            if (full_bias && in) bv = p.bias[tile_at + at + j];
            if (full_alpha && in) al = p.prelu[tile_at + at + j];
          }
          out[j] = FULL ? activate(res[i][j][r] + bv, act, al) : clamp(res[i][j][r] + bv, cl);
        }
        if (vec_store && (INTERIOR || col0 + TN - 1 < p.N)) {
          if (TN == 2) {
            f32x2 t = {out[0], out[TN - 1]};
            *reinterpret_cast<f32x2*>(Ct + at) = t;
          } else {
            f32x4 t;
#pragma unroll
            for (int j = 0; j < TN; j++) t[j] = out[j];
            *reinterpret_cast<f32x4*>(Ct + at) = t;
          }
        } else {
#pragma unroll
          for (int j = 0; j < TN; j++)
            if (INTERIOR || col0 + j < p.N) Ct[at + j] = out[j];
        }
      }
    }
  };
  const bool interior = bm0 + BM <= p.M && bn0 + BN <= p.N;
  if (full_bias || full_alpha || prelu) {
    store(std::true_type{}, std::false_type{});
  } else if (!interior) {
    store(std::false_type{}, std::false_type{});
  } else if (STAGED_STORE && (p.N & 3) == 0 && (long long)BM * p.N * 4 < 0x7fffffffll) {
    // One accumulator column per lane would mean 4-byte stores (two 128-byte runs per
    // instruction).  Pass the tile through LDS instead and store it as 16 bytes per lane,
    // whole 256/512-byte row segments per instruction: a quarter of the store instructions.
    // (Ct is 16-byte aligned: buffers are, bn0 is a multiple of 64 and N of 4.)
    __syncthreads();  // every wavefront is done with the k-loop buffers
    float* cs = lds + lrow0 * LDC_S + lcol0;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++)
        cs[(i * 32 + 8 * (r >> 2) + (r & 3)) * LDC_S] = res[i][0][r];
    __syncthreads();
    constexpr int QUADS_PER_ROW = BN / 4;
    // (a tile inside the matrix, its byte offsets below 2 GiB: no store relies on the range
    // check.  Written through the L2: see STORE_WRITE_THROUGH.)
    const __amdgpu_buffer_rsrc_t rsrc_ct = make_rsrc(Ct, 0x7fffffffu);
    constexpr int ROWS_PER_PASS = THREADS / QUADS_PER_ROW;
    static_assert(THREADS % QUADS_PER_ROW == 0 && BM % ROWS_PER_PASS == 0, "tile / block shape");
    const int cq = tid % QUADS_PER_ROW, r0 = tid / QUADS_PER_ROW;
    f32x4 bv = {0.f, 0.f, 0.f, 0.f};
    if (p.bias_kind == TFHIP_BCAST_SCALAR) bv = f32x4{p.bias[0], p.bias[0], p.bias[0], p.bias[0]};
    if (p.bias_kind == TFHIP_BCAST_COLUMN)
#pragma unroll
      for (int e = 0; e < 4; e++) bv[e] = p.bias[bn0 + 4 * cq + e];
#pragma unroll
    for (int pass = 0; pass < BM / ROWS_PER_PASS; pass++) {
      const int row = r0 + pass * ROWS_PER_PASS;
      f32x4 v = *reinterpret_cast<const f32x4*>(lds + row * LDC_S + 4 * cq);
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = clamp(v[e] + bv[e], cl);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc_ct,
                                             (row * p.N + 4 * cq) * 4, 0, STORE_WRITE_THROUGH);
    }
  } else {
    store(std::false_type{}, std::true_type{});
  }
}

// Finishes the tiles that were split along K: adds the `splits` partial tiles in ascending
// k order (fixed order, so the result does not depend on scheduling), then bias,
// activation and store.  One thread per 4 columns of a tile row.
__global__ void splitk_finish_kernel(const GemmArgs p, int BM, int BN, int first_tile) {
  const int tiles_per_batch = p.tiles_m * p.tiles_n;
  const int quads = BM * BN / 4;
  const long long total = (long long)p.tail_tiles * quads;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < total; q += stride) {
    const int tt = (int)(q / quads);
    const int e = (int)(q - (long long)tt * quads) * 4;
    const int lr = e / BN, lc = e - lr * BN;
    const int tile = first_tile + tt;
    const int batch = tile / tiles_per_batch;
    const int t = tile - batch * tiles_per_batch;
    const int row = (t / p.tiles_n) * BM + lr;
    const int col = (t % p.tiles_n) * BN + lc;
    if (row >= p.M || col >= p.N) continue;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    const float* src = p.partials + ((long long)tt * p.splits) * (BM * BN) + e;
    // four partial tiles in flight at a time; added in ascending k order
    int s = 0;
    for (; s + 4 <= p.splits; s += 4) {
      f32x4 t[4];
#pragma unroll
      for (int u = 0; u < 4; u++)
        t[u] = *reinterpret_cast<const f32x4*>(src + (long long)(s + u) * (BM * BN));
#pragma unroll
      for (int u = 0; u < 4; u++) v += t[u];
    }
    for (; s < p.splits; s++) v += *reinterpret_cast<const f32x4*>(src + (long long)s * (BM * BN));
    const long long base = (long long)batch * p.strideC + (long long)row * p.N + col;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if (col + j >= p.N) break;
      float x = v[j];
      if (p.bias_kind == TFHIP_BCAST_SCALAR) x += p.bias[0];
      else if (p.bias_kind == TFHIP_BCAST_COLUMN) x += p.bias[col + j];
      else if (p.bias_kind == TFHIP_BCAST_FULL) x += p.bias[base + j];
      float al = 0.f;
      if (p.prelu_kind == TFHIP_BCAST_SCALAR) al = p.prelu[0];
      else if (p.prelu_kind == TFHIP_BCAST_COLUMN) al = p.prelu[col + j];
      else if (p.prelu_kind == TFHIP_BCAST_FULL) al = p.prelu[base + j];
      p.C[base + j] = activate(x, act_cfg(p.act), al);
    }
  }
}

// Convolution with a short contraction (KH*KW*Cin <= 32, e.g. a 3x3 stem over RGB) and at
// most 64 output channels.  The im2col rows of such a layer are 27 scattered, unaligned
// floats per pixel, which the tiled kernel above can only gather element by element; here a
// workgroup takes output rows (n, oh) in turn: it copies the KH input rows that the row reads into
// LDS with coalesced loads (zeros where the padding is), and every wavefront then builds the
// MFMA operand of 32 output pixels straight out of LDS.  The whole filter lives in
// registers (k = 8q + 4*(lane/32) + e of MFMA group q, the same summation-order permutation
// as above).  HBM traffic is the input once (rows shared by neighbouring output rows come out
// of L2) plus the output once.  SPLIT (the staged rows of one output row are at most 2048
// floats): two more wavefronts do the loading, into two LDS buffers of SPLIT_BUF floats.
constexpr int SPLIT_BUF = 2048 + 16;
template <int TN, bool QUANT, bool SPLIT>
__global__ __launch_bounds__(SPLIT ? 384 : 256) void conv_smallk_kernel(const GemmArgs p,
                                                                       int row_floats, int n_rows) {
  extern __shared__ __attribute__((aligned(16))) float rows[];  // [KH][row_floats] (+ 1), x 2 if SPLIT
  __builtin_amdgcn_s_setprio(WAVE_PRIORITY_MEMORY_BOUND);
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const int row_in = p.W * p.Cin;
  const int stage_n = p.KH * row_floats;
  // A grid that is a multiple of 8 cuts the output rows into one run per XCD (workgroup b runs
  // on XCD b % 8): neighbouring output rows, which share input rows, then meet in one L2, and
  // the kernel that reads the result cuts it the same way.
  int row_first = blockIdx.x, row_step = gridDim.x, row_end = n_rows;
  if ((gridDim.x & 7) == 0) {
    const int xcd = (int)blockIdx.x & 7, per = n_rows >> 3, rem = n_rows & 7;
    const int run0 = xcd * per + (xcd < rem ? xcd : rem);
    row_end = run0 + per + (xcd < rem ? 1 : 0);
    row_first = run0 + ((int)blockIdx.x >> 3);
    row_step = (int)gridDim.x >> 3;
  }
  // (image, output row) of a row of this workgroup, advanced by additions: a division per row
  // would run on the vector ALU
  const int step_n = row_step / p.OH, step_oh = row_step - step_n * p.OH;
  auto advance = [&](int& n, int& oh) {
    n += step_n;
    oh += step_oh;
    if (oh >= p.OH) {
      oh -= p.OH;
      n++;
    }
  };
  int n = row_first / p.OH, oh = row_first - n * p.OH;

  // rows this workgroup takes
  const int count = row_first < row_end ? (row_end - row_first + row_step - 1) / row_step : 0;
  if constexpr (SPLIT) {
    // (the zero slots of both buffers, which no loader writes)
    if (tid == 0) rows[p.KH * row_floats] = rows[SPLIT_BUF + p.KH * row_floats] = 0.f;
    if (wave >= 4) {
      const int ptid = tid - 256;
      // Per lane and staged element, fixed for the lifetime of the workgroup: the byte offset of
      // (kh, column) relative to the first input row of an output row, or a value that stays out
      // of range whatever row offset is added (elements past the block, columns in the padding).
      // The rows above and below the image fall out of the descriptor's range by themselves: a
      // negative offset wraps to a huge one.  So a staged element costs one add and one load.
      unsigned ld_const[16];
#pragma unroll
      for (int u = 0; u < 16; u++) {
        const int i = ptid + u * 128;
        const int kh = i / row_floats;
        const int e = i - kh * row_floats - p.pl * p.Cin;
        const bool ok = i < stage_n && (unsigned)e < (unsigned)row_in;
        ld_const[u] = ok ? (unsigned)((kh * p.dh * row_in + e) * 4) : OOB_OFFSET;
      }
      const unsigned img_bytes = (unsigned)(p.H * row_in) * 4u;
      int ld_n = n, ld_oh = oh;  // the row whose loads are issued next
      auto stage_load = [&](float (&v)[16]) {
        const __amdgpu_buffer_rsrc_t rimg = make_rsrc(p.A + (long long)ld_n * p.H * row_in, img_bytes);
        const unsigned first = (unsigned)((ld_oh * p.sh - p.pt) * row_in * 4);  // may be "negative"
#pragma unroll
        for (int u = 0; u < 16; u++)
          v[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                               rimg, (int)(ld_const[u] + first), 0, 0));
        advance(ld_n, ld_oh);
      };
      auto put = [&](const float (&v)[16], float* rb) {
#pragma unroll
        for (int u = 0; u < 16; u++)
          if (ptid + u * 128 < stage_n) rb[ptid + u * 128] = v[u];
      };
      float v0[16], v1[16];
      if (count > 0) stage_load(v0);
      if (count > 1) stage_load(v1);
      if (count > 0) put(v0, rows);
      if (count > 2) stage_load(v0);
      __syncthreads();
      for (int it = 0; it < count; it += 2) {
        // while row `it` is multiplied out of buffer 0
        if (it + 1 < count) put(v1, rows + SPLIT_BUF);
        if (it + 3 < count) stage_load(v1);
        __syncthreads();
        if (it + 1 >= count) break;
        // while row `it + 1` is multiplied out of buffer 1
        if (it + 2 < count) put(v0, rows);
        if (it + 4 < count) stage_load(v0);
        __syncthreads();
      }
      return;
    }
  }
  // this lane's 16 contraction indices k = 8q + 4g + e: LDS offset of (kh, kw, c), or -1 past
  // K, and row k of the filter.  (kh, kw, c) is counted up with k, which keeps the walk in
  // scalar registers; the filter loads are unconditional (clamped index) so that they are
  // all in flight together.
  int a_off[4][4];
  float b[4][4][TN];
  {
    int kh = 0, kw = 0, c = 0;
#pragma unroll
    for (int k = 0; k < 32; k++) {
      const int q = k >> 3, gk = (k >> 2) & 1, e = k & 3;
      const bool k_ok = k < p.K;
      const int off = k_ok ? kh * row_floats + kw * p.dw * p.Cin + c : -1;
      if (g == gk) a_off[q][e] = off;
      if (++c == p.Cin) {
        c = 0;
        if (++kw == p.KW) {
          kw = 0;
          kh++;
        }
      }
    }
  }
#pragma unroll
  for (int q = 0; q < 4; q++)
#pragma unroll
    for (int e = 0; e < 4; e++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const int k = 8 * q + 4 * g + e, col = 32 * j + l32;
        const bool ok = k < p.K && col < p.N;
        const int at = ok ? k * p.N + col : 0;
        float w;
        if (QUANT) w = dequant(static_cast<const unsigned char*>(p.B)[at], p.qscale, p.qmin);
        else w = static_cast<const float*>(p.B)[at];
        b[q][e][j] = ok ? w : 0.f;
      }
  float bias_c[TN], alpha_c[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int col = 32 * j + l32;
    bias_c[j] = alpha_c[j] = 0.f;
    if (p.bias_kind == TFHIP_BCAST_SCALAR) bias_c[j] = p.bias[0];
    if (p.bias_kind == TFHIP_BCAST_COLUMN && col < p.N) bias_c[j] = p.bias[col];
    if (p.prelu_kind == TFHIP_BCAST_SCALAR) alpha_c[j] = p.prelu[0];
    if (p.prelu_kind == TFHIP_BCAST_COLUMN && col < p.N) alpha_c[j] = p.prelu[col];
  }
  // Where this lane reads its 16 operand values of a strip of 32 output pixels: the LDS index
  // of (kh, kw, c) at its pixel, or a slot behind the staged rows that holds 0 for k past K.
  // Every output row has the same strips, so the first strip's addresses are computed once.
  const int zero_slot = p.KH * row_floats;
  if (!SPLIT && tid == 0) rows[zero_slot] = 0.f;
  // (a copy of a lane constant that the optimiser cannot see through: the address arithmetic of
  // the rarely taken paths below then stays inside them instead of being hoisted out of the row
  // loop into registers that every row pays for)
  auto opaque = [](int x) {
    asm volatile("" : "+v"(x));
    return x;
  };
  auto pixel_base = [&](int strip, int lane32) {
    const int ow = min(strip * 32 + lane32, p.OW - 1);  // clamped: lanes past the row compute a copy
    return ow * p.sw * p.Cin;
  };
  const int base_first = pixel_base(wave, l32);
  int a_first[4][4];
#pragma unroll
  for (int q = 0; q < 4; q++)
#pragma unroll
    for (int e = 0; e < 4; e++) a_first[q][e] = a_off[q][e] >= 0 ? a_off[q][e] + base_first : zero_slot;
  // (rows wider than 128 output pixels: further strips shift the first strip's addresses)
  auto strip_addresses = [&](int strip, int (&addr)[4][4]) {
    const int shift = pixel_base(strip, opaque(l32)) - base_first;
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
      for (int e = 0; e < 4; e++)
        addr[q][e] = a_first[q][e] == zero_slot ? zero_slot : a_first[q][e] + shift;
  };

  // One output row out of the staged input rows `rb`: each wavefront multiplies strips of 32
  // pixels and stores them.
  auto compute_row = [&](int n, int oh, const float* rb) {
    const long long out_at = (((long long)n * p.OH + oh) * p.OW) * p.N;  // workgroup-uniform
    float* __restrict__ crow = p.C + out_at;
    const ActCfg act = act_cfg(p.act);
    const Clamp cl = clamp_of(p.act);
    const bool prelu = p.act == TFHIP_ACT_PRELU;  // (takes the general path below)
    const float* bias_row = p.bias_kind == TFHIP_BCAST_FULL ? p.bias + out_at : nullptr;
    const float* alpha_row = p.prelu_kind == TFHIP_BCAST_FULL ? p.prelu + out_at : nullptr;
    // the output row as a descriptor: pixels past the row fall out of its range
    const __amdgpu_buffer_rsrc_t rout = make_rsrc(crow, (unsigned)(p.OW * p.N) * 4u);
    for (int strip = wave; strip * 32 < p.OW; strip += 4) {
      f32x16 acc[TN];
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[j][r] = 0.f;
      auto multiply = [&](const int (&addr)[4][4]) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
          float a[4];
#pragma unroll
          for (int e = 0; e < 4; e++) a[e] = rb[addr[q][e]];
#pragma unroll
          for (int e = 0; e < 4; e++)
#pragma unroll
            for (int j = 0; j < TN; j++)
              acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[q][e][j], acc[j], 0, 0, 0);
        }
      };
      if (strip == wave) {
        multiply(a_first);
      } else {
        int addr[4][4];
        strip_addresses(strip, addr);
        multiply(addr);
      }
      // accumulator register r holds pixel 8*(r/4) + 4*(lane/32) + r%4 of the strip
      const int px0 = strip * 32 + 4 * g;
      if (bias_row || alpha_row || prelu) {
        const int px0_ = opaque(px0), l32_ = opaque(l32);
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int px = px0_ + 8 * (r >> 2) + (r & 3);
#pragma unroll
          for (int j = 0; j < TN; j++) {
            const int col = 32 * j + l32_;
            if (px < p.OW && col < p.N) {
              const int at = px * p.N + col;
              const float bv = bias_row ? bias_row[at] : bias_c[j];
              const float al = alpha_row ? alpha_row[at] : alpha_c[j];
              crow[at] = activate(acc[j][r] + bv, act, al);
            }
          }
        }
      } else {
        // one add per store: the lane's base offset (out of range for a column past N) plus
        // the register's pixel offset, which is the same for all lanes (that offset as the
        // store's scalar offset instead was measured: 42.8 us against 33.3)
        unsigned lane_at[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) {
          const int col = 32 * j + l32;
          lane_at[j] = col < p.N ? (unsigned)((px0 * p.N + col) * 4) : OOB_OFFSET;
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const unsigned px_at = (unsigned)((8 * (r >> 2) + (r & 3)) * p.N * 4);
#pragma unroll
          for (int j = 0; j < TN; j++) {
            const float v = clamp(acc[j][r] + bias_c[j], cl);
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), rout,
                                                  (int)(lane_at[j] + px_at), 0, STORE_WRITE_THROUGH);
          }
        }
      }
    }
  };

  if constexpr (SPLIT) {
    // Wavefronts 0..3 multiply and store, wavefronts 4 and 5 only load: a wavefront that does
    // both finds the acknowledgements of its stores in front of its loads' data (they share one
    // counter) and waits a trip to memory per row.  The loaders keep two rows in flight and
    // fill the LDS buffer that is not being read; one barrier per row hands the buffers over.
    __syncthreads();
    for (int it = 0; it < count; it += 2) {
      compute_row(n, oh, rows);
      advance(n, oh);
      __syncthreads();
      if (it + 1 >= count) break;
      compute_row(n, oh, rows + SPLIT_BUF);
      advance(n, oh);
      __syncthreads();
    }
  } else {
    // Input rows of any length, staged in passes by the wavefronts that also multiply.
    for (int row = row_first; row < row_end; row += row_step, advance(n, oh)) {
      __syncthreads();  // the previous row's readers are done
      for (int i0 = opaque(tid); i0 < stage_n; i0 += 256 * 8) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const int i = i0 + u * 256;
          const int kh = i / row_floats, r = i - kh * row_floats;
          const int ih = oh * p.sh - p.pt + kh * p.dh;
          const int e = r - p.pl * p.Cin;
          const bool ok = i < stage_n && (unsigned)ih < (unsigned)p.H && (unsigned)e < (unsigned)row_in;
          const long long at = ok ? ((long long)n * p.H + ih) * row_in + e : 0;
          const float x = p.A[at];
          t[u] = ok ? x : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const int i = i0 + u * 256;
          if (i < stage_n) rows[i] = t[u];
        }
      }
      __syncthreads();
      compute_row(n, oh, rows);
    }
  }
}

// Products of many rows with a small right-hand side (K <= 128, K * N floats <= 64 KB: the
// first pointwise layers of a MobileNet are [802816, 32] x [32, 64] ... [200704, 128] x
// [128, 128]).  A tile of such a product has only K / 16 steps, so the tiled kernel above
// spends its time filling and draining its pipeline.  Here B is copied into LDS once per
// workgroup, already in operand order, and every wavefront streams blocks of 32 rows of A
// straight from memory into the registers that the MFMA reads (lane = row, 16-byte loads of 4
// consecutive k), with the next block's loads in flight while the current one is multiplied and
// stored.  Same summation-order permutation as above: MFMA e of group q multiplies
// k = 8q + e (lanes 0..31) and k = 8q + 4 + e (lanes 32..63).
template <int KQ, int NJ>
__global__ __launch_bounds__(256, 2) void gemm_rowstream_kernel(const GemmArgs p, int n_blocks,
                                                                int quant) {
  constexpr int K = 8 * KQ, N = 32 * NJ;
  extern __shared__ __attribute__((aligned(16))) float bl[];  // B as [K / 4][N][4] = (k / 4, col, k % 4)
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  {
    // B into operand order: an item is 4 consecutive k of one column (one 16-byte LDS write,
    // lanes side by side along the column); all loads first, they are independent
    constexpr int PER = K / 4 * N / 256;
    auto fill = [&](auto quant_tag) {
      f32x4 w[PER];
#pragma unroll
      for (int u = 0; u < PER; u++) {
        const int item = tid + 256 * u;
        const int k4 = item / N, col = item - k4 * N;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int at = (4 * k4 + e) * N + col;
          if (decltype(quant_tag)::value)
            w[u][e] = dequant(static_cast<const unsigned char*>(p.B)[at], p.qscale, p.qmin);
          else
            w[u][e] = static_cast<const float*>(p.B)[at];
        }
      }
#pragma unroll
      for (int u = 0; u < PER; u++)
        *reinterpret_cast<f32x4*>(&bl[(tid + 256 * u) * 4]) = w[u];
    };
    if (quant) fill(std::true_type{});
    else fill(std::false_type{});
  }
  float bias_c[NJ];  // of column 32j + l32
#pragma unroll
  for (int j = 0; j < NJ; j++) {
    const int col = 32 * j + l32;
    bias_c[j] = 0.f;
    if (p.bias_kind == TFHIP_BCAST_SCALAR) bias_c[j] = p.bias[0];
    if (p.bias_kind == TFHIP_BCAST_COLUMN) bias_c[j] = p.bias[col];
  }
  const Clamp cl = clamp_of(p.act);  // (prelu never comes here: the tiled kernel takes it)
  __syncthreads();

  // The 32-row blocks are cut into 8 runs, one per XCD (workgroup b runs on XCD b % 8; the grid
  // is a multiple of 8): the kernels before and after this one split their rows the same way,
  // so what an XCD leaves in its L2 is what the same XCD reads next.  Within its run this
  // wavefront takes blocks first, first + stride, ... (the same for all its lanes).
  const int xcd = (int)blockIdx.x & 7;
  const int per = n_blocks >> 3, rem = n_blocks & 7;
  const int run0 = xcd * per + (xcd < rem ? xcd : rem);
  const int run1 = run0 + per + (xcd < rem ? 1 : 0);
  const int first = __builtin_amdgcn_readfirstlane(run0 + ((int)blockIdx.x >> 3) * 4 + wave);
  const int stride = ((int)gridDim.x >> 3) * 4;
  const unsigned a_at = (unsigned)((l32 * K + 4 * g) * 4);
  const unsigned c_at = (unsigned)((4 * g * N + l32) * 4);

  // One descriptor per block over its rows that exist: rows at or past M (and whole blocks
  // past the end of the run) read as zeros and their stores are dropped.
  auto load = [&](int blk, f32x4 (&a)[KQ]) {
    const long long row0 = (long long)(p.reverse ? run0 + run1 - 1 - blk : blk) * 32;
    const long long left = (long long)p.M - row0;
    const unsigned bytes = blk >= run1 ? 0u : (unsigned)((left < 32 ? left : 32) * K * 4);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.A + row0 * K, bytes);
#pragma unroll
    for (int q = 0; q < KQ; q++) a[q] = buffer_load_f32x4(ra, a_at + 32 * q);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto multiply_store = [&](int blk, const f32x4 (&a)[KQ]) {
    f32x16 acc[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[j][r] = 0.f;
    // B operands of group q + 1 are read while group q is multiplied; the order is pinned so
    // that no more than two groups of them are ever live
    f32x4 b[2][NJ];
    auto read_b = [&](int q, f32x4 (&dst)[NJ]) {
#pragma unroll
      for (int j = 0; j < NJ; j++)
        dst[j] = *reinterpret_cast<const f32x4*>(&bl[((q * 2 + g) * N + 32 * j + l32) * 4]);
    };
    read_b(0, b[0]);
#pragma unroll
    for (int q = 0; q < KQ; q++) {
      if (q + 1 < KQ) read_b(q + 1, b[(q + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int e = 0; e < 4; e++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q][e], b[q & 1][j][e], acc[j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    // accumulator register r holds row 8*(r/4) + 4*(lane/32) + r%4 of the block, column l32 of
    // column block j: a store writes two runs of 32 consecutive floats.  The part of the address
    // that is known at compile time rides in the scalar offset, which the range check of the
    // descriptor does not see: in the one block that is cut short by M the rows past the end are
    // therefore turned away through the lane's own offset.
    const long long row0 = (long long)(p.reverse ? run0 + run1 - 1 - blk : blk) * 32;
    const int left = (int)((long long)p.M - row0 < 32 ? (long long)p.M - row0 : 32);
    const __amdgpu_buffer_rsrc_t rc = make_rsrc(p.C + row0 * N, (unsigned)(left * N * 4));
    auto store = [&](auto whole_tag) {
      constexpr bool whole = decltype(whole_tag)::value;
#pragma unroll
      for (int r = 0; r < 16; r++)
#pragma unroll
        for (int j = 0; j < NJ; j++) {
          const int row_c = 8 * (r >> 2) + (r & 3);  // + 4 * g
          const float v = clamp(acc[j][r] + bias_c[j], cl);
          const unsigned at = whole || row_c + 4 * g < left ? c_at : OOB_OFFSET;
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), rc, (int)at,
                                                /*scalar offset=*/(row_c * N + 32 * j) * 4, 0);
        }
    };
    if (left == 32) store(std::true_type{});
    else store(std::false_type{});
  };

  f32x4 a0[KQ], a1[KQ];
  load(first, a0);
  for (int blk = first; blk < run1; blk += 2 * stride) {
    load(blk + stride, a1);
    multiply_store(blk, a0);
    load(blk + 2 * stride, a0);
    if (blk + stride < run1) multiply_store(blk + stride, a1);
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

// How one tile shape would run a problem: whole tiles, tiles split along K, and a cost.
struct Plan {
  int grid = 0, full_tiles = 0, tail_tiles = 0, splits = 1, kt_per = 0, tiles_m = 0, tiles_n = 0;
  int minis = 0;  // > 0: the tail tiles run as this many 16 x 16 pieces each (no split over workgroups)
  double cost = 0;
};

// Cost of a plan in microseconds: matrix-core time of the busiest CU (its workgroups share
// the CU's 4 matrix pipes: 2 flop * 256 MACs per clock at 2.4 GHz = 0.614 Mflop/us), and for a
// split along K the partial tiles written and read back (about 4 TB/s) plus the finishing
// kernel (a second launch costs about 5 us in a busy stream; summing the partials inside the
// first kernel instead was tried and is slower: a device-scope fence writes back the whole L2
// of the XCD it is issued on).  The numbers need only rank the candidates of one problem.
static void price_plan(Plan& pl, int bm, int bn, int cus, double efficiency, int k_tiles) {
  const double tile_us = 2.0 * bm * bn * (double)k_tiles * BK / 0.614e6 / efficiency;
  const double per_split = (double)pl.kt_per / k_tiles;
  const long long split_wgs = (long long)pl.tail_tiles * pl.splits;
  pl.cost = tile_us * (ceil_div(pl.full_tiles, cus) +
                       (pl.splits > 1 ? per_split * ceil_div(split_wgs, cus)
                                      : (double)ceil_div(pl.tail_tiles, cus)));
  // a k step is a chain of global load, LDS store, barrier, LDS read and MFMAs: about 0.4 us
  // even when the matrix cores would be done sooner, which is what a sparse grid pays
  const double chain_us = 0.4 * (pl.full_tiles > 0 || pl.splits == 1 ? k_tiles : pl.kt_per);
  if (pl.cost < chain_us) pl.cost = chain_us;
  if (pl.splits > 1) pl.cost += 6.0 + 2.0 * split_wgs * (double)bm * bn * sizeof(float) / 4.0e6;
}

// k ranges for `tail` tiles cut `want` ways: at least 4 steps each (whole 48-wide blocks for
// matMul).  Returns false when that leaves a single range.
static bool split_tail(Plan& pl, int tail, int want, int k_tiles, bool kblocked) {
  const int unit = kblocked ? TILES_PER_KBLOCK : 1;
  if (want < 2 || k_tiles < 8) return false;
  int per = (int)ceil_div(k_tiles, want);
  if (per < 4) per = 4;
  per = (int)ceil_div(per, unit) * unit;
  pl.kt_per = per;
  pl.splits = (int)ceil_div(k_tiles, per);
  pl.tail_tiles = tail;
  return pl.splits > 1;
}

static Plan make_plan(const GemmArgs& p, int batch, int bm, int bn, int resident, int cus,
                      double efficiency, bool kblocked, bool minis_ok) {
  Plan pl;
  pl.tiles_m = (int)ceil_div(p.M, bm);
  pl.tiles_n = (int)ceil_div(p.N, bn);
  const int tiles = (int)((long long)pl.tiles_m * pl.tiles_n * batch);
  const int slots = cus * resident;
  const int k_tiles = (int)ceil_div(p.K, BK);
  // candidate 1: one workgroup per tile
  pl.full_tiles = tiles;
  pl.tail_tiles = 0;
  pl.splits = 1;
  pl.kt_per = k_tiles;
  pl.grid = tiles < 1 ? 1 : tiles;
  price_plan(pl, bm, bn, cus, efficiency, k_tiles);
  // candidate 2: fewer tiles than half the machine's workgroup slots: cut every tile
  if (tiles > 0 && tiles * 2 <= slots) {
    Plan sp = pl;
    sp.full_tiles = 0;
    if (split_tail(sp, tiles, slots / tiles, k_tiles, kblocked)) {
      sp.grid = sp.tail_tiles * sp.splits;
      price_plan(sp, bm, bn, cus, efficiency, k_tiles);
      if (sp.cost < pl.cost) pl = sp;
    }
  }
  // candidate 3: whole rounds of one tile per CU, and the tiles left over (at most half a
  // round) cut so that every CU gets one short piece instead of some CUs a whole extra tile
  const int left = tiles % cus;
  if (tiles > cus && left > 0 && left * 2 <= cus) {
    Plan sp = pl;
    sp.full_tiles = tiles - left;
    if (split_tail(sp, left, cus / left, k_tiles, kblocked)) {
      sp.grid = sp.full_tiles + sp.tail_tiles * sp.splits;
      price_plan(sp, bm, bn, cus, efficiency, k_tiles);
      if (sp.cost < pl.cost) pl = sp;
    }
  }
  // candidate 4: whole rounds, and the tiles left over cut into pieces of 16 x 16, each a
  // workgroup whose wavefronts share K among themselves (kwaves_tile: no partial sums in
  // memory, no second launch).  The pieces are small enough to spread evenly over the CUs; they
  // run at about a third of the efficiency of a whole tile (operands straight from L2, no
  // reuse).  Measured on MI355X: [12544, 512] x [512, 512] in 64 x 64 tiles (6.125 per CU)
  // 53.1 us against 58.8 with a seventh tile on 32 CUs; [3136, 1024] x [1024, 512] 28.4
  // against 35.0; in 128 x 128 tiles, where more than half a round is left over, 94.0 against 67.1.
  if (minis_ok && tiles > cus && left > 0) {
    Plan sp = pl;
    sp.full_tiles = tiles - left;
    sp.tail_tiles = left;
    sp.splits = 1;
    sp.kt_per = k_tiles;
    sp.minis = (bm / 16) * (bn / 16);
    sp.grid = sp.full_tiles + (int)ceil_div(left, 8) * 8 * sp.minis;  // (see the kernel's tail branch)
    const double tile_us = 2.0 * bm * bn * (double)k_tiles * BK / 0.614e6 / efficiency;
    sp.cost = tile_us * (sp.full_tiles / cus + 3.0 * left / cus) + 1.0;
    if (sp.cost < pl.cost) pl = sp;
  }
  return pl;
}

// How many column groups the tiles of an unbatched row-major product are dealt in.  Workgroup b
// runs on XCD b % 8 and every XCD has an L2 of its own (4 MiB), so with the tiles numbered row by
// row an L2 reads an eighth of A and all of B: A + 8 B over the chip.  Numbered in c column groups
// it reads c / 8 of A and 1 / c of B: c A + (8 / c) B.  A share of B that does not fit half an L2
// next to the stream of A is fetched more than once (measured: [3136, 1024] x [1024, 1024], B =
// 4 MiB, fetched 46 to 67 MiB over the chip against the 44 the formula gives), hence the
// surcharge.  c must divide the tile columns into groups of a power of two, and has to save 15 %
// to be taken.  Measured (FETCH_SIZE over the chip, every choice forced in turn): the product
// above 67.6 MiB with c = 1, 48.3 with c = 2 (the formula gives 40.6, and the 16 leftover tiles
// that run as 16 x 16 pieces add 8), 64.9 with c = 4, durations 51.6 / 52.0 / 52.4 us;
// [3136, 512] x [512, 1024] 23.2 / 23.4 / 31.7 MiB; [12544, 512] x [512, 512] 36.2 / 57.0 / 105.5.
static int choose_col_groups(const GemmArgs& p, const Plan& pl, double b_elem_bytes) {
  if (pl.splits > 1 || pl.tiles_m < 16) return 1;
  const double a_bytes = 4.0 * p.M * p.K, b_bytes = b_elem_bytes * p.K * p.N;
  int best = 1;
  double best_cost = 0;
  for (int c = 1; c <= 4; c *= 2) {
    if (pl.tiles_n % c) break;
    const int w = pl.tiles_n / c;
    if (w & (w - 1)) break;
    const double share = b_bytes / c;
    const double cost = c * a_bytes + (8.0 / c) * b_bytes * (share > 2.0 * (1 << 20) ? 1.5 : 1.0);
    if (c == 1 || cost < 0.85 * best_cost) {
      best = c;
      best_cost = cost;
    }
  }
  return best;
}

// Scratch memory of tfhip_matmul_noalloc: a static device array, one copy per GPU, that takes
// the place of the pool block in which a product cut along K keeps its partial tiles.  Host
// code reaches it only through the address hipGetSymbolAddress returns for the current
// device (the array's name is not a device address on the host), asked once per device.
constexpr size_t kScratchBytes = 8u << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mu;

int scratch_init(tfhip_ctx* ctx) {
  if (ctx->device < 0 || ctx->device >= kMaxDevices)
    return ctx->fail(TFHIP_EINVAL, "device index %d beyond %d", ctx->device, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[ctx->device]) {
    void* ptr = nullptr;
    // (the context's device is current: tfhip_init has just selected it)
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return ctx->fail(TFHIP_EDEVICE, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    }
    g_scratch_ptr[ctx->device] = ptr;
  }
  ctx->scratch = g_scratch_ptr[ctx->device];
  return TFHIP_OK;
}

static void* scratch_address(tfhip_ctx* ctx) {
  if (!ctx->scratch) ctx->fail(TFHIP_EDEVICE, "static scratch memory was not set up");
  return ctx->scratch;
}

template <class T, int AMODE, int BMODE, bool KBLOCKED, bool FAST>
static int resident_blocks(tfhip_ctx* ctx) {
  static int cached = 0;
  if (!cached) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &n, gemm_kernel<T::WM, T::WN, T::TM, T::TN, AMODE, BMODE, KBLOCKED, FAST>,
            T::WM * T::WN * 64, 0) != hipSuccess || n < 1) {
      (void)hipGetLastError();
      n = 1;
    }
    cached = n;
  }
  (void)ctx;
  return cached;
}

template <class T, int AMODE, int BMODE, bool KBLOCKED, bool FAST>
static int launch_cfg(tfhip_ctx* ctx, GemmArgs& p, const Plan& pl) {
  static const char* const a_names[] = {"rowmajor", "transposed", "im2col", "im2col_up", "im2col_t"};
  static const char* const b_names[] = {"f32", "f32t", "u8"};
  ctx->name_kernel("gemm_%dx%d_%s_%s%s%s", T::BM, T::BN,
           a_names[AMODE], b_names[BMODE], KBLOCKED ? "_kb48" : "",
           pl.minis ? "_tail16" : pl.splits > 1 ? (pl.full_tiles ? "_tailk" : "_splitk") : "");
  if (!FAST) strncat(ctx->last_kernel, "_unaligned", sizeof ctx->last_kernel - strlen(ctx->last_kernel) - 1);
  p.tiles_m = pl.tiles_m;
  p.tiles_n = pl.tiles_n;
  p.tiles_n_shift = (pl.tiles_n & (pl.tiles_n - 1)) == 0 ? __builtin_ctz((unsigned)pl.tiles_n) : -1;
  p.col_groups = 1;
  p.cg_shift = 0;
  if (FAST && AMODE == A_ROWMAJOR && BMODE != B_TRANSPOSED && pl.tiles_m * pl.tiles_n == pl.full_tiles + pl.tail_tiles) {
    // (an unbatched product: the planner counted tiles_m * tiles_n tiles)
    p.col_groups = choose_col_groups(p, pl, BMODE == B_UINT8 ? 1.0 : 4.0);
    if (p.col_groups > 1) p.cg_shift = __builtin_ctz((unsigned)(pl.tiles_n / p.col_groups));
  }
  p.full_tiles = pl.full_tiles;
  p.tail_tiles = pl.tail_tiles;
  p.splits = pl.splits;
  p.kt_per = pl.kt_per;
  p.k_tiles = (int)ceil_div(p.K, BK);
  p.minis = pl.minis;
  p.mini_k_per = (int)ceil_div(ceil_div(p.K, T::WM * T::WN), 16) * 16;
  p.reverse = ctx->take_sweep();
  Temp partials(ctx);
  p.partials = nullptr;
  if (pl.splits > 1) {
    const size_t need = (size_t)pl.tail_tiles * pl.splits * T::BM * T::BN * sizeof(float);
    if (ctx->no_alloc) {
      // the partial tiles go into the library's static device array instead of a pool block
      if (need > kScratchBytes)
        return ctx->fail(TFHIP_ENOTSUP,
                         "matmul_noalloc: this product is cut along K and its partial tiles take "
                         "%zu bytes, more than the %zu bytes of static scratch memory; use "
                         "tfhip_matmul", need, kScratchBytes);
      p.partials = static_cast<float*>(scratch_address(ctx));
      if (!p.partials) return TFHIP_EDEVICE;
      // one array per device, two compute streams: behind the other stream's last use of it
      if (ctx->scratch_sidx >= 0 && ctx->scratch_sidx != ctx->cur) ctx->order(ctx->scratch_sidx, ctx->cur);
      ctx->scratch_sidx = ctx->cur;
      if (ctx->capturing) ctx->capture_used_scratch = true;
    } else {
      if (!partials.get(need)) return TFHIP_EDEVICE;
      p.partials = static_cast<float*>(partials.ptr);
    }
  }
  tfhip::launch(ctx, (gemm_kernel<T::WM, T::WN, T::TM, T::TN, AMODE, BMODE, KBLOCKED, FAST>),
                     dim3(pl.grid), dim3(T::WM * T::WN * 64), 0, p);
  TFHIP_LAUNCH_CHECK(ctx);
  if (pl.splits > 1) {
    const long long quads = (long long)pl.tail_tiles * T::BM * T::BN / 4;
    const long long blocks = ceil_div(quads, 256);
    const long long cap = (long long)ctx->num_cus * 8;
    tfhip::launch(ctx, splitk_finish_kernel, dim3((unsigned)(blocks > cap ? cap : blocks)), dim3(256),
                       0, p, T::BM, T::BN, pl.full_tiles);
    TFHIP_LAUNCH_CHECK_NAMED(ctx, "splitk_finish");
  }
  return TFHIP_OK;
}

// Tile choice: every shape is planned (grid, split along K, leftover tiles in small pieces) and
// priced, and the cheapest wins; ties go to the larger tile.  The efficiency per flop of a tile
// shape is measured on MI355X (every tile forced on every shape, interleaved, clocks warm).
// Row-major operands: [4096, 1024] x [1024, 1024], where every shape fills whole rounds, takes
// 77.0 us in 128 x 128 tiles, 80.7 in 128 x 64, 74.0 in 64 x 128 and 73.4 in 64 x 64 (four
// wavefronts of one 32 x 32 accumulator; seven workgroups share a CU, which hides latency better
// than a deeper pipeline in fewer, larger wavefronts); at [8192, 4096] x [4096, 4096] the large
// tile, with half the LDS traffic per flop, wins: 2086 / 2233 / 2219 / 2281 us.
// Implicit GEMM (the A tile is gathered, so reusing it over more columns pays): a 3 x 3
// convolution of 112 x 112 x 64 -> 128 takes 514 / 536 / 514 / 561 us, 56 x 56 x 128 -> 128
// 502 / 520 / 494 / 554.
template <int AMODE, int BMODE, bool KBLOCKED, bool FAST>
static int launch_mode(tfhip_ctx* ctx, GemmArgs& p, int batch) {
  using Big = TileCfg<4, 2, 1, 2>;     // 128 x 128, 8 wavefronts of 32 x 64
  using Mid = TileCfg<2, 2, 2, 1>;     // 128 x 64, 4 wavefronts of 64 x 32
  using Wide = TileCfg<2, 4, 1, 1>;    // 64 x 128, 8 wavefronts of 32 x 32
  using Thin = TileCfg<4, 1, 2, 1>;    // 256 x 32, 4 wavefronts of 64 x 32 (N <= 32)
  using Small = TileCfg<2, 2, 1, 1>;   // 64 x 64, 4 wavefronts of 32 x 32
  constexpr int NCFG = 5;
  const int cus = ctx->num_cus;
  // (what kwaves_tile needs: unbatched row-major operands it can read with range-checked loads)
  const bool mk = FAST && AMODE == A_ROWMAJOR && BMODE != B_TRANSPOSED && batch == 1 &&
                  p.ldb == p.N && (p.K & 3) == 0 && (p.lda & 3) == 0 &&
                  (long long)p.M * p.N <= 0x7fffffffLL;
  Plan plans[NCFG];
  const bool gathered = AMODE == A_IM2COL || AMODE == A_IM2COL_UP || AMODE == A_IM2COL_T;
  const bool huge = (double)p.M * p.N * p.K * batch >= 5e10;
  const double eff_big = gathered ? 0.98 : huge ? 1.00 : 0.95;
  const double eff_mid = gathered ? 0.95 : huge ? 0.93 : 0.91;
  const double eff_wide = gathered ? 1.00 : huge ? 0.94 : 0.99;
  const double eff_small = gathered ? 0.92 : huge ? 0.92 : 1.00;
  plans[0] = make_plan(p, batch, Big::BM, Big::BN, resident_blocks<Big, AMODE, BMODE, KBLOCKED, FAST>(ctx), cus, eff_big, KBLOCKED, mk);
  plans[1] = make_plan(p, batch, Mid::BM, Mid::BN, resident_blocks<Mid, AMODE, BMODE, KBLOCKED, FAST>(ctx), cus, eff_mid, KBLOCKED, mk);
  plans[2] = make_plan(p, batch, Wide::BM, Wide::BN, resident_blocks<Wide, AMODE, BMODE, KBLOCKED, FAST>(ctx), cus, eff_wide, KBLOCKED, mk);
  plans[3] = make_plan(p, batch, Thin::BM, Thin::BN, resident_blocks<Thin, AMODE, BMODE, KBLOCKED, FAST>(ctx), cus, 0.80, KBLOCKED, mk);
  plans[4] = make_plan(p, batch, Small::BM, Small::BN, resident_blocks<Small, AMODE, BMODE, KBLOCKED, FAST>(ctx), cus, eff_small, KBLOCKED, mk);
  // rows and columns beyond M and N are wasted matrix-core work: charge it
  const int bns[NCFG] = {Big::BN, Mid::BN, Wide::BN, Thin::BN, Small::BN};
  const int bms[NCFG] = {Big::BM, Mid::BM, Wide::BM, Thin::BM, Small::BM};
  int best = -1;
  for (int i = 0; i < NCFG; i++) {
    const double useful = ((double)p.N / (ceil_div(p.N, bns[i]) * bns[i])) *
                          ((double)p.M / (ceil_div(p.M, bms[i]) * bms[i]));
    plans[i].cost /= useful;
    if (best < 0 || plans[i].cost < plans[best].cost) best = i;
  }
  switch (best) {
    case 0: return launch_cfg<Big, AMODE, BMODE, KBLOCKED, FAST>(ctx, p, plans[0]);
    case 1: return launch_cfg<Mid, AMODE, BMODE, KBLOCKED, FAST>(ctx, p, plans[1]);
    case 2: return launch_cfg<Wide, AMODE, BMODE, KBLOCKED, FAST>(ctx, p, plans[2]);
    case 3: return launch_cfg<Thin, AMODE, BMODE, KBLOCKED, FAST>(ctx, p, plans[3]);
    default: return launch_cfg<Small, AMODE, BMODE, KBLOCKED, FAST>(ctx, p, plans[4]);
  }
}

// The row-streaming kernel for the shapes it is built for; returns -1 when the product is not
// one of them (the tiled kernels take it then).
template <int KQ, int NJ>
static int launch_rowstream_cfg(tfhip_ctx* ctx, const GemmArgs& p, int quant) {
  auto kernel = gemm_rowstream_kernel<KQ, NJ>;
  const size_t lds = (size_t)KQ * 8 * NJ * 32 * sizeof(float);
  static int per_cu = 0;
  if (!per_cu) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, lds) != hipSuccess || n < 1) {
      (void)hipGetLastError();
      n = 1;
    }
    per_cu = n;
  }
  const int n_blocks = (int)ceil_div(p.M, 32);
  const long long slots = (long long)ctx->num_cus * per_cu / 8 * 8;  // a multiple of the XCD count
  const long long want = ceil_div(ceil_div(n_blocks, 8), 4) * 8;
  ctx->name_kernel("gemm_rowstream_k%dxn%d_%s", KQ * 8, NJ * 32,
           quant ? "u8" : "f32");
  GemmArgs q = p;
  q.reverse = ctx->take_sweep();
  tfhip::launch(ctx, kernel, dim3((unsigned)(want < slots || slots < 8 ? want : slots)), dim3(256),
                     lds, q, n_blocks, quant);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

static int launch_rowstream(tfhip_ctx* ctx, const GemmArgs& p, int batch, int amode, int bmode) {
  if (batch != 1 || amode != A_ROWMAJOR || (bmode != B_ROWMAJOR && bmode != B_UINT8)) return -1;
  if (p.lda != p.K || p.ldb != p.N || !p.a_vec || !p.b_vec) return -1;
  if (p.bias_kind == TFHIP_BCAST_FULL || p.act == TFHIP_ACT_PRELU) return -1;
  // enough 32-row blocks to give every wavefront of a full machine several
  if ((long long)p.M < (long long)ctx->num_cus * 8 * 32 * 3) return -1;
  const int quant = bmode == B_UINT8;
#define TFHIP_ROWSTREAM(KK, NN) \
  if (p.K == KK && p.N == NN) return launch_rowstream_cfg<KK / 8, NN / 32>(ctx, p, quant);
  // Measured on MI355X inside a batch-64 MobileNet: [802816, 32] x [32, 64] (bound by HBM) runs
  // 58 us here against 66 us tiled; at K = 64 and 128 with N = 128 the tiled kernel, whose
  // tiles balance better over the CUs (24.5 per CU against 6.1 row blocks per SIMD), stays
  // 4 us ahead, so those shapes are not routed here.
  TFHIP_ROWSTREAM(32, 64)
#undef TFHIP_ROWSTREAM
  return -1;
}

// The kernel that cuts K over the wavefronts of a workgroup, for the products it suits;
// returns -1 for the others.  Measured on MI355X against the tiled kernels (which cut such
// products along K over workgroups and add the pieces in a second kernel): [256, 512] x
// [512, 256] 4.0 us against 9.8, [196, 512] x [512, 512] 5.1 against 10.0, [64, 1024] x
// [1024, 1000] 6.5 against 10.7, [512, 512] x [512, 512] 8.8 against 13.8; it runs at about
// 3 us + 14.5 us per 2^20 (tiles x K), its operands coming out of L2 without reuse, and meets
// the tiled kernels there ([1024, 1024] x [1024, 256]: 17.6 against 17.9).  Beyond 256 k per
// wavefront a workgroup waits for memory more than twice and loses ([128, 4096] x [4096, 128]:
// 16.6 against 13.8).  With more than 4 tiles per CU the tiled kernels have enough whole tiles.
static int launch_kwaves(tfhip_ctx* ctx, const GemmArgs& p, int batch, int amode, int bmode,
                         long long a_bytes, long long b_bytes) {
  if (batch != 1 || amode != A_ROWMAJOR || (bmode != B_ROWMAJOR && bmode != B_UINT8)) return -1;
  if (!p.a_vec || p.ldb != p.N || (p.K & 3) || (p.lda & 3)) return -1;
  if (a_bytes > 0x7fffffffLL || b_bytes > 0x7fffffffLL) return -1;
  if (p.M < 1 || p.N < 1 || (long long)p.M * p.N > 0x7fffffffLL) return -1;
  const long long tiles = ceil_div(p.M, 16) * ceil_div(p.N, 16);
  if (p.K < 128 || p.K > 2048 || tiles > 4 * ctx->num_cus || tiles * p.K > (1LL << 20)) return -1;
  GemmArgs q = p;
  q.a_bytes = (unsigned)a_bytes;
  q.b_bytes = (unsigned)b_bytes;
  q.tiles_m = (int)ceil_div(p.M, 16);
  q.tiles_n = (int)ceil_div(p.N, 16);
  const int k_per = (int)ceil_div(ceil_div(p.K, 8), 16) * 16;
  // (see the kernel: pairs of tile columns dealt to the 8 XCDs when there are enough of them)
  const int by_columns = q.tiles_n >= 16;
  const long long grid = by_columns ? 8 * ceil_div(ceil_div(q.tiles_n, 2), 8) * 2 * q.tiles_m : tiles;
  ctx->name_kernel("gemm_16x16_kwaves_%s", bmode == B_UINT8 ? "u8" : "f32");
  if (bmode == B_UINT8)
    tfhip::launch(ctx, gemm_kwaves_kernel<true>, dim3((unsigned)grid), dim3(512), 0, q, k_per, by_columns);
  else
    tfhip::launch(ctx, gemm_kwaves_kernel<false>, dim3((unsigned)grid), dim3(512), 0, q, k_per, by_columns);
  TFHIP_LAUNCH_CHECK(ctx);
  return TFHIP_OK;
}

static int launch_gemm(tfhip_ctx* ctx, GemmArgs& p, int batch, int amode, int bmode,
                       bool kblocked) {
  {
    const int rc = launch_rowstream(ctx, p, batch, amode, bmode);
    if (rc >= 0) return rc;
  }
  if ((long long)p.N * 256 >= (1LL << 31))
    return ctx->fail(TFHIP_ENOTSUP, "matmul/conv2d: more than 2^23 output columns");
  // Byte extents of one batch entry of A and B, for the range check of the buffer loads.
  long long a_el, b_el;
  if (amode == A_ROWMAJOR) a_el = (long long)(p.M - 1) * p.lda + p.K;
  else if (amode == A_TRANSPOSED) a_el = (long long)(p.K - 1) * p.lda + p.M;
  else if (amode == A_IM2COL_T)
    a_el = p.OH * p.OW > 0 ? (long long)(p.K / (p.OH * p.OW)) * p.H * p.W * p.Cin : 0;
  else a_el = p.OH * p.OW > 0 ? (long long)(p.M / (p.OH * p.OW)) * p.H * p.W * p.Cin : 0;
  if (bmode == B_TRANSPOSED) b_el = (long long)(p.N - 1) * p.ldb + p.K;
  else b_el = (long long)(p.K - 1) * p.ldb + p.N;
  const long long a_bytes = a_el * 4, b_bytes = b_el * (bmode == B_UINT8 ? 1 : 4);
  const long long lim = 0x7fffffffLL;
  // (an empty contraction has no readable operand bytes: keep it on the guarded path)
  const bool fast = p.a_vec && p.b_vec && p.K > 0 && p.M > 0 && p.N > 0 && a_bytes <= lim &&
                    b_bytes <= lim;
  {
    const int rc = launch_kwaves(ctx, p, batch, amode, bmode, a_bytes, b_bytes);
    if (rc >= 0) return rc;
  }
  p.a_bytes = fast ? (unsigned)a_bytes : 0;
  p.b_bytes = fast ? (unsigned)b_bytes : 0;
#define TFHIP_CASE(AM, BM_, KB)                                \
  if (amode == AM && bmode == BM_ && kblocked == KB)           \
    return fast ? launch_mode<AM, BM_, KB, true>(ctx, p, batch) \
                : launch_mode<AM, BM_, KB, false>(ctx, p, batch);
  TFHIP_CASE(A_ROWMAJOR, B_ROWMAJOR, true)
  TFHIP_CASE(A_ROWMAJOR, B_TRANSPOSED, true)
  TFHIP_CASE(A_ROWMAJOR, B_UINT8, true)
  TFHIP_CASE(A_TRANSPOSED, B_ROWMAJOR, true)
  TFHIP_CASE(A_TRANSPOSED, B_TRANSPOSED, true)
  TFHIP_CASE(A_ROWMAJOR, B_ROWMAJOR, false)
  TFHIP_CASE(A_ROWMAJOR, B_UINT8, false)
  TFHIP_CASE(A_IM2COL, B_ROWMAJOR, false)
  TFHIP_CASE(A_IM2COL, B_UINT8, false)
  TFHIP_CASE(A_IM2COL_UP, B_ROWMAJOR, false)
  TFHIP_CASE(A_IM2COL_T, B_ROWMAJOR, false)
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

static int matmul_impl(tfhip_ctx* ctx, int64_t a, int64_t b, int64_t out, int batch,
                            int m, int n, int k, int transpose_a, int transpose_b,
                            int64_t bias, int bias_kind, int act, int64_t prelu,
                            int prelu_kind, const tfhip_qparams* q);

extern "C" int tfhip_matmul(tfhip_ctx* ctx, int64_t a, int64_t b, int64_t out, int batch,
                            int m, int n, int k, int transpose_a, int transpose_b,
                            int64_t bias, int bias_kind, int act, int64_t prelu,
                            int prelu_kind, const tfhip_qparams* q) {
  if (!ctx) return TFHIP_EINVAL;
  return matmul_impl(ctx, a, b, out, batch, m, n, k, transpose_a, transpose_b, bias, bias_kind,
                     act, prelu, prelu_kind, q);
}

// The same product for callers that must not allocate device memory.  Nothing here or below
// takes a block from the pool or asks the driver for memory: operands have to be stored as
// float32 already (a converted copy would need a block), and the partial tiles of a product
// cut along K live in the static array `scratch`.
extern "C" int tfhip_matmul_noalloc(tfhip_ctx* ctx, int64_t a, int64_t b, int64_t out, int batch,
                                    int m, int n, int k, int transpose_a, int transpose_b,
                                    int64_t bias, int bias_kind, int act, int64_t prelu,
                                    int prelu_kind, const tfhip_qparams* q) {
  if (!ctx) return TFHIP_EINVAL;
  const int64_t ids[4] = {a, b, bias_kind != TFHIP_BCAST_NONE ? bias : -1,
                          (act == TFHIP_ACT_PRELU && prelu_kind != TFHIP_BCAST_NONE) ? prelu : -1};
  for (int i = 0; i < 4; i++) {
    if (ids[i] < 0 && i >= 2) continue;
    TFHIP_GET(ctx, buf, ids[i]);
    if (buf->dtype != TFHIP_FLOAT32 && !(i == 1 && buf->dtype == TFHIP_UINT8Q))
      return ctx->fail(TFHIP_ENOTSUP, "matmul_noalloc: operand %d is not stored as float32 (a "
                                      "converted copy would need device memory); use tfhip_matmul",
                       i);
  }
  ctx->no_alloc = true;
  const int rc = matmul_impl(ctx, a, b, out, batch, m, n, k, transpose_a, transpose_b, bias,
                             bias_kind, act, prelu, prelu_kind, q);
  ctx->no_alloc = false;
  return rc;
}

static int matmul_impl(tfhip_ctx* ctx, int64_t a, int64_t b, int64_t out, int batch,
                            int m, int n, int k, int transpose_a, int transpose_b,
                            int64_t bias, int bias_kind, int act, int64_t prelu,
                            int prelu_kind, const tfhip_qparams* q) {
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
  if (amode == A_IM2COL && !p.a_vec && p.K >= 1 && p.K <= 32 && p.N <= 64 &&
      (int64_t)ci->in_h * ci->in_w * ci->in_c < (1LL << 31) &&
      (int64_t)ci->out_w * ci->out_c < (1LL << 31)) {
    // columns the output row reads, from -pad_left on
    const long long span = (long long)(ci->out_w - 1) * ci->stride_w +
                           (long long)(ci->filter_w - 1) * ci->dilation_w + 1;
    const long long row_floats = span * ci->in_c;
    const long long stage_n = row_floats * ci->filter_h;
    // loader wavefronts of their own when a row's input fits their registers (and 32-bit byte
    // offsets reach every element of an image)
    const bool split = stage_n <= 2048 && (int64_t)ci->in_h * ci->in_w * ci->in_c * 4 < (1LL << 30);
    const long long lds = split ? 2LL * SPLIT_BUF * (long long)sizeof(float)
                                : (stage_n + 1) * (long long)sizeof(float);  // + the zero slot
    if (lds <= 64 * 1024) {
      const int n_rows = ci->batch * ci->out_h;
      const unsigned threads = split ? 384 : 256;
      // one workgroup per resident slot: each walks its share of the output rows
      auto launch = [&](auto kernel, const char* name) {
        // resident workgroups per CU for this kernel and LDS size, asked once (the query
        // costs microseconds, which a batch-1 step would pay on every call)
        static std::map<std::pair<const void*, size_t>, int> resident;
        int& per_cu = resident[{reinterpret_cast<const void*>(kernel), (size_t)lds}];
        if (per_cu == 0 &&
            (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, (int)threads, (size_t)lds) !=
                 hipSuccess || per_cu < 1)) {
          (void)hipGetLastError();
          per_cu = 1;
        }
        const long long cap = (long long)ctx->num_cus * per_cu;
        unsigned grid = (unsigned)(n_rows < cap ? n_rows : cap);
        if (grid >= 64) grid &= ~7u;  // a multiple of the XCD count: one run of rows per XCD
        ctx->name_kernel("%s_%s", name, quant ? "u8" : "f32");
        ctx->sweep = 1;  // this kernel walks the rows forward: its consumer should start at the end
        tfhip::launch(ctx, kernel, dim3(grid), dim3(threads), (size_t)lds, p,
                           (int)row_floats, n_rows);
      };
      if (p.N <= 32) {
        if (split) {
          if (quant) launch(conv_smallk_kernel<1, true, true>, "conv_smallk_n32");
          else launch(conv_smallk_kernel<1, false, true>, "conv_smallk_n32");
        } else {
          if (quant) launch(conv_smallk_kernel<1, true, false>, "conv_smallk_n32_long");
          else launch(conv_smallk_kernel<1, false, false>, "conv_smallk_n32_long");
        }
      } else {
        if (split) {
          if (quant) launch(conv_smallk_kernel<2, true, true>, "conv_smallk_n64");
          else launch(conv_smallk_kernel<2, false, true>, "conv_smallk_n64");
        } else {
          if (quant) launch(conv_smallk_kernel<2, true, false>, "conv_smallk_n64_long");
          else launch(conv_smallk_kernel<2, false, false>, "conv_smallk_n64_long");
        }
      }
      TFHIP_LAUNCH_CHECK(ctx);
      return TFHIP_OK;
    }
  }
  return launch_gemm(ctx, p, 1, amode, quant ? B_UINT8 : B_ROWMAJOR, /*kblocked=*/false);
}

namespace tfhip {
// out[(kh, kw, co)][ci] = w[KH - 1 - kh][KW - 1 - kw][ci][co]: the filter as conv2dDerInput
// reads it (backend_cpu.ts:1741-1742), laid out as the row-major B operand of the product.
__global__ void flip_filter_kernel(const float* w, float* out, int KH, int KW, int Cin, int Cout) {
  const int total = KH * KW * Cin * Cout;
  for (int g = blockIdx.x * blockDim.x + threadIdx.x; g < total; g += gridDim.x * blockDim.x) {
    const int ci = g % Cin;
    int t = g / Cin;
    const int co = t % Cout;
    t /= Cout;
    const int kw = t % KW, kh = t / KW;
    out[g] = w[(((KH - 1 - kh) * KW + (KW - 1 - kw)) * Cin + ci) * Cout + co];
  }
}

// The same for the taps wr = r0 + sr * i (i < KHc), wc = c0 + sc * j (j < KWc) only:
// out[(i, j, co)][ci] = w[KH - 1 - wr][KW - 1 - wc][ci][co].
__global__ void flip_filter_taps_kernel(const float* w, float* out, int KH, int KW, int Cin,
                                        int Cout, int r0, int sr, int KHc, int c0, int sc, int KWc) {
  const int total = KHc * KWc * Cin * Cout;
  for (int g = blockIdx.x * blockDim.x + threadIdx.x; g < total; g += gridDim.x * blockDim.x) {
    const int ci = g % Cin;
    int t = g / Cin;
    const int co = t % Cout;
    t /= Cout;
    const int j = t % KWc, i = t / KWc;
    const int wr = r0 + sr * i, wc = c0 + sc * j;
    out[g] = w[(((KH - 1 - wr) * KW + (KW - 1 - wc)) * Cin + ci) * Cout + co];
  }
}

// dx[n, r0 + sr * i, c0 + sc * j, :] = src[(n, i, j), :] for a [batch * Hc * Wc, C] block.
__global__ void scatter_pixels_kernel(const float* __restrict__ src, float* __restrict__ dx,
                                      int64_t total, int Hc, int Wc, int C, int in_h, int in_w,
                                      int r0, int sr, int c0, int sc) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
    const int c = (int)(g % C);
    int64_t t = g / C;
    const int j = (int)(t % Wc);
    t /= Wc;
    const int i = (int)(t % Hc);
    const int64_t n = t / Hc;
    dx[((n * in_h + r0 + sr * i) * in_w + c0 + sc * j) * C + c] = src[g];
  }
}

static int check_backward_geometry(tfhip_ctx* ctx, const char* op, const tfhip_conv2d_info* ci) {
  if (ci->batch < 0 || ci->in_h < 0 || ci->in_w < 0 || ci->in_c < 0 || ci->out_h < 0 ||
      ci->out_w < 0 || ci->out_c < 0 || ci->filter_h <= 0 || ci->filter_w <= 0 ||
      ci->stride_h <= 0 || ci->stride_w <= 0)
    return ctx->fail(TFHIP_EINVAL, "%s: bad geometry", op);
  // the reference's gradient of conv2D rejects dilation rates above 1 (ops/conv.ts:240-243)
  if (ci->dilation_h != 1 || ci->dilation_w != 1)
    return ctx->fail(TFHIP_EINVAL, "%s: dilation rates greater than 1 are not yet supported", op);
  if ((int64_t)(ci->out_h - 1) * ci->stride_h - ci->pad_top >= ci->in_h ||
      (int64_t)(ci->out_w - 1) * ci->stride_w - ci->pad_left >= ci->in_w)
    return ctx->fail(TFHIP_EINVAL, "%s: output extent does not fit the input", op);
  return TFHIP_OK;
}
}  // namespace tfhip

extern "C" int tfhip_conv2d_der_input(tfhip_ctx* ctx, int64_t dy, int64_t filter, int64_t dx,
                                      const tfhip_conv2d_info* ci) {
  if (!ctx || !ci) return TFHIP_EINVAL;
  int rc;
  if ((rc = check_backward_geometry(ctx, "conv2dDerInput", ci))) return rc;
  TFHIP_GET(ctx, bdy, dy);
  TFHIP_GET(ctx, bw, filter);
  TFHIP_GET(ctx, bdx, dx);
  const int64_t x_n = (int64_t)ci->batch * ci->in_h * ci->in_w * ci->in_c;
  const int64_t w_n = (int64_t)ci->filter_h * ci->filter_w * ci->in_c * ci->out_c;
  const int64_t y_n = (int64_t)ci->batch * ci->out_h * ci->out_w * ci->out_c;
  if (bdy->numel != y_n || bw->numel != w_n || bdx->numel != x_n)
    return ctx->fail(TFHIP_EINVAL, "conv2dDerInput: buffer sizes do not match the geometry");
  if (bdx->dtype != TFHIP_FLOAT32 || bw->dtype == TFHIP_UINT8Q)
    return ctx->fail(TFHIP_EINVAL, "conv2dDerInput: dx must be float32 and the filter not quantised");
  if (x_n == 0) return TFHIP_OK;
  if ((int64_t)ci->batch * ci->in_h * ci->in_w > 0x7fffffffLL || w_n > 0x7fffffffLL)
    return ctx->fail(TFHIP_ENOTSUP, "conv2dDerInput: more than 2^31 input pixels");
  if (y_n == 0 || ci->out_c == 0) {  // nothing flows back
    return tfhip_fill(ctx, dx, 0.0);
  }
  Temp tdy(ctx), tw(ctx), tflip(ctx);
  GemmArgs p = {};
  const float* wf;
  if ((rc = as_f32(ctx, bdy, &tdy, &p.A))) return rc;
  if ((rc = as_f32(ctx, bw, &tw, &wf))) return rc;
  if (!tflip.get((size_t)w_n * sizeof(float))) return TFHIP_EDEVICE;
  {
    const int64_t blocks = ceil_div(w_n, 256);
    tfhip::launch(ctx, flip_filter_kernel, dim3((unsigned)(blocks > 4096 ? 4096 : blocks)), dim3(256),
                       0, wf, static_cast<float*>(tflip.ptr), ci->filter_h,
                       ci->filter_w, ci->in_c, ci->out_c);
    TFHIP_LAUNCH_CHECK(ctx);
  }
  p.B = tflip.ptr;
  p.C = static_cast<float*>(bdx->ptr);
  p.bias_kind = p.prelu_kind = TFHIP_BCAST_NONE;
  p.act = TFHIP_ACT_LINEAR;
  p.M = ci->batch * ci->in_h * ci->in_w;   // rows: input pixels
  p.N = ci->in_c;
  p.K = ci->filter_h * ci->filter_w * ci->out_c;
  p.ldb = ci->in_c;
  p.b_vec = aligned16(p.B) && (p.ldb % 4 == 0);
  // the image gathered from is dy: "input" geometry of the loader = dy, rows = dx pixels
  p.H = ci->out_h; p.W = ci->out_w; p.Cin = ci->out_c;
  p.OH = ci->in_h; p.OW = ci->in_w;
  p.KH = ci->filter_h; p.KW = ci->filter_w;
  p.sh = p.sw = 1;
  p.dh = p.dw = 1;
  p.pt = ci->filter_h - 1 - ci->pad_top;   // may be negative (padding larger than the filter)
  p.pl = ci->filter_w - 1 - ci->pad_left;
  p.up_h = ci->stride_h; p.up_w = ci->stride_w;
  p.a_vec = aligned16(p.A) && (ci->out_c % 4 == 0);
  // Stride above 1 on a large layer: dx pixels of one parity class (row % stride_h, column %
  // stride_w) all use the same subset of filter taps, and over that subset the gather is an
  // ordinary stride-1 convolution of dy.  One product per class on the forward kernels, none of
  // them multiplying the zeros of a stretched dy; the class results are scattered into dx.
  // (Small layers stay on the single stretched-gather launch: a class costs three launches.)
  if ((ci->stride_h > 1 || ci->stride_w > 1) &&
      2.0 * p.M * (double)p.N * p.K >= 8e9 && ci->stride_h * ci->stride_w <= 16) {
    const int top_pad = ci->filter_h - 1 - ci->pad_top, left_pad = ci->filter_w - 1 - ci->pad_left;
    auto mod = [](int a, int m) { return ((a % m) + m) % m; };
    bool some_empty = false;
    for (int r0 = 0; r0 < ci->stride_h && !some_empty; r0++)
      for (int c0 = 0; c0 < ci->stride_w; c0++)
        if (mod(top_pad - r0, ci->stride_h) >= ci->filter_h ||
            mod(left_pad - c0, ci->stride_w) >= ci->filter_w)
          some_empty = true;
    if (some_empty) {  // (a fill kernel, not a memset node: this may run inside a captured graph)
      const int rc_fill = tfhip_fill(ctx, dx, 0.0);
      if (rc_fill) return rc_fill;
    }
    for (int r0 = 0; r0 < ci->stride_h; r0++)
      for (int c0 = 0; c0 < ci->stride_w; c0++) {
        const int Hc = (int)ceil_div(ci->in_h - r0, ci->stride_h);
        const int Wc = (int)ceil_div(ci->in_w - c0, ci->stride_w);
        const int wr0 = mod(top_pad - r0, ci->stride_h), wc0 = mod(left_pad - c0, ci->stride_w);
        if (Hc <= 0 || Wc <= 0 || wr0 >= ci->filter_h || wc0 >= ci->filter_w) continue;
        const int KHc = (int)ceil_div(ci->filter_h - wr0, ci->stride_h);
        const int KWc = (int)ceil_div(ci->filter_w - wc0, ci->stride_w);
        const int64_t taps_n = (int64_t)KHc * KWc * ci->in_c * ci->out_c;
        const int64_t rows = (int64_t)ci->batch * Hc * Wc;
        Temp tsub(ctx), tout(ctx);
        if (!tsub.get((size_t)taps_n * sizeof(float)) ||
            !tout.get((size_t)(rows * ci->in_c) * sizeof(float)))
          return TFHIP_EDEVICE;
        const int64_t fb = ceil_div(taps_n, 256);
        tfhip::launch(ctx, flip_filter_taps_kernel, dim3((unsigned)(fb > 4096 ? 4096 : fb)), dim3(256),
                           0, wf, static_cast<float*>(tsub.ptr), ci->filter_h,
                           ci->filter_w, ci->in_c, ci->out_c, wr0, ci->stride_h, KHc, wc0,
                           ci->stride_w, KWc);
        TFHIP_LAUNCH_CHECK(ctx);
        GemmArgs q = p;
        q.B = tsub.ptr;
        q.C = static_cast<float*>(tout.ptr);
        q.M = (int)rows;
        q.K = KHc * KWc * ci->out_c;
        q.OH = Hc; q.OW = Wc;
        q.KH = KHc; q.KW = KWc;
        // dy row of tap i for class row a: a + i + (r0 - top_pad + wr0) / stride_h
        q.pt = -((r0 - top_pad + wr0) / ci->stride_h);
        q.pl = -((c0 - left_pad + wc0) / ci->stride_w);
        q.up_h = q.up_w = 1;
        q.b_vec = aligned16(q.B) && (q.ldb % 4 == 0);
        if ((rc = launch_gemm(ctx, q, 1, A_IM2COL, B_ROWMAJOR, /*kblocked=*/false))) return rc;
        const int64_t total = rows * ci->in_c;
        const int64_t sb = ceil_div(total, 256), cap = (int64_t)ctx->num_cus * 16;
        tfhip::launch(ctx, scatter_pixels_kernel, dim3((unsigned)(sb > cap ? cap : sb)), dim3(256), 0, static_cast<const float*>(tout.ptr), p.C, total, Hc, Wc,
                           ci->in_c, ci->in_h, ci->in_w, r0, ci->stride_h, c0, ci->stride_w);
        TFHIP_LAUNCH_CHECK(ctx);
      }
    strncat(ctx->last_kernel, "_by_parity", sizeof ctx->last_kernel - strlen(ctx->last_kernel) - 1);
    return TFHIP_OK;
  }
  if (ci->filter_h == 1 && ci->filter_w == 1 && ci->stride_h == 1 && ci->stride_w == 1 &&
      ci->pad_top == 0 && ci->pad_left == 0 && ci->out_h == ci->in_h && ci->out_w == ci->in_w) {
    // pointwise: dx = dy [pixels, out_c] x W^T [out_c, in_c], a plain product
    p.lda = ci->out_c;
    p.a_vec = aligned16(p.A) && (p.lda % 4 == 0);
    return launch_gemm(ctx, p, 1, A_ROWMAJOR, B_ROWMAJOR, /*kblocked=*/false);
  }
  return launch_gemm(ctx, p, 1, A_IM2COL_UP, B_ROWMAJOR, /*kblocked=*/false);
}

extern "C" int tfhip_conv2d_der_filter(tfhip_ctx* ctx, int64_t x, int64_t dy, int64_t dw,
                                       const tfhip_conv2d_info* ci) {
  if (!ctx || !ci) return TFHIP_EINVAL;
  int rc;
  if ((rc = check_backward_geometry(ctx, "conv2dDerFilter", ci))) return rc;
  TFHIP_GET(ctx, bx, x);
  TFHIP_GET(ctx, bdy, dy);
  TFHIP_GET(ctx, bdw, dw);
  const int64_t x_n = (int64_t)ci->batch * ci->in_h * ci->in_w * ci->in_c;
  const int64_t w_n = (int64_t)ci->filter_h * ci->filter_w * ci->in_c * ci->out_c;
  const int64_t y_n = (int64_t)ci->batch * ci->out_h * ci->out_w * ci->out_c;
  if (bx->numel != x_n || bdy->numel != y_n || bdw->numel != w_n)
    return ctx->fail(TFHIP_EINVAL, "conv2dDerFilter: buffer sizes do not match the geometry");
  if (bdw->dtype != TFHIP_FLOAT32)
    return ctx->fail(TFHIP_EINVAL, "conv2dDerFilter: dW must be float32");
  if (w_n == 0) return TFHIP_OK;
  if ((int64_t)ci->batch * ci->out_h * ci->out_w > 0x7fffffffLL || w_n > 0x7fffffffLL ||
      x_n > (1LL << 40))
    return ctx->fail(TFHIP_ENOTSUP, "conv2dDerFilter: more than 2^31 output pixels");
  if (x_n == 0 || y_n == 0) {
    return tfhip_fill(ctx, dw, 0.0);
  }
  Temp tx(ctx), tdy(ctx);
  GemmArgs p = {};
  const float* dyf;
  if ((rc = as_f32(ctx, bx, &tx, &p.A))) return rc;
  if ((rc = as_f32(ctx, bdy, &tdy, &dyf))) return rc;
  p.B = dyf;
  p.C = static_cast<float*>(bdw->ptr);
  p.bias_kind = p.prelu_kind = TFHIP_BCAST_NONE;
  p.act = TFHIP_ACT_LINEAR;
  p.M = ci->filter_h * ci->filter_w * ci->in_c;   // rows: (filter row, filter column, channel)
  p.N = ci->out_c;
  p.K = ci->batch * ci->out_h * ci->out_w;        // contraction over the output pixels
  p.ldb = ci->out_c;
  p.b_vec = aligned16(p.B) && (p.ldb % 4 == 0);
  p.H = ci->in_h; p.W = ci->in_w; p.Cin = ci->in_c;
  p.OH = ci->out_h; p.OW = ci->out_w;
  p.KH = ci->filter_h; p.KW = ci->filter_w;
  p.sh = ci->stride_h; p.sw = ci->stride_w;
  p.dh = p.dw = 1;
  p.pt = ci->pad_top; p.pl = ci->pad_left;
  p.a_vec = aligned16(p.A) && (ci->in_c % 4 == 0);
  return launch_gemm(ctx, p, 1, A_IM2COL_T, B_ROWMAJOR, /*kblocked=*/false);
}
