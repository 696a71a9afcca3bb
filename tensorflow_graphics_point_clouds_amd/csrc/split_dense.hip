// Dense products of the convolution layers on the bf16 matrix pipe with float32 accuracy
// (three-way operand splits, split.h).
#include <atomic>
#include <stdlib.h>

#include "common.h"
#include "mfma.h"
#include "split.h"

namespace mccnn {

static std::atomic<int> g_split_products{-1};

bool split_products_enabled() {
  int v = g_split_products.load(std::memory_order_relaxed);
  if (v < 0) {
    const char *env = getenv("MCCNN_DENSE_FP32");
    v = (env && env[0] && env[0] != '0') ? 0 : 1;
    g_split_products.store(v, std::memory_order_relaxed);
  }
  return v != 0;
}

// Gradient of the projection that enters a layer's final product (MCConv.py:187,
// KPConv.py:226-230): out[n, r] = sum_f x[n, f] * w[r, f], x = output gradient [N, F],
// w = dense final weights [R, F].  Write-bound (4 R bytes per point leave, 4 F arrive).
// A wavefront keeps the F columns of its 32 kCT rows of w in registers for its whole life as
// split B operands (96 registers) and streams tiles of 32 points through: the tile of x is
// split in registers, kCT * F / 16 * 6 matrix instructions, and the rows leave through an LDS
// transposition as contiguous runs.  The reduction index of matrix step ks, lane half h,
// element i is f = (F / 2) h + 8 ks + i, so that every lane fetches F / 2 consecutive floats
// of a row of x or w.
template <int F, int kCT>
__global__ void __launch_bounds__(256, 2) nt_split_kernel(int64_t n, int R,
                                                          const float *__restrict__ x,
                                                          const float *__restrict__ w, int slices,
                                                          float *__restrict__ out) {
  constexpr int KS = F / 16;                    // matrix steps per tile
  constexpr int kPairCols = kCT >= 2 ? 64 : 32; // columns that leave together
  constexpr int kLd = kPairCols + 4;
  __shared__ __align__(16) float tr[kWavesPerBlock][32][kLd];
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int p = lane & 31, h = lane >> 5;
  const int groups = R / (kWavesPerBlock * 32 * kCT);
  const int grp = blockIdx.x % groups, slice = blockIdx.x / groups;
  const int col0 = (grp * kWavesPerBlock + wave) * 32 * kCT;
  Split8 b[kCT][KS];
#pragma unroll
  for (int ct = 0; ct < kCT; ++ct) {
    const float *wr = w + (int64_t)(col0 + 32 * ct + p) * F + (F / 2) * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      b[ct][ks] = split8(*reinterpret_cast<const v4f *>(wr + 8 * ks),
                         *reinterpret_cast<const v4f *>(wr + 8 * ks + 4));
  }
  const int64_t tiles_total = (n + 31) >> 5;
  const int64_t per = (tiles_total + slices - 1) / slices;
  const int64_t t0 = slice * per;
  const int64_t t1 = t0 + per < tiles_total ? t0 + per : tiles_total;
  // the next tile of x is fetched ahead while it fits the registers beside the weights
  constexpr bool kAhead = F <= 64;
  v4f a[2 * KS], an[kAhead ? 2 * KS : 1];
  auto load_a = [&](int64_t t, v4f *dst) {
    int64_t pt = 32 * t + p;
    pt = pt < n ? pt : n - 1;            // rows past the end repeat the last one; never stored
    const v4f *src = reinterpret_cast<const v4f *>(x + pt * F + (F / 2) * h);
#pragma unroll
    for (int j = 0; j < 2 * KS; ++j) dst[j] = t < t1 ? src[j] : v4f{0.0f, 0.0f, 0.0f, 0.0f};
  };
  if (kAhead && t0 < t1) load_a(t0, a);
  for (int64_t t = t0; t < t1; ++t) {
    if constexpr (kAhead) load_a(t + 1, an);
    else load_a(t, a);
    v16f acc[kCT];
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[ct][i] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const Split8 as = split8(a[2 * ks], a[2 * ks + 1]);
#pragma unroll
      for (int ct = 0; ct < kCT; ++ct) acc[ct] = mma_split(as, b[ct][ks], acc[ct]);
    }
    // acc[ct][i]: point 32 t + (i / 4) * 8 + 4 h + i % 4, column col0 + 32 ct + p
    constexpr int kPieces = kPairCols / 4;            // 16-byte pieces per row
    constexpr int kRowsPer = kWave / kPieces;         // rows per store instruction
    const int piece = lane % kPieces, rr = lane / kPieces;
#pragma unroll
    for (int c0 = 0; c0 < kCT; c0 += kPairCols / 32) {
#pragma unroll
      for (int cc = 0; cc < kPairCols / 32; ++cc)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          tr[wave][(i / 4) * 8 + 4 * h + (i % 4)][32 * cc + p] = acc[c0 + cc][i];
      wave_lds_sync();
      v4f rows[32 / kRowsPer];
#pragma unroll
      for (int j = 0; j < 32 / kRowsPer; ++j)
        rows[j] = *reinterpret_cast<const v4f *>(&tr[wave][kRowsPer * j + rr][4 * piece]);
#pragma unroll
      for (int j = 0; j < 32 / kRowsPer; ++j) {
        const int64_t row = 32 * t + kRowsPer * j + rr;
        if (row < n)      // streamed: the product is read once, by a later kernel
          __builtin_nontemporal_store(
              rows[j], reinterpret_cast<v4f *>(out + row * R + col0 + 32 * c0 + 4 * piece));
      }
      wave_lds_sync();
    }
    if constexpr (kAhead) {
#pragma unroll
      for (int j = 0; j < 2 * KS; ++j) a[j] = an[j];
    }
  }
}

// The same product with the split of x shared by the four wavefronts of a block.  Above, a
// wavefront splits its tile of x for its own 32 kCT output columns; with F = 128 (registers
// for 32 columns only) that split costs more vector instructions than the six matrix
// instructions save (4.5 ms against 4.2 ms of the float32 kernel on [825 274, 128] x
// [2048, 128]^T; this kernel 2.5 ms), and with F = 64 the shared split is still the faster
// one (0.65 against 0.79 ms on [763 063, 64] x [1024, 64]^T).  Here the block owns 128 kCT columns and splits a tile
// of 32 points once: a thread fetches its runs of 8 values two tiles ahead, splits them while
// the current tile is multiplied, and parks the three parts as 16-byte vectors in operand
// order ([part][matrix step][lane half][point], one slot of padding per 32 points, so that
// the lanes of a store phase -- the runs of one point -- fall into different bank groups);
// every A operand is one 16-byte LDS read.  The 32 x 128 kCT tile of the output leaves
// through a block-wide LDS transposition as runs of 512 kCT bytes.
template <int F, int kCT>
__global__ void __launch_bounds__(256, 2) nt_split_shared_kernel(int64_t n, int R,
                                                                 const float *__restrict__ x,
                                                                 const float *__restrict__ w,
                                                                 int slices,
                                                                 float *__restrict__ out) {
  constexpr int KS = F / 16;                    // matrix steps per tile
  constexpr int kRuns = F / 8;                  // runs of 8 reduction values per point
  constexpr int kItems = 32 * kRuns / 256;      // (point, run) items per thread
  constexpr int kCols = 128 * kCT;              // output columns of the block
  constexpr int kLdA = 32 + 1;
  constexpr int kLdO = kCols + 8;               // lane halves (4 rows apart) 32 banks apart
  constexpr int kPieces = kCols / 4;            // 16-byte pieces per output row
  constexpr int kRowsPer = kWave / kPieces;     // rows per store instruction
  static_assert(kItems >= 1 && kRowsPer >= 1, "tile shape");
  __shared__ v8bf a_lds[2][3 * kRuns * kLdA];
  __shared__ __align__(16) float o_lds[32][kLdO];
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int p = lane & 31, h = lane >> 5;
  const int groups = R / kCols;
  // the hardware deals consecutive blocks to the eight XCDs in turn: the column groups of a
  // slice share its rows of x, so they are numbered onto one XCD (one L2)
  const int in_xcd = blockIdx.x / 8;
  const int grp = in_xcd % groups, slice = (in_xcd / groups) * 8 + blockIdx.x % 8;
  if (slice >= slices) return;
  const int wcol = wave * 32 * kCT;             // first column of this wavefront in the block
  Split8 b[kCT][KS];
#pragma unroll
  for (int ct = 0; ct < kCT; ++ct) {
    const float *wr = w + (int64_t)(grp * kCols + wcol + 32 * ct + p) * F + (F / 2) * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      b[ct][ks] = split8(*reinterpret_cast<const v4f *>(wr + 8 * ks),
                         *reinterpret_cast<const v4f *>(wr + 8 * ks + 4));
  }
  const int64_t tiles_total = (n + 31) >> 5;
  const int64_t per = (tiles_total + slices - 1) / slices;
  const int64_t t0 = slice * per;
  const int64_t t1 = t0 + per < tiles_total ? t0 + per : tiles_total;
  v4f xa[kItems][2], xb[kItems][2];
  auto fetch = [&](int64_t t, v4f (*dst)[2]) {
#pragma unroll
    for (int i = 0; i < kItems; ++i) {
      const int idx = threadIdx.x + 256 * i, pt_in = idx / kRuns, g = idx % kRuns;
      int64_t pt = 32 * t + pt_in;
      pt = pt < n ? pt : n - 1;          // rows past the end repeat the last one; never stored
      const v4f *src = reinterpret_cast<const v4f *>(x + pt * F + 8 * g);
      dst[i][0] = src[0];                // kept in L2: every column group reads the tile
      dst[i][1] = src[1];
    }
  };
  auto park = [&](int buf, v4f (*src)[2]) {
#pragma unroll
    for (int i = 0; i < kItems; ++i) {
      const int idx = threadIdx.x + 256 * i, pt_in = idx / kRuns, g = idx % kRuns;
      const Split8 sp = split8(src[i][0], src[i][1]);
      // run g holds f = 8 g ..: matrix step g % KS of lane half g / KS
#pragma unroll
      for (int q = 0; q < 3; ++q)
        a_lds[buf][((q * KS + g % KS) * 2 + g / KS) * kLdA + pt_in] = sp.p[q];
    }
  };
  // One tile: `parked` holds the tile after this one (fetched a whole step ago), `fetched`
  // receives the tile after that.
  auto step = [&](int64_t t, int cur, v4f (*parked)[2], v4f (*fetched)[2]) {
    if (t + 2 < t1) fetch(t + 2, fetched);
    v16f acc[kCT];
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[ct][i] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Split8 a;
#pragma unroll
      for (int q = 0; q < 3; ++q) a.p[q] = a_lds[cur][((q * KS + ks) * 2 + h) * kLdA + p];
#pragma unroll
      for (int ct = 0; ct < kCT; ++ct) acc[ct] = mma_split(a, b[ct][ks], acc[ct]);
    }
    // acc[ct][i]: point 32 t + (i / 4) * 8 + 4 h + i % 4, column wcol + 32 ct + p of the block
#pragma unroll
    for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        o_lds[(i / 4) * 8 + 4 * h + (i % 4)][wcol + 32 * ct + p] = acc[ct][i];
    if (t + 1 < t1) park(cur ^ 1, parked);
    block_lds_sync();             // the output tile and the next tile of x are complete
    // wavefront w sends rows 8 w .. 8 w + 7 of the tile
    const int piece = lane % kPieces, rr = lane / kPieces;
    v4f rows[8 / kRowsPer];
#pragma unroll
    for (int j = 0; j < 8 / kRowsPer; ++j)
      rows[j] = *reinterpret_cast<const v4f *>(&o_lds[8 * wave + kRowsPer * j + rr][4 * piece]);
#pragma unroll
    for (int j = 0; j < 8 / kRowsPer; ++j) {
      const int64_t row = 32 * t + 8 * wave + kRowsPer * j + rr;
      if (row < n)        // streamed: the product is read once, by a later kernel
        __builtin_nontemporal_store(
            rows[j], reinterpret_cast<v4f *>(out + row * R + grp * kCols + 4 * piece));
    }
    block_lds_sync();             // the output tile has been read
  };
  if (t0 < t1) {
    fetch(t0, xa);
    park(0, xa);
    if (t0 + 1 < t1) fetch(t0 + 1, xa);
  }
  block_lds_sync();
  for (int64_t t = t0; t < t1; t += 2) {
    step(t, 0, xa, xb);
    if (t + 1 < t1) step(t + 1, 1, xb, xa);
  }
}

// F = 32: every wavefront splits its own tile (128 columns); F = 64 and 128: shared split.
static int nt_split_cols(int F) { return F == 128 ? 128 : F == 64 ? 256 : F == 32 ? 512 : 0; }

bool nt_split_supported(int F, int R) {
  const int cols = nt_split_cols(F);
  return cols > 0 && R >= cols && R % cols == 0;
}

int launch_nt_split(hipStream_t s, int64_t n, int F, const float *x, int R, const float *w,
                    float *out) {
  const int groups = R / nt_split_cols(F);
  int device = 0, cus = 0;
  MCCNN_HIP_CHECK(hipGetDevice(&device));
  MCCNN_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  // one resident round of blocks (two blocks of four wavefronts per compute unit)
  int slices = 2 * cus / groups;
  if (slices < 1) slices = 1;
  const int64_t tiles = (n + 31) / 32;
  if (slices > tiles) slices = (int)tiles;
  // (the kernels with a shared split number their blocks per XCD: slices rounded up to eight)
  const dim3 grid(groups * (F >= 64 ? (slices + 7) / 8 * 8 : slices)), block(256);
  switch (F) {
    case 128: hipLaunchKernelGGL((nt_split_shared_kernel<128, 1>), grid, block, 0, s, n, R, x, w, slices, out); break;
    case 64: hipLaunchKernelGGL((nt_split_shared_kernel<64, 2>), grid, block, 0, s, n, R, x, w, slices, out); break;
    default: hipLaunchKernelGGL((nt_split_kernel<32, 4>), grid, block, 0, s, n, R, x, w, slices, out); break;
  }
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

// out[out_rows[n] or n, :] = x[n, :] * w for x [N, R] and the weights given transposed,
// wt [F, R]: the tiled product on the bf16 pipe.  A block of four wavefronts owns a BM x BN
// tile of the output (128 x 128, 256 x 128 or 256 x 64), every wavefront 64 x 64 or 128 x 64
// of it as accumulator tiles of 32 x 32, and walks the reduction in chunks of 32.  The chunk of x and
// of wt for the next step is fetched into registers while the current one is multiplied;
// the thread that fetched eight consecutive values splits them once and parks the three
// bfloat16 parts as 16-byte vectors in operand order ([part][group of 8 along the
// reduction][row]; groups 4 vectors further apart than the tile is high, so that the 16 lanes
// of a store phase -- 4 rows x 4 groups -- land in 16 different bank groups), and every
// matrix operand is one 16-byte LDS read.  x is read once per column block; wt comes from L2.
constexpr int kSplitK = 32, kSplitGroups = kSplitK / 8, kSplitThreads = 256;

template <int BN, int BM = 16384 / BN>
__global__ void __launch_bounds__(kSplitThreads) tile_split_kernel(
    int64_t n, int R, int F, const float *__restrict__ x, const float *__restrict__ wt,
    const int *__restrict__ out_rows, float *__restrict__ out) {
  constexpr int kWN = BN / 64, kWM = 4 / kWN;      // wavefronts across / down the tile
  constexpr int kRT = BM / kWM / 32;               // 32-row accumulator tiles per wavefront
  constexpr int kLdA = BM + 4, kLdB = BN + 4;                   // vectors per group
  constexpr int kAItems = BM * kSplitGroups / kSplitThreads;    // (row, group) items per thread
  constexpr int kBItems = BN * kSplitGroups / kSplitThreads;
  __shared__ v8bf a_lds[3 * kSplitGroups * kLdA];
  __shared__ v8bf b_lds[3 * kSplitGroups * kLdB];
  const int t = threadIdx.x, lane = lane_id(), wave = t / kWave;
  const int p = lane & 31, h = lane >> 5;
  const int wm = wave / kWN, wn = wave % kWN;
  const int col_blocks = F / BN;
  const int64_t row0 = (int64_t)(blockIdx.x / col_blocks) * BM;
  const int col0 = (blockIdx.x % col_blocks) * BN;

  v16f acc[kRT][2];
#pragma unroll
  for (int i = 0; i < kRT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  v4f xa[kAItems][2], wb[kBItems][2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < kAItems; ++i) {
      const int idx = t + kSplitThreads * i, row = idx >> 2, g = idx & 3;
      // rows past the end repeat the last row (their results are never stored): no branch
      const int64_t r = row0 + row < n ? row0 + row : n - 1;
      const v4f *src = reinterpret_cast<const v4f *>(x + r * R + k0 + 8 * g);
      xa[i][0] = __builtin_nontemporal_load(src);
      xa[i][1] = __builtin_nontemporal_load(src + 1);
    }
#pragma unroll
    for (int i = 0; i < kBItems; ++i) {
      const int idx = t + kSplitThreads * i, col = idx >> 2, g = idx & 3;
      const v4f *src = reinterpret_cast<const v4f *>(wt + (int64_t)(col0 + col) * R + k0 + 8 * g);
      wb[i][0] = src[0];
      wb[i][1] = src[1];
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int i = 0; i < kAItems; ++i) {
      const int idx = t + kSplitThreads * i, row = idx >> 2, g = idx & 3;
      const Split8 s = split8(xa[i][0], xa[i][1]);
#pragma unroll
      for (int q = 0; q < 3; ++q) a_lds[(q * kSplitGroups + g) * kLdA + row] = s.p[q];
    }
#pragma unroll
    for (int i = 0; i < kBItems; ++i) {
      const int idx = t + kSplitThreads * i, col = idx >> 2, g = idx & 3;
      const Split8 s = split8(wb[i][0], wb[i][1]);
#pragma unroll
      for (int q = 0; q < 3; ++q) b_lds[(q * kSplitGroups + g) * kLdB + col] = s.p[q];
    }
  };

  fetch(0);
  for (int k0 = 0; k0 < R; k0 += kSplitK) {
    __syncthreads();                  // the previous chunk has been multiplied
    park();
    __syncthreads();
    if (k0 + kSplitK < R) fetch(k0 + kSplitK);
#pragma unroll
    for (int ks = 0; ks < kSplitK / 16; ++ks) {
      Split8 a[kRT], b[2];
#pragma unroll
      for (int q = 0; q < 3; ++q) {
#pragma unroll
        for (int i = 0; i < kRT; ++i)
          a[i].p[q] = a_lds[(q * kSplitGroups + 2 * ks + h) * kLdA + wm * (32 * kRT) + 32 * i + p];
#pragma unroll
        for (int j = 0; j < 2; ++j)
          b[j].p[q] = b_lds[(q * kSplitGroups + 2 * ks + h) * kLdB + wn * 64 + 32 * j + p];
      }
#pragma unroll
      for (int i = 0; i < kRT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mma_split(a[i], b[j], acc[i][j]);
    }
  }
  // acc[i][j][e]: row row0 + 32 kRT wm + 32 i + (e / 4) * 8 + 4 h + e % 4, column col0 + 64 wn + 32 j + p
#pragma unroll
  for (int i = 0; i < kRT; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int64_t row = row0 + wm * (32 * kRT) + 32 * i + (e / 4) * 8 + 4 * h + (e % 4);
      if (row < n) {
        const int64_t orow = out_rows ? out_rows[row] : row;
        float *o = out + orow * F + col0 + wn * 64 + p;
#pragma unroll
        for (int j = 0; j < 2; ++j) o[32 * j] = acc[i][j][e];
      }
    }
}

int launch_tile_split(hipStream_t s, int64_t n, int R, const float *x, int F, const float *wt,
                      const int *out_rows, float *out) {
  const int bn = F % 128 == 0 ? 128 : 64;
  // 128 columns: tiles of 256 rows (every wavefront 128 x 64) while they still fill the device
  // twice over -- the weights' chunk is split once per 256 instead of once per 128 rows
  // (825 k x 2048 by 2048 x 128: 2.31 against 2.40 ms) --, tiles of 128 rows below that
  int device = 0, cus = 0;
  MCCNN_HIP_CHECK(hipGetDevice(&device));
  MCCNN_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  const bool tall = bn == 128 && (n + 255) / 256 * (F / 128) >= 2 * (int64_t)cus;
  const int bm = tall ? 256 : 16384 / bn;
  const dim3 block(kSplitThreads), grid((unsigned)((n + bm - 1) / bm * (F / bn)));
  if (tall)
    hipLaunchKernelGGL((tile_split_kernel<128, 256>), grid, block, 0, s, n, R, F, x, wt, out_rows, out);
  else if (bn == 128)
    hipLaunchKernelGGL((tile_split_kernel<128>), grid, block, 0, s, n, R, F, x, wt, out_rows, out);
  else
    hipLaunchKernelGGL((tile_split_kernel<64>), grid, block, 0, s, n, R, F, x, wt, out_rows, out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

// Gradient of the final weights (MCConv.py:187, KPConv.py:226-230): out[c, r] = sum_n
// x[n, c] * y[n, r] on the bf16 pipe, reduction over all N points.  As in the float32
// kernels of dense.hip the points are cut into slices; a block owns (slice, 128 columns of
// y) and all C rows of the output, and the per-slice partial sums are added afterwards in a
// fixed order.  The reduction index runs along the rows of both operands, so a thread
// fetches a patch of 8 points x 4 columns (eight 16-byte loads from eight rows), turns it
// into four vectors of 8 points, splits them and parks them as [part][group of 8
// points][column]; every matrix operand is then one 16-byte LDS read.  Per step of 32
// points: C x 32 values of x and 128 x 32 of y.
// Blocks are numbered so that the column groups of one slice run on the same XCD (the
// hardware deals consecutive blocks to the eight XCDs in turn): the slice of x they all read
// then comes from HBM once and from that XCD's L2 for the other groups.
template <int C, int BN>
__global__ void __launch_bounds__(kSplitThreads) tn_split_kernel(
    int64_t n, int R, const float *__restrict__ x, const float *__restrict__ y, int slices,
    float *__restrict__ partials) {
  constexpr int kCT = C / 32;                                   // row tiles of the output
  constexpr int kWM = kCT >= 2 ? 2 : 1, kWN = 4 / kWM;          // wavefronts down / across
  constexpr int kTM = kCT / kWM, kTN = BN / 32 / kWN;           // 32 x 32 tiles per wavefront
  constexpr int kLdA = C + 4, kLdB = BN + 4;
  constexpr int kAPatches = C * kSplitK / 32;                   // patches of 8 points x 4 columns
  constexpr int kBPatches = BN * kSplitK / 32;
  constexpr int kAPer = (kAPatches + kSplitThreads - 1) / kSplitThreads;
  constexpr int kBPer = (kBPatches + kSplitThreads - 1) / kSplitThreads;
  // the patches of y go to the first threads, those of x to the last ones
  constexpr int kAShift = kAPer * kSplitThreads - kAPatches;
  __shared__ v8bf a_lds[3 * kSplitGroups * kLdA];
  __shared__ v8bf b_lds[3 * kSplitGroups * kLdB];
  const int t = threadIdx.x, lane = lane_id(), wave = t / kWave;
  const int p = lane & 31, h = lane >> 5;
  const int wm = wave / kWN, wn = wave % kWN;
  const int groups = R / BN;
  const int in_xcd = blockIdx.x / 8;
  const int grp = in_xcd % groups, slice = (in_xcd / groups) * 8 + blockIdx.x % 8;
  if (slice >= slices) return;
  const int col0 = grp * BN;
  const int64_t steps_total = (n + kSplitK - 1) / kSplitK;
  const int64_t per = (steps_total + slices - 1) / slices;
  const int64_t s0 = slice * per;
  const int64_t s1 = s0 + per < steps_total ? s0 + per : steps_total;

  v16f acc[kTM][kTN];
#pragma unroll
  for (int i = 0; i < kTM; ++i)
#pragma unroll
    for (int j = 0; j < kTN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // patch idx of an operand with W columns: group g = idx / (W / 4), columns 4 c4 .. 4 c4 + 3
  v4f xa[kAPer][8], yb[kBPer][8];
  auto fetch = [&](int64_t step) {
    const int64_t p0 = step * kSplitK;
#pragma unroll
    for (int i = 0; i < kAPer; ++i) {
      const int idx = t + kSplitThreads * i - kAShift, g = idx / (C / 4), c4 = idx % (C / 4);
      if (kAShift == 0 || idx >= 0) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const int64_t pt = p0 + 8 * g + r;        // points past the end count as zeros
          const v4f v = *reinterpret_cast<const v4f *>(x + (pt < n ? pt : n - 1) * C + 4 * c4);
          xa[i][r] = pt < n ? v : v4f{0.0f, 0.0f, 0.0f, 0.0f};
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kBPer; ++i) {
      const int idx = t + kSplitThreads * i, g = idx / (BN / 4), c4 = idx % (BN / 4);
      if (kBPatches % kSplitThreads == 0 || idx < kBPatches) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const int64_t pt = p0 + 8 * g + r;
          const v4f v = __builtin_nontemporal_load(
              reinterpret_cast<const v4f *>(y + (pt < n ? pt : n - 1) * R + col0 + 4 * c4));
          yb[i][r] = pt < n ? v : v4f{0.0f, 0.0f, 0.0f, 0.0f};
        }
      }
    }
  };
  auto park_patch = [&](const v4f *patch, v8bf *lds, int ld, int g, int c4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const v4f lo = {patch[0][j], patch[1][j], patch[2][j], patch[3][j]};
      const v4f hi = {patch[4][j], patch[5][j], patch[6][j], patch[7][j]};
      const Split8 s = split8(lo, hi);
#pragma unroll
      for (int q = 0; q < 3; ++q) lds[(q * kSplitGroups + g) * ld + 4 * c4 + j] = s.p[q];
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int i = 0; i < kAPer; ++i) {
      const int idx = t + kSplitThreads * i - kAShift;
      if (kAShift == 0 || idx >= 0) park_patch(xa[i], a_lds, kLdA, idx / (C / 4), idx % (C / 4));
    }
#pragma unroll
    for (int i = 0; i < kBPer; ++i) {
      const int idx = t + kSplitThreads * i;
      if (kBPatches % kSplitThreads == 0 || idx < kBPatches)
        park_patch(yb[i], b_lds, kLdB, idx / (BN / 4), idx % (BN / 4));
    }
  };

  if (s0 < s1) fetch(s0);
  for (int64_t step = s0; step < s1; ++step) {
    __syncthreads();                  // the previous step has been multiplied
    park();
    __syncthreads();
    if (step + 1 < s1) fetch(step + 1);
#pragma unroll
    for (int ks = 0; ks < kSplitK / 16; ++ks) {
      Split8 a[kTM], b[kTN];
#pragma unroll
      for (int q = 0; q < 3; ++q) {
#pragma unroll
        for (int i = 0; i < kTM; ++i)
          a[i].p[q] = a_lds[(q * kSplitGroups + 2 * ks + h) * kLdA + (wm * kTM + i) * 32 + p];
#pragma unroll
        for (int j = 0; j < kTN; ++j)
          b[j].p[q] = b_lds[(q * kSplitGroups + 2 * ks + h) * kLdB + (wn * kTN + j) * 32 + p];
      }
#pragma unroll
      for (int i = 0; i < kTM; ++i)
#pragma unroll
        for (int j = 0; j < kTN; ++j) acc[i][j] = mma_split(a[i], b[j], acc[i][j]);
    }
  }
  // acc[i][j][e]: channel 32 (wm kTM + i) + (e / 4) * 8 + 4 h + e % 4, column col0 + 32 (wn kTN + j) + p
  float *o = partials + (int64_t)slice * C * R + col0 + p;
#pragma unroll
  for (int i = 0; i < kTM; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int c = 32 * (wm * kTM + i) + (e / 4) * 8 + 4 * h + (e % 4);
#pragma unroll
      for (int j = 0; j < kTN; ++j) o[(int64_t)c * R + 32 * (wn * kTN + j)] = acc[i][j][e];
    }
}

// Columns of y per block: 128 with all 128 rows of the output, 256 below that.
static int tn_split_cols(int C) { return C == 128 ? 128 : 256; }

bool tn_split_supported(int C, int R) {
  if (!(C == 32 || C == 64 || C == 128)) return false;
  const int bn = tn_split_cols(C);
  return R >= bn && R % bn == 0 && R <= 4096;
}

// Slices of the point range for an output of C x R (also sizes the partial sums): a
// multiple of 8, one eighth per XCD, about 1024 blocks in all.
int tn_split_slices(int C, int R) {
  const int groups = R / tn_split_cols(C);
  int s = 1024 / groups / 8 * 8;
  return s < 8 ? 8 : s;
}

int launch_tn_split(hipStream_t s, int64_t n, int C, const float *x, int R, const float *y,
                    int slices, float *partials) {
  const int groups = R / tn_split_cols(C);
  const dim3 grid((unsigned)(groups * ((slices + 7) / 8) * 8)), block(kSplitThreads);
  switch (C) {
    case 128: hipLaunchKernelGGL((tn_split_kernel<128, 128>), grid, block, 0, s, n, R, x, y, slices, partials); break;
    case 64: hipLaunchKernelGGL((tn_split_kernel<64, 256>), grid, block, 0, s, n, R, x, y, slices, partials); break;
    default: hipLaunchKernelGGL((tn_split_kernel<32, 256>), grid, block, 0, s, n, R, x, y, slices, partials); break;
  }
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_set_split_products(int enabled) {
  const int before = split_products_enabled() ? 1 : 0;
  g_split_products.store(enabled ? 1 : 0, std::memory_order_relaxed);
  return before;
}

extern "C" int mccnn_split_products_enabled(void) { return split_products_enabled() ? 1 : 0; }
