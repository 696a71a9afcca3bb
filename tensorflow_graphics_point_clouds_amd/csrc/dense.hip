// Gradient of the final weights of a convolution layer (pylib/pc/layers/MCConv.py:187,
// KPConv.py:226-230): out[c, r] = sum_n x[n, c] * y[n, r] with a reduction over all
// N points and a small output (C <= 128 rows, R = C_out * K columns).  A library
// GEMM re-reads the long operand for every tile of the small output; here y
// streams from HBM exactly once: the points are cut into slices, a block owns
// (slice, 256 columns), each wavefront 64 of them with all C rows as 16x16
// matrix-core accumulators, and the per-slice partial sums are added up
// afterwards in a fixed order.
#include "common.h"
#include "fill.h"
#include "mfma.h"
#include "split.h"

namespace mccnn {

static int tn_slices(int R) {
  const int groups = R / 256;
  int s = 1024 / groups;
  return s < 1 ? 1 : s;
}

template <int kRT>
__global__ void __launch_bounds__(256) tn_product_kernel(int64_t n, int R,
                                                         const float *__restrict__ x,
                                                         const float *__restrict__ y,
                                                         int slices, float *__restrict__ partials) {
  constexpr int C = 16 * kRT;
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int quarter = lane >> 4, c16 = lane & 15;
  const int groups = R >> 8;
  const int grp = blockIdx.x % groups, slice = blockIdx.x / groups;
  const int col0 = grp * 256 + wave * 64;
  const int64_t steps_total = (n + 3) >> 2;                 // 4 points per matrix step
  const int64_t per = (steps_total + slices - 1) / slices;
  const int64_t s0 = slice * per;
  const int64_t s1 = s0 + per < steps_total ? s0 + per : steps_total;
  v4f acc[kRT][4];
#pragma unroll
  for (int i = 0; i < kRT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
  // lane (quarter, c16): point 4 s + quarter, channels kRT*c16 + i, columns col0 + 4*c16 + j
  const float *xl = x + kRT * c16;
  const float *yl = y + col0 + 4 * c16;
  auto load_a = [&](int64_t s) {
    const int64_t pt = 4 * s + quarter;
    return load_vec<kRT>(xl + pt * C, s < s1 && pt < n);
  };
  auto load_b = [&](int64_t s) {
    const int64_t pt = 4 * s + quarter;
    return load_vec<4>(yl + pt * R, s < s1 && pt < n);
  };
  FVec<kRT> a0 = load_a(s0), a1 = load_a(s0 + 1);
  FVec<4> b0 = load_b(s0), b1 = load_b(s0 + 1);
  for (int64_t s = s0; s < s1; s += 2) {
    const FVec<kRT> a2 = load_a(s + 2), a3 = load_a(s + 3);
    const FVec<4> b2 = load_b(s + 2), b3 = load_b(s + 3);
#pragma unroll
    for (int i = 0; i < kRT; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0.v[i], b0.v[j], acc[i][j], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < kRT; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1.v[i], b1.v[j], acc[i][j], 0, 0, 0);
    a0 = a2; a1 = a3; b0 = b2; b1 = b3;
  }
  // accumulator (i, j), register r: channel kRT*(4*quarter + r) + i, column col0 + 4*c16 + j
  float *o = partials + (int64_t)slice * C * R + col0 + 4 * c16;
#pragma unroll
  for (int i = 0; i < kRT; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const v4f v = {acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]};
      *reinterpret_cast<v4f *>(o + (int64_t)(kRT * (4 * quarter + r) + i) * R) = v;
    }
}

// The same product with both operands staged through LDS: per step the block fetches 32
// points of x (all C channels) and of its 256 columns of y with coalesced 16-byte loads (the
// next step's while the current one is multiplied), parks them as they are (rows of 32
// points, C + 16 and 272 floats apart, so that the four points of a matrix step sit in four
// different bank groups) and every lane picks its operands with 4-byte LDS reads: lane
// (quarter, c16) of step s reads point 4 s + quarter, channel 16 i + c16 / column 16 j + c16.
constexpr int kTnPts = 32;

template <int kRT>
__global__ void __launch_bounds__(256) tn_tile_kernel(int64_t n, int R,
                                                      const float *__restrict__ x,
                                                      const float *__restrict__ y, int slices,
                                                      float *__restrict__ partials) {
  constexpr int C = 16 * kRT, kLdA = C + 16, kLdB = 256 + 16;
  constexpr int kAVecs = kTnPts * C / 4;                    // 16-byte pieces of the x tile
  constexpr int kALoads = (kAVecs + 255) / 256, kBLoads = kTnPts * 256 / 4 / 256;
  __shared__ __align__(16) float a_lds[kTnPts * kLdA];
  __shared__ __align__(16) float b_lds[kTnPts * kLdB];
  const int t = threadIdx.x, lane = lane_id(), wave = t / kWave;
  const int q = lane >> 4, c16 = lane & 15;
  const int groups = R >> 8;
  const int grp = blockIdx.x % groups, slice = blockIdx.x / groups;
  const int col0 = grp * 256;
  const int64_t steps_total = (n + kTnPts - 1) / kTnPts;
  const int64_t per = (steps_total + slices - 1) / slices;
  const int64_t s0 = slice * per;
  const int64_t s1 = s0 + per < steps_total ? s0 + per : steps_total;
  v4f acc[kRT][4];
#pragma unroll
  for (int i = 0; i < kRT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

  v4f xa[kALoads], yb[kBLoads];
  auto fetch = [&](int64_t step) {
    const int64_t p0 = step * kTnPts;
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      const int idx = (t + 256 * i) % kAVecs, pt = idx / (C / 4), c4 = idx % (C / 4);
      const bool live = p0 + pt < n;           // points past the end count as zeros
      const v4f v = *reinterpret_cast<const v4f *>(x + (live ? p0 + pt : n - 1) * C + 4 * c4);
      xa[i] = live ? v : v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      const int idx = t + 256 * i, pt = idx >> 6, c4 = idx & 63;
      const bool live = p0 + pt < n;
      const v4f v = __builtin_nontemporal_load(
          reinterpret_cast<const v4f *>(y + (live ? p0 + pt : n - 1) * R + col0 + 4 * c4));
      yb[i] = live ? v : v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      const int idx = (t + 256 * i) % kAVecs, pt = idx / (C / 4), c4 = idx % (C / 4);
      *reinterpret_cast<v4f *>(a_lds + pt * kLdA + 4 * c4) = xa[i];   // (C = 16: written twice)
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      const int idx = t + 256 * i, pt = idx >> 6, c4 = idx & 63;
      *reinterpret_cast<v4f *>(b_lds + pt * kLdB + 4 * c4) = yb[i];
    }
  };
  const float *a_rd = a_lds + q * kLdA + c16;
  const float *b_rd = b_lds + q * kLdB + wave * 64 + c16;
  if (s0 < s1) fetch(s0);
  for (int64_t step = s0; step < s1; ++step) {
    __syncthreads();                  // the previous step has been multiplied
    park();
    __syncthreads();
    if (step + 1 < s1) fetch(step + 1);
#pragma unroll
    for (int s = 0; s < kTnPts / 4; ++s) {
      float a[kRT], b[4];
#pragma unroll
      for (int i = 0; i < kRT; ++i) a[i] = a_rd[4 * s * kLdA + 16 * i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = b_rd[4 * s * kLdB + 16 * j];
#pragma unroll
      for (int i = 0; i < kRT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  }
  // acc[i][j][r]: channel 16 i + 4 q + r, column col0 + 64 wave + 16 j + c16
  float *o = partials + (int64_t)slice * C * R + col0 + wave * 64 + c16;
#pragma unroll
  for (int i = 0; i < kRT; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int j = 0; j < 4; ++j) o[(int64_t)(16 * i + 4 * q + r) * R + 16 * j] = acc[i][j][r];
}

__global__ void __launch_bounds__(256) tn_reduce_kernel(int64_t elems, int slices,
                                                        const float *__restrict__ partials,
                                                        float *__restrict__ out) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= elems) return;
  // eight slices in flight per trip; the additions keep the order of the slices
  float s = 0.0f;
  int k = 0;
  for (; k + 8 <= slices; k += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = partials[(int64_t)(k + u) * elems + e];
#pragma unroll
    for (int u = 0; u < 8; ++u) s += v[u];
  }
  for (; k < slices; ++k) s += partials[(int64_t)k * elems + e];
  out[e] = s;
}

// out[n, r] = sum_f x[n, f] * w[r, f]: the gradient of the projection that enters
// a layer's final product (x = output gradient [N, F], w = dense final weights
// [R, F], R = C * K).  Write-bound: 4 R bytes per point leave, 4 F arrive.  A
// wavefront keeps its (16 kCols) x F slice of w in registers for its whole life (64
// registers: kCols = 4 columns per lane up to F = 64, 2 for F = 128, 1 for F = 256) and
// streams tiles of 16 points through the matrix cores; a lane owns kCols consecutive
// output columns so that every row of a tile leaves as 64 kCols contiguous bytes.
template <int kCols> struct ColVec;
template <> struct ColVec<4> { using type = v4f; };
template <> struct ColVec<2> { using type = v2f; };
template <> struct ColVec<1> { using type = float; };

template <int F, int kCols>
__global__ void __launch_bounds__(256) nt_product_kernel(int64_t n, int R,
                                                         const float *__restrict__ x,
                                                         const float *__restrict__ w,
                                                         int slices, float *__restrict__ out) {
  using Row = typename ColVec<kCols>::type;
  constexpr int kSteps = F / 4;            // reduction steps; lane (kk, row) owns f = kk*kSteps + s
  constexpr int kWaveCols = 16 * kCols;    // output columns of a wavefront
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int kk = lane >> 4, c16 = lane & 15;
  const int groups = R / (4 * kWaveCols);
  const int grp = blockIdx.x % groups, slice = blockIdx.x / groups;
  const int col0 = (grp * 4 + wave) * kWaveCols;
  // B operand of step s, column tile j: w[col0 + kCols*c16 + j][kk*kSteps + s]
  float b[kCols][kSteps];
#pragma unroll
  for (int j = 0; j < kCols; ++j) {
    const FVec<kSteps> t = load_vec<kSteps>(
        w + (int64_t)(col0 + kCols * c16 + j) * F + kk * kSteps, true);
#pragma unroll
    for (int s = 0; s < kSteps; ++s) b[j][s] = t.v[s];
  }
  const int64_t tiles_total = (n + 15) >> 4;
  const int64_t per = (tiles_total + slices - 1) / slices;
  const int64_t t0 = slice * per;
  const int64_t t1 = t0 + per < tiles_total ? t0 + per : tiles_total;
  auto load_a = [&](int64_t t) {
    const int64_t pt = 16 * t + c16;
    return load_vec<kSteps>(x + pt * F + kk * kSteps, t < t1 && pt < n);
  };
  FVec<kSteps> a = load_a(t0);
  for (int64_t t = t0; t < t1; ++t) {
    const FVec<kSteps> an = load_a(t + 1);
    v4f acc[kCols];
#pragma unroll
    for (int j = 0; j < kCols; ++j) acc[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int s = 0; s < kSteps; ++s)
#pragma unroll
      for (int j = 0; j < kCols; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[s], b[j][s], acc[j], 0, 0, 0);
    // acc[j][r]: point 16 t + 4*kk + r, column col0 + kCols*c16 + j.  The four rows leave from
    // four register tuples of their own: a store fetches its data only when the memory
    // pipeline gets to it, and whatever overwrites a register with a store pending on it
    // (the next row's copy, the next tile's matrix instructions) waits for that fetch.
    Row rows[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if constexpr (kCols == 4) rows[r] = v4f{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
      else if constexpr (kCols == 2) rows[r] = v2f{acc[0][r], acc[1][r]};
      else rows[r] = acc[0][r];
      asm volatile("" : "+v"(rows[r]));
    }
    float *o = out + (16 * t + 4 * kk) * R + col0 + kCols * c16;
#pragma unroll
    for (int r = 0; r < 4; ++r)     // streamed: the product is read once, by a later kernel
      if (16 * t + 16 <= n || 16 * t + 4 * kk + r < n)
        __builtin_nontemporal_store(rows[r], reinterpret_cast<Row *>(o + (int64_t)r * R));
    a = an;
  }
}

static int nt_cols(int F) { return F <= 64 ? 4 : F == 128 ? 2 : 1; }

static bool nt_supported(int F, int R) {
  if (!(F == 16 || F == 32 || F == 64 || F == 128 || F == 256)) return false;
  const int block_cols = 64 * nt_cols(F);
  return R >= block_cols && R % block_cols == 0;
}

// out[out_rows[n] or n, :] = x[n, :] * w for x [N, R], w [R, F] when w is too large to sit in
// the registers of one block (R * F > 65536: the 128 -> 128 kernel-point layers, R = 2048):
// the classic tiled product.  A block of four wavefronts owns a BM x BN tile of the output,
// 128 x 128 or 256 x 64, every wavefront 64 x 64 of it as 4 x 4 accumulator tiles, and walks
// the reduction in steps of 32: the BM x 32 block of x and the 32 x BN block of w of the next
// step are fetched into registers while the current one is multiplied out of LDS (both with
// the reduction index running along a row, rows 36 floats apart), two barriers per step.
// The reduction index of a matrix step may be permuted as long as both operands agree: lane
// quarter q takes indices 4q .. 4q+3 of each group of 16, so every operand fetch is one
// 16-byte LDS read.  x is read once per column block (F / BN times); w comes from L2.
// w is taken as it is ([R, F]) or transposed (wt [F, R], kWT): transposed, its rows are
// fetched and parked exactly like those of x (129 TFLOP/s on [825 274, 2048] x [2048, 128]).
// As it is, the lanes of a wavefront fetch their pieces with the reduction index running
// fastest (32 rows of w, 16 bytes of each), so that the four transposing LDS writes of a
// lane land in 32 consecutive banks: 113 TFLOP/s; with the columns running fastest the
// fetch is coalesced but the writes hit two banks 16 ways (0.9 G conflict cycles per
// launch, 104 TFLOP/s).  A second LDS buffer (one barrier per step) costs a resident block
// per compute unit and is slower (107 TFLOP/s); fetching the operands of the next half
// group ahead of the matrix steps changes nothing, and neither does copying the blocks
// straight from global memory into (swizzled, double-buffered) LDS with
// global_load_lds_dwordx4 instead of through registers (118 against 119 TFLOP/s).
constexpr int kTileK = 32, kTileLd = kTileK + 4, kTileThreads = 256;

template <int BN, bool kWT>
__global__ void __launch_bounds__(kTileThreads) tile_product_kernel(
    int64_t n, int R, int F, const float *__restrict__ x, const float *__restrict__ w,
    const int *__restrict__ out_rows, float *__restrict__ out) {
  constexpr int BM = 16384 / BN;                  // 4 wavefronts x (64 x 64)
  constexpr int kWN = BN / 64;                    // wavefronts side by side
  constexpr int kALoads = BM * kTileK / 4 / kTileThreads;   // 16-byte loads per thread and step
  constexpr int kBLoads = BN * kTileK / 4 / kTileThreads;
  __shared__ __align__(16) float a_lds[BM * kTileLd];
  __shared__ __align__(16) float b_lds[BN * kTileLd];
  const int t = threadIdx.x, lane = lane_id(), wave = t / kWave;
  const int q = lane >> 4, c16 = lane & 15;
  const int wm = wave / kWN, wn = wave % kWN;
  const int col_blocks = F / BN;
  const int64_t row0 = (int64_t)(blockIdx.x / col_blocks) * BM;
  const int col0 = (blockIdx.x % col_blocks) * BN;

  v4f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

  // this thread's pieces of a step: (row, 4 k) of x and of w^T, or (k, 4 columns) of w
  v4f xa[kALoads], wb[kBLoads];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      const int idx = t + kTileThreads * i, row = idx >> 3, c4 = idx & 7;
      // rows past the end repeat the last row (their results are never stored): no branch
      const int64_t r = row0 + row < n ? row0 + row : n - 1;
      xa[i] = *reinterpret_cast<const v4f *>(x + r * R + k0 + 4 * c4);
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      const int idx = t + kTileThreads * i;
      if constexpr (kWT) {
        const int col = idx >> 3, c4 = idx & 7;
        wb[i] = *reinterpret_cast<const v4f *>(w + (int64_t)(col0 + col) * R + k0 + 4 * c4);
      } else {
        const int kk = idx % kTileK, c4 = idx / kTileK;
        wb[i] = *reinterpret_cast<const v4f *>(w + (int64_t)(k0 + kk) * F + col0 + 4 * c4);
      }
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      const int idx = t + kTileThreads * i, row = idx >> 3, c4 = idx & 7;
      *reinterpret_cast<v4f *>(a_lds + row * kTileLd + 4 * c4) = xa[i];
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) {
      const int idx = t + kTileThreads * i;
      if constexpr (kWT) {
        const int col = idx >> 3, c4 = idx & 7;
        *reinterpret_cast<v4f *>(b_lds + col * kTileLd + 4 * c4) = wb[i];
      } else {
        const int kk = idx % kTileK, c4 = idx / kTileK;
#pragma unroll
        for (int j = 0; j < 4; ++j) b_lds[(4 * c4 + j) * kTileLd + kk] = wb[i][j];
      }
    }
  };

  const float *a_rd = a_lds + (wm * 64 + c16) * kTileLd + 4 * q;
  const float *b_rd = b_lds + (wn * 64 + c16) * kTileLd + 4 * q;
  fetch(0);
  for (int k0 = 0; k0 < R; k0 += kTileK) {
    __syncthreads();                  // the previous step has been multiplied
    park();
    __syncthreads();
    if (k0 + kTileK < R) fetch(k0 + kTileK);
#pragma unroll
    for (int ks = 0; ks < kTileK / 16; ++ks) {
      v4f a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a[i] = *reinterpret_cast<const v4f *>(a_rd + 16 * i * kTileLd + 16 * ks);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        b[j] = *reinterpret_cast<const v4f *>(b_rd + 16 * j * kTileLd + 16 * ks);
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i][s], b[j][s], acc[i][j], 0, 0, 0);
    }
  }
  // acc[i][j][r]: row row0 + 64 wm + 16 i + 4 q + r, column col0 + 64 wn + 16 j + c16
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int64_t row = row0 + wm * 64 + 16 * i + 4 * q + r;
      if (row < n) {
        const int64_t orow = out_rows ? out_rows[row] : row;
        float *o = out + orow * F + col0 + wn * 64 + c16;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[16 * j] = acc[i][j][r];
      }
    }
}

bool tile_product_supported(int R, int F) { return R >= 32 && R % 32 == 0 && F >= 64 && F % 64 == 0; }

// Output rows per block of the tiled product for F columns.
int tile_product_rows(int F) { return F % 128 == 0 ? 128 : 256; }

int launch_tile_product(hipStream_t s, int64_t n, int R, const float *x, int F, const float *w,
                        bool w_transposed, const int *out_rows, float *out) {
  if (w_transposed && split_products_enabled())
    return launch_tile_split(s, n, R, x, F, w, out_rows, out);
  const int bn = F % 128 == 0 ? 128 : 64, bm = tile_product_rows(F);
  const dim3 block(kTileThreads), grid((unsigned)((n + bm - 1) / bm * (F / bn)));
  if (bn == 128) {
    if (w_transposed)
      hipLaunchKernelGGL((tile_product_kernel<128, true>), grid, block, 0, s, n, R, F, x, w, out_rows, out);
    else
      hipLaunchKernelGGL((tile_product_kernel<128, false>), grid, block, 0, s, n, R, F, x, w, out_rows, out);
  } else {
    if (w_transposed)
      hipLaunchKernelGGL((tile_product_kernel<64, true>), grid, block, 0, s, n, R, F, x, w, out_rows, out);
    else
      hipLaunchKernelGGL((tile_product_kernel<64, false>), grid, block, 0, s, n, R, F, x, w, out_rows, out);
  }
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

static bool tn_supported(int C, int R) {
  return (C == 16 || C == 32 || C == 64 || C == 128) && R >= 256 && R % 256 == 0 && R <= 4096;
}

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_weight_grad_product_supported(int num_rows_out, int num_cols_out) {
  return tn_supported(num_rows_out, num_cols_out) ? 1 : 0;
}

extern "C" size_t mccnn_weight_grad_product_workspace_bytes(int num_rows_out, int num_cols_out) {
  if (!tn_supported(num_rows_out, num_cols_out)) return 0;
  int slices = tn_slices(num_cols_out);          // room for either arrangement of the slices
  if (tn_split_supported(num_rows_out, num_cols_out) &&
      tn_split_slices(num_rows_out, num_cols_out) > slices)
    slices = tn_split_slices(num_rows_out, num_cols_out);
  return align256(sizeof(float) * (size_t)slices * num_rows_out * num_cols_out);
}

extern "C" int mccnn_weight_grad_product(mccnn_stream_t stream, int64_t num_pts, int num_rows_out,
                                         const float *x, int num_cols_out, const float *y,
                                         void *workspace, size_t workspace_bytes, float *out) {
  MCCNN_REQUIRE(tn_supported(num_rows_out, num_cols_out),
                "weight_grad_product supports 16/32/64/128 output rows and a multiple of 256 "
                "(at most 4096) output columns (got %d x %d)", num_rows_out, num_cols_out);
  MCCNN_REQUIRE(num_pts >= 0 && num_pts < ((int64_t)1 << 31),
                "weight_grad_product expects a size in [0, 2^31)");
  MCCNN_REQUIRE(out && workspace && (num_pts == 0 || (x && y)),
                "weight_grad_product received a null tensor");
  MCCNN_REQUIRE(workspace_bytes >=
                    mccnn_weight_grad_product_workspace_bytes(num_rows_out, num_cols_out),
                "weight_grad_product workspace too small");
  hipStream_t s = as_stream(stream);
  // slices of the point range, each reduced on its own: at least 128 points per slice, so that a
  // small cloud does not pay for summing a thousand empty partials and still fills the device
  const int C = num_rows_out, R = num_cols_out;
  const bool split = split_products_enabled() && tn_split_supported(C, R);
  int slices = split ? tn_split_slices(C, R) : tn_slices(R);
  const int64_t by_size = (num_pts + 127) / 128;
  if (slices > by_size) slices = by_size < 1 ? 1 : (int)by_size;
  const dim3 grid((R / 256) * slices), block(256);
  float *partials = (float *)workspace;
  const int64_t elems = (int64_t)C * R;
  if (split) {
    int rc = launch_tn_split(s, num_pts, C, x, R, y, slices, partials);
    if (rc != MCCNN_OK) return rc;
    hipLaunchKernelGGL(tn_reduce_kernel, dim3(blocks_for(elems, 256)), dim3(256), 0, s, elems,
                       slices, partials, out);
    MCCNN_LAUNCH_CHECK();
    return MCCNN_OK;
  }
  // 128 channels: operands staged through LDS (3.80 against 4.14 ms on [825 274, 128]^T x
  // [825 274, 2048]); up to 64 channels the direct kernel is as fast (1.18 / 1.21 ms on
  // [763 063, 64]^T x [763 063, 1024])
  switch (C / 16) {
    case 8: hipLaunchKernelGGL(tn_tile_kernel<8>, grid, block, 0, s, num_pts, R, x, y, slices, partials); break;
    case 4: hipLaunchKernelGGL(tn_product_kernel<4>, grid, block, 0, s, num_pts, R, x, y, slices, partials); break;
    case 2: hipLaunchKernelGGL(tn_product_kernel<2>, grid, block, 0, s, num_pts, R, x, y, slices, partials); break;
    default: hipLaunchKernelGGL(tn_product_kernel<1>, grid, block, 0, s, num_pts, R, x, y, slices, partials); break;
  }
  MCCNN_LAUNCH_CHECK();
  hipLaunchKernelGGL(tn_reduce_kernel, dim3(blocks_for(elems, 256)), dim3(256), 0, s, elems,
                     slices, partials, out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_projection_grad_product_supported(int num_cols_in, int num_cols_out) {
  return nt_supported(num_cols_in, num_cols_out) ? 1 : 0;
}

extern "C" int mccnn_projection_grad_product(mccnn_stream_t stream, int64_t num_pts,
                                             int num_cols_in, const float *x, int num_cols_out,
                                             const float *w, float *out) {
  MCCNN_REQUIRE(nt_supported(num_cols_in, num_cols_out),
                "projection_grad_product supports 16/32/64/128/256 input columns and a multiple of "
                "256/256/256/128/64 output columns (got %d -> %d)", num_cols_in, num_cols_out);
  MCCNN_REQUIRE(num_pts >= 0 && num_pts < ((int64_t)1 << 31),
                "projection_grad_product expects a size in [0, 2^31)");
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(x && w && out, "projection_grad_product received a null tensor");
  hipStream_t s = as_stream(stream);
  if (split_products_enabled() && nt_split_supported(num_cols_in, num_cols_out))
    return launch_nt_split(s, num_pts, num_cols_in, x, num_cols_out, w, out);
  const int F = num_cols_in, R = num_cols_out, groups = R / (64 * nt_cols(F));
  // one round of blocks: the kernel keeps 3 blocks of 4 wavefronts resident per compute unit
  // (136 registers), and a grid of exactly that many leaves no partly filled last round
  // (2048 blocks on 256 units: 2.7 rounds, 8 % slower)
  int device = 0, cus = 0;
  MCCNN_HIP_CHECK(hipGetDevice(&device));
  MCCNN_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  int slices = 3 * cus / groups;
  if (slices < 1) slices = 1;
  const int64_t tiles = (num_pts + 15) / 16;
  if (slices > tiles) slices = (int)tiles;
  const dim3 grid(groups * slices), block(256);
  switch (F) {
    case 256: hipLaunchKernelGGL((nt_product_kernel<256, 1>), grid, block, 0, s, num_pts, R, x, w, slices, out); break;
    case 128: hipLaunchKernelGGL((nt_product_kernel<128, 2>), grid, block, 0, s, num_pts, R, x, w, slices, out); break;
    case 64: hipLaunchKernelGGL((nt_product_kernel<64, 4>), grid, block, 0, s, num_pts, R, x, w, slices, out); break;
    case 32: hipLaunchKernelGGL((nt_product_kernel<32, 4>), grid, block, 0, s, num_pts, R, x, w, slices, out); break;
    default: hipLaunchKernelGGL((nt_product_kernel<16, 4>), grid, block, 0, s, num_pts, R, x, w, slices, out); break;
  }
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
