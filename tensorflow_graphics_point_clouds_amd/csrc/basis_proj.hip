// Basis projection and its gradients
// (custom_ops/tfg_custom_ops/basis_proj/cc/kernels/basis_proj_kernels.cu.cc:29-127,
//  basis_proj_grads_kernels.cu.cc:29-151):
//   out[i,c,k]   = sum_m feat[nbr_m, c] * basis[m, k]        (pairs m of centre i)
//   dbasis[m,k]  = sum_c g[i,c,k] * feat[nbr_m, c]
//   dfeat[n,c]  += sum_k g[i,c,k] * basis[m,k]               (n = nbr_m)
//
// Per centre this is a [C x n_i] x [n_i x K] contraction whose operands are
// streamed once: the basis rows of a centre are contiguous, the feature rows
// are gathered.  All element offsets are 64-bit (N*C*K and M*K exceed 2^31 at
// the benchmark sizes).
//
// Generic path (any valid C, K): one wavefront per (centre, chunk of up to
// 64*kAcc output elements); lane l owns elements l + 64*j, so its basis column
// k = l % K is fixed and its channel advances by 64/K per j.
#include "common.h"
#include "fill.h"
#include "mfma.h"

namespace mccnn {

constexpr int kAcc = 16;   // accumulators per lane in the generic kernels

template <int K>
__global__ void __launch_bounds__(256) basis_proj_generic_kernel(
    int64_t n_out, int C, int chunks, const float *__restrict__ basis,
    const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, const int *__restrict__ order, float *__restrict__ out) {
  constexpr int kChanStep = kWave / K;            // channels covered by one j
  const int lane = lane_id();
  const int64_t wid = wave_slot();
  const int64_t slot_centre = wid / chunks;
  if (slot_centre >= n_out) return;
  const int chunk = (int)(wid - slot_centre * chunks);
  const int64_t centre = centre_of(slot_centre, order);
  const int c0 = chunk * kAcc * kChanStep + lane / K;
  const int k = lane % K;
  const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
  float acc[kAcc];
#pragma unroll
  for (int j = 0; j < kAcc; ++j) acc[j] = 0.0f;
  for (int m = a; m < b; ++m) {
    const int64_t nb = nbrs[m].x;
    const float w = basis[(int64_t)m * K + k];
    const float *f = feat + nb * C;
#pragma unroll
    for (int j = 0; j < kAcc; ++j) {
      const int c = c0 + j * kChanStep;
      if (c < C) acc[j] += f[c] * w;
    }
  }
  float *o = out + centre * (int64_t)C * K;
#pragma unroll
  for (int j = 0; j < kAcc; ++j) {
    const int c = c0 + j * kChanStep;
    if (c < C) o[c * K + k] = acc[j];
  }
}

// kAtomicBasis: more than one chunk contributes to dbasis[m,:].
template <int K>
__global__ void __launch_bounds__(256) basis_proj_grads_generic_kernel(
    int64_t n_out, int C, int chunks, const float *__restrict__ basis,
    const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, const int *__restrict__ order, const float *__restrict__ in_grad,
    float *__restrict__ dbasis, float *__restrict__ dfeat) {
  constexpr int kChanStep = kWave / K;
  const int lane = lane_id();
  const int64_t wid = wave_slot();
  const int64_t slot_centre = wid / chunks;
  if (slot_centre >= n_out) return;
  const int chunk = (int)(wid - slot_centre * chunks);
  const int64_t centre = centre_of(slot_centre, order);
  const int c0 = chunk * kAcc * kChanStep + lane / K;
  const int k = lane % K;
  const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
  const float *gi = in_grad + centre * (int64_t)C * K;
  float g[kAcc];
#pragma unroll
  for (int j = 0; j < kAcc; ++j) {
    const int c = c0 + j * kChanStep;
    g[j] = c < C ? gi[c * K + k] : 0.0f;
  }
  for (int m = a; m < b; ++m) {
    const int64_t nb = nbrs[m].x;
    const float w = basis[(int64_t)m * K + k];
    const float *f = feat + nb * C;
    float db = 0.0f;
#pragma unroll
    for (int j = 0; j < kAcc; ++j) {
      const int c = c0 + j * kChanStep;
      const float fc = c < C ? f[c] : 0.0f;
      db += g[j] * fc;
      // sum over k (the K consecutive lanes that share this channel)
      float df = g[j] * w;
#pragma unroll
      for (int off = K / 2; off > 0; off >>= 1) df += __shfl_xor(df, off, kWave);
      if (k == 0 && c < C) unsafeAtomicAdd(&dfeat[nb * C + c], df);
    }
    // sum over the lanes that hold the same k (stride K)
#pragma unroll
    for (int off = K; off < kWave; off <<= 1) db += __shfl_xor(db, off, kWave);
    if (lane < K) {
      if (chunks > 1) unsafeAtomicAdd(&dbasis[(int64_t)m * K + k], db);
      else dbasis[(int64_t)m * K + k] = db;
    }
  }
}

// ---------------------------------------------------------------------------
// Matrix-core forward path.  One wavefront owns a centre (and a chunk of kCW
// channels) and accumulates the [channels x K] tile in MFMA accumulators while
// it streams the centre's pairs:
//   K = 32 / 64 : v_mfma_f32_32x32x2f32, rows = channels, columns = basis, two
//                 pairs per instruction (lanes 0-31 feed pair 2t, 32-63 pair 2t+1)
//   K = 16      : v_mfma_f32_16x16x4f32, rows = basis, columns = channels, four
//                 pairs per instruction (one per 16-lane quarter)
// Operands go from global memory straight into the MFMA register layout: a lane
// reads kCPL consecutive channels of one feature row (up to 16 B) and its basis
// column(s); kCPL tiles share the lane's row/column index, tile j holding the
// channels {lane_channel_base + j}.  Neighbour ids are read 64 at a time,
// coalesced, and broadcast with a lane shuffle.  Results leave with
// non-temporal stores (write-once stream).

constexpr int kUnroll = 4;   // MFMA steps whose loads are issued together

template <int K, int kCPL>
__global__ void __launch_bounds__(256) basis_proj_mfma32_kernel(
    int64_t n_out, int C, int chunks, const float *__restrict__ basis,
    const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, const int *__restrict__ order, float *__restrict__ out) {
  static_assert(K == 32 || K == 64, "32x32x2 path");
  constexpr int kNT = K / 32;        // basis columns per lane
  constexpr int kCW = 32 * kCPL;     // channels per wave
  const int lane = lane_id();
  const int64_t wid = wave_slot();
  const int64_t slot_centre = wid / chunks;
  if (slot_centre >= n_out) return;
  const int chunk = (int)(wid - slot_centre * chunks);
  const int64_t centre = centre_of(slot_centre, order);
  const int half = lane >> 5, col = lane & 31;
  const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
  const float *fbase = feat + chunk * kCW + col * kCPL;
  const float *bbase = basis + col * kNT;
  v16f acc[kCPL][kNT];
#pragma unroll
  for (int j = 0; j < kCPL; ++j)
#pragma unroll
    for (int q = 0; q < kNT; ++q)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][q][r] = 0.0f;

  for (int m0 = a; m0 < b; m0 += kWave) {
    const int cnt = b - m0 < kWave ? b - m0 : kWave;
    const int myidx = nbrs[m0 + (lane < cnt ? lane : 0)].x;
    const int steps = (cnt + 1) >> 1;
    for (int t = 0; t < steps; t += kUnroll) {
      FVec<kCPL> f[kUnroll];
      FVec<kNT> w[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int n = 2 * (t + u) + half;
        const bool valid = n < cnt;
        const int idx = __shfl(myidx, n & (kWave - 1), kWave);
        f[u] = load_vec<kCPL>(fbase + (int64_t)idx * C, valid);
        w[u] = load_vec<kNT>(bbase + (int64_t)(m0 + n) * K, valid);
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
#pragma unroll
        for (int j = 0; j < kCPL; ++j)
#pragma unroll
          for (int q = 0; q < kNT; ++q)
            acc[j][q] = __builtin_amdgcn_mfma_f32_32x32x2f32(f[u].v[j], w[u].v[q], acc[j][q], 0, 0, 0);
    }
  }
  // D[i][col]: i = 8*(r/4) + (r%4) + 4*half is the lane-row whose channels are
  // i*kCPL + j; column col holds basis columns col*kNT + q.
  float *o = out + centre * (int64_t)C * K + (int64_t)chunk * kCW * K + col * kNT;
#pragma unroll
  for (int j = 0; j < kCPL; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 8 * (r >> 2) + (r & 3) + 4 * half;
      float *dst = o + (i * kCPL + j) * K;
      if constexpr (kNT == 1) {
        __builtin_nontemporal_store(acc[j][0][r], dst);
      } else {
        __builtin_nontemporal_store(acc[j][0][r], dst);
        __builtin_nontemporal_store(acc[j][1][r], dst + 1);
      }
    }
}

template <int kCPL>
__global__ void __launch_bounds__(256) basis_proj_mfma16_kernel(
    int64_t n_out, int C, int chunks, const float *__restrict__ basis,
    const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, const int *__restrict__ order, float *__restrict__ out) {
  constexpr int K = 16;
  constexpr int kCW = 16 * kCPL;
  const int lane = lane_id();
  const int64_t wid = wave_slot();
  const int64_t slot_centre = wid / chunks;
  if (slot_centre >= n_out) return;
  const int chunk = (int)(wid - slot_centre * chunks);
  const int64_t centre = centre_of(slot_centre, order);
  const int quarter = lane >> 4, col = lane & 15;
  const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
  const float *fbase = feat + chunk * kCW + col * kCPL;
  const float *bbase = basis + col;
  v4f acc[kCPL];
#pragma unroll
  for (int j = 0; j < kCPL; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[j][r] = 0.0f;

  for (int m0 = a; m0 < b; m0 += kWave) {
    const int cnt = b - m0 < kWave ? b - m0 : kWave;
    const int myidx = nbrs[m0 + (lane < cnt ? lane : 0)].x;
    const int steps = (cnt + 3) >> 2;
    for (int t = 0; t < steps; t += kUnroll) {
      FVec<kCPL> f[kUnroll];
      float w[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int n = 4 * (t + u) + quarter;
        const bool valid = n < cnt;
        const int idx = __shfl(myidx, n & (kWave - 1), kWave);
        f[u] = load_vec<kCPL>(fbase + (int64_t)idx * C, valid);
        w[u] = valid ? bbase[(int64_t)(m0 + n) * K] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
#pragma unroll
        for (int j = 0; j < kCPL; ++j)
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u], f[u].v[j], acc[j], 0, 0, 0);
    }
  }
  // D[k][c]: rows k = 4*quarter + r, column col <-> channel col*kCPL + j:
  // four consecutive basis columns per lane -> one 16-byte store.
  float *o = out + centre * (int64_t)C * K + (int64_t)chunk * kCW * K + 4 * quarter;
#pragma unroll
  for (int j = 0; j < kCPL; ++j) {
    float *dst = o + (col * kCPL + j) * K;
    *reinterpret_cast<v4f *>(dst) = acc[j];
  }
}

// ---------------------------------------------------------------------------
// Matrix-core gradient path.  One wavefront owns a centre and walks its pairs in
// tiles of 32 (K = 32) or 16 (K = 16).  Per tile, two contractions:
//   dbasis^T [K x pairs]   = G^T [K x C] * F^T [C x pairs]   (reduction over c)
//   dfeat    [pairs x C]   = B [pairs x K] * G^T [K x C]     (reduction over k)
// with G = in_grad[centre] ([C, K]).  The reduction index of an MFMA may be
// permuted freely as long as both operands agree, so each lane is given a
// CONTIGUOUS run of the reduction index: its share of a feature row, of a basis
// row and of a G row are 16-byte vector loads.  dbasis rows leave as contiguous
// 16-byte stores (each pair belongs to exactly one centre: no atomics); dfeat
// rows are added with one fp32 atomic per element, 64/128 consecutive bytes per
// row and instruction.

template <int C>
__global__ void __launch_bounds__(256) basis_proj_grads_mfma32_kernel(
    int64_t n_out, const float *__restrict__ basis, const float *__restrict__ feat,
    const int2 *__restrict__ nbrs, const int *__restrict__ ranges, const int *__restrict__ order,
    const float *__restrict__ in_grad, float *__restrict__ dbasis, float *__restrict__ dfeat,
    float *__restrict__ pair_rows) {
  constexpr int K = 32;
  constexpr int kHalfC = C / 2;      // reduction run of a lane in the dbasis product
  const int lane = lane_id();
  const int64_t slot_centre = wave_slot();
  if (slot_centre >= n_out) return;
  const int64_t centre = centre_of(slot_centre, order);
  const int half = lane >> 5, col = lane & 31;
  const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
  if (b <= a) return;
  const float *gi = in_grad + centre * (int64_t)C * K;
  // A operand of the dbasis product: G[c = half*C/2 + s][k = col]
  float gk[kHalfC];
#pragma unroll
  for (int s = 0; s < kHalfC; ++s) gk[s] = gi[(half * kHalfC + s) * K + col];

  for (int m0 = a; m0 < b; m0 += 32) {
    const int cnt = b - m0 < 32 ? b - m0 : 32;
    const bool valid = col < cnt;
    const int idx = nbrs[m0 + (valid ? col : 0)].x;
    // ---- dbasis: D[i = k][j = pair]; B operand F[nbr_col][half*C/2 + s]
    {
      const FVec<kHalfC> f = load_vec<kHalfC>(feat + (int64_t)idx * C + half * kHalfC, valid);
      v16f acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
      for (int s = 0; s < kHalfC; ++s)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(gk[s], f.v[s], acc, 0, 0, 0);
      // rows k = 8q + 4*half + (0..3) of column pair `col`
      if (valid) {
        float *dst = dbasis + (int64_t)(m0 + col) * K + 4 * half;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          v4f v = {acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
          *reinterpret_cast<v4f *>(dst + 8 * q) = v;
        }
      }
    }
    // ---- dfeat: D[i = pair][j = channel]; A operand B[pair col][k = 16*half + s]
    {
      const FVec<16> w = load_vec<16>(basis + (int64_t)(m0 + col) * K + 16 * half, valid);
#pragma unroll 1
      for (int ct = 0; ct < C; ct += 32) {
        const FVec<16> gt = load_vec<16>(gi + (ct + col) * K + 16 * half, true);
        v16f acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
        for (int s = 0; s < 16; ++s)
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w.v[s], gt.v[s], acc, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int n = 8 * (r >> 2) + (r & 3) + 4 * half;
          const int nidx = __shfl(idx, n, kWave);
          if (n < cnt) {
            if (pair_rows) pair_rows[(int64_t)(m0 + n) * C + ct + col] = acc[r];
            else unsafeAtomicAdd(dfeat + (int64_t)nidx * C + ct + col, acc[r]);
          }
        }
      }
    }
  }
}

template <int C>
__global__ void __launch_bounds__(256) basis_proj_grads_mfma16_kernel(
    int64_t n_out, const float *__restrict__ basis, const float *__restrict__ feat,
    const int2 *__restrict__ nbrs, const int *__restrict__ ranges, const int *__restrict__ order,
    const float *__restrict__ in_grad, float *__restrict__ dbasis, float *__restrict__ dfeat,
    float *__restrict__ pair_rows) {
  constexpr int K = 16;
  constexpr int kQuarterC = C / 4;
  constexpr int kTiles = C / 16;
  const int lane = lane_id();
  const int64_t slot_centre = wave_slot();
  if (slot_centre >= n_out) return;
  const int64_t centre = centre_of(slot_centre, order);
  const int quarter = lane >> 4, col = lane & 15;
  const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
  if (b <= a) return;
  const float *gi = in_grad + centre * (int64_t)C * K;
  // dbasis product, A operand: G[c = quarter*C/4 + s][k = col]
  float gk[kQuarterC];
#pragma unroll
  for (int s = 0; s < kQuarterC; ++s) gk[s] = gi[(quarter * kQuarterC + s) * K + col];
  // dfeat product, B operand of channel tile t: G[c = 16 t + col][k = 4*quarter + s]
  FVec<4> gt[kTiles];
#pragma unroll
  for (int t = 0; t < kTiles; ++t) gt[t] = load_vec<4>(gi + (16 * t + col) * K + 4 * quarter, true);

  for (int m0 = a; m0 < b; m0 += 16) {
    const int cnt = b - m0 < 16 ? b - m0 : 16;
    const bool valid = col < cnt;
    const int idx = nbrs[m0 + (valid ? col : 0)].x;
    {
      const FVec<kQuarterC> f =
          load_vec<kQuarterC>(feat + (int64_t)idx * C + quarter * kQuarterC, valid);
      v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int s = 0; s < kQuarterC; ++s)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(gk[s], f.v[s], acc, 0, 0, 0);
      // D[i = k][j = pair]: rows k = 4*quarter + (0..3)
      if (valid)
        __builtin_nontemporal_store(
            acc, reinterpret_cast<v4f *>(dbasis + (int64_t)(m0 + col) * K + 4 * quarter));
    }
    {
      const FVec<4> w = load_vec<4>(basis + (int64_t)(m0 + col) * K + 4 * quarter, valid);
#pragma unroll
      for (int t = 0; t < kTiles; ++t) {
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < 4; ++s)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.v[s], gt[t].v[s], acc, 0, 0, 0);
        // D[i = pair][j = channel]: rows pair = 4*quarter + r, column channel 16 t + col
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = 4 * quarter + r;
          const int nidx = __shfl(idx, n, kWave);
          if (n < cnt) {
            if (pair_rows) pair_rows[(int64_t)(m0 + n) * C + 16 * t + col] = acc[r];
            else unsafeAtomicAdd(dfeat + (int64_t)nidx * C + 16 * t + col, acc[r]);
          }
        }
      }
    }
  }
}

// Second phase of the atomic-free feature gradient: dfeat[n, :] = sum of the
// per-pair rows of the pairs whose neighbour is n.  point_ranges (inclusive ends)
// and pair_order list those pairs per point, in ascending pair index, so the sum
// has a fixed order.  kLanes lanes per point, one float4 each (C = 4 * kLanes).
template <int kLanes>
__global__ void __launch_bounds__(256) dfeat_gather_kernel(
    int64_t n_in, const int *__restrict__ point_ranges, const int *__restrict__ pair_order,
    const float *__restrict__ pair_rows, float *__restrict__ dfeat) {
  constexpr int C = 4 * kLanes;
  const int64_t n = (int64_t)blockIdx.x * (256 / kLanes) + threadIdx.x / kLanes;
  if (n >= n_in) return;
  const int sub = threadIdx.x % kLanes;
  const int a = n > 0 ? point_ranges[n - 1] : 0, b = point_ranges[n];
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  int j = a;
  for (; j + 4 <= b; j += 4) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      v[u] = *reinterpret_cast<const float4 *>(pair_rows + (int64_t)pair_order[j + u] * C + 4 * sub);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w;
    }
  }
  for (; j < b; ++j) {
    const float4 v =
        *reinterpret_cast<const float4 *>(pair_rows + (int64_t)pair_order[j] * C + 4 * sub);
    acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
  }
  *reinterpret_cast<float4 *>(dfeat + n * C + 4 * sub) = acc;
}

int launch_dfeat_gather(hipStream_t s, int64_t num_pts, int C, const int *point_ranges,
                        const int *pair_order, const float *pair_rows, float *dfeat) {
  if (num_pts == 0) return MCCNN_OK;
  const int lanes = C / 4;
  const dim3 grid(blocks_for(num_pts, 256 / lanes)), block(256);
  switch (lanes) {
    case 4: hipLaunchKernelGGL(dfeat_gather_kernel<4>, grid, block, 0, s, num_pts, point_ranges, pair_order, pair_rows, dfeat); break;
    case 8: hipLaunchKernelGGL(dfeat_gather_kernel<8>, grid, block, 0, s, num_pts, point_ranges, pair_order, pair_rows, dfeat); break;
    case 16: hipLaunchKernelGGL(dfeat_gather_kernel<16>, grid, block, 0, s, num_pts, point_ranges, pair_order, pair_rows, dfeat); break;
    case 32: hipLaunchKernelGGL(dfeat_gather_kernel<32>, grid, block, 0, s, num_pts, point_ranges, pair_order, pair_rows, dfeat); break;
    default:
      set_error("feature-gradient gather supports C in {16, 32, 64, 128} (got %d)", C);
      return MCCNN_INVALID_ARGUMENT;
  }
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

static bool mfma_grads_supported(int C, int K) {
  if (K == 32) return C == 32 || C == 64 || C == 128;
  if (K == 16) return C == 16 || C == 32 || C == 64 || C == 128;
  return false;
}

// Channels per lane for the matrix-core path, 0 when the shape needs the generic
// kernel.  Accumulator budget: at most 128 registers per lane.
static int mfma_channels_per_lane(int C, int K) {
  if (K == 16) {
    for (int cpl = 8; cpl >= 1; cpl >>= 1)
      if (C % (16 * cpl) == 0) return cpl;
  } else if (K == 32 || K == 64) {
    for (int cpl = 4; cpl >= 1; cpl >>= 1)
      if (C % (32 * cpl) == 0) return cpl;
  }
  return 0;
}

static int check_basis_args(const char *op, int64_t basis_rows, int num_basis, int num_features,
                            int64_t num_neighbors, int neighbors_rank, int neighbors_cols) {
  MCCNN_REQUIRE(num_basis == 8 || num_basis == 16 || num_basis == 32 || num_basis == 64,
                "%s expects a valid number of basis functions (8, 16, 32 or 64; got %d)", op,
                num_basis);
  MCCNN_REQUIRE(num_features > 0 && (num_features < 8 || num_features % 8 == 0),
                "%s expects a valid number of input features, between 1 and 8 or multiple of 8 "
                "(got %d)", op, num_features);
  MCCNN_REQUIRE(basis_rows == num_neighbors,
                "%s expects the same number of basis as the number of neighbors", op);
  MCCNN_REQUIRE(neighbors_rank == 2 && neighbors_cols == 2,
                "%s expects a neighbor tensor with 2 dimensions and 2 indices per neighbor", op);
  return MCCNN_OK;
}

static int generic_chunks(int C, int K) {
  const int per_chunk = kAcc * (kWave / K);   // channels per chunk
  return (C + per_chunk - 1) / per_chunk;
}

#define MCCNN_BASIS_SWITCH(K_, ...)                              \
  switch (K_) {                                                  \
    case 8:  { constexpr int K = 8;  __VA_ARGS__; } break;       \
    case 16: { constexpr int K = 16; __VA_ARGS__; } break;       \
    case 32: { constexpr int K = 32; __VA_ARGS__; } break;       \
    case 64: { constexpr int K = 64; __VA_ARGS__; } break;       \
  }

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_basis_proj_ordered(mccnn_stream_t stream, int64_t basis_rows, int num_basis,
                                        const float *basis, int64_t num_pts, int num_features,
                                        const float *features, int64_t num_neighbors,
                                        int neighbors_rank, int neighbors_cols,
                                        const int32_t *neighbors, int64_t num_samples,
                                        const int32_t *ranges, const int32_t *centre_order,
                                        float *out) {
  const int32_t *order = centre_order;
  int rc = check_basis_args("BasisProj", basis_rows, num_basis, num_features, num_neighbors,
                            neighbors_rank, neighbors_cols);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(num_pts >= 0 && num_samples >= 0 && num_neighbors >= 0 &&
                    num_neighbors < ((int64_t)1 << 31),
                "BasisProj expects sizes in [0, 2^31)");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && out && (num_neighbors == 0 || (basis && features && neighbors)),
                "BasisProj received a null tensor");
  hipStream_t s = as_stream(stream);
  const int cpl = mfma_channels_per_lane(num_features, num_basis);
  if (cpl > 0) {
    const int lanes_per_pair = num_basis == 16 ? 16 : 32;
    const int chunks = num_features / (lanes_per_pair * cpl);
    const int64_t waves = num_samples * chunks;
    MCCNN_REQUIRE(waves < ((int64_t)1 << 31), "BasisProj launch too large");
    const dim3 grid(wave_grid(waves)), block(256);
    const int2 *nb = (const int2 *)neighbors;
#define MCCNN_FWD32(K_, CPL_)                                                                  \
  hipLaunchKernelGGL((basis_proj_mfma32_kernel<K_, CPL_>), grid, block, 0, s, num_samples,     \
                     num_features, chunks, basis, features, nb, ranges, order, out)
#define MCCNN_FWD16(CPL_)                                                                      \
  hipLaunchKernelGGL((basis_proj_mfma16_kernel<CPL_>), grid, block, 0, s, num_samples,         \
                     num_features, chunks, basis, features, nb, ranges, order, out)
    if (num_basis == 16) {
      switch (cpl) {
        case 8: MCCNN_FWD16(8); break;
        case 4: MCCNN_FWD16(4); break;
        case 2: MCCNN_FWD16(2); break;
        default: MCCNN_FWD16(1); break;
      }
    } else if (num_basis == 32) {
      switch (cpl) {
        case 4: MCCNN_FWD32(32, 4); break;
        case 2: MCCNN_FWD32(32, 2); break;
        default: MCCNN_FWD32(32, 1); break;
      }
    } else {
      switch (cpl) {
        case 4: MCCNN_FWD32(64, 4); break;
        case 2: MCCNN_FWD32(64, 2); break;
        default: MCCNN_FWD32(64, 1); break;
      }
    }
#undef MCCNN_FWD32
#undef MCCNN_FWD16
    MCCNN_LAUNCH_CHECK();
    return MCCNN_OK;
  }
  const int chunks = generic_chunks(num_features, num_basis);
  const int64_t waves = num_samples * chunks;
  MCCNN_REQUIRE(waves < ((int64_t)1 << 31), "BasisProj launch too large");
  const unsigned grid = wave_grid(waves);
  MCCNN_BASIS_SWITCH(num_basis,
                     hipLaunchKernelGGL(basis_proj_generic_kernel<K>, dim3(grid), dim3(256), 0,
                                        s, num_samples, num_features, chunks,
                                        basis, features, (const int2 *)neighbors, ranges, order,
                                        out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

static int basis_proj_grads_impl(
    mccnn_stream_t stream, int64_t basis_rows, int num_basis, const float *basis, int64_t num_pts,
    int num_features, const float *features, int64_t num_neighbors, int neighbors_rank,
    int neighbors_cols, const int32_t *neighbors, int64_t num_samples, const int32_t *ranges,
    const int32_t *order, int in_grads_rank, int64_t in_grads_dim0, int64_t in_grads_dim1,
    int64_t in_grads_dim2, const float *in_grads, const int32_t *point_ranges,
    const int32_t *pair_order, float *pair_rows, float *basis_grads_out,
    float *feature_grads_out) {
  const bool gathered = pair_rows != nullptr;
  if (gathered) {
    MCCNN_REQUIRE(point_ranges && pair_order,
                  "BasisProjGrads needs the transposed pair lists with a pair-row workspace");
    MCCNN_REQUIRE(mfma_grads_supported(num_features, num_basis),
                  "the gathered feature gradient supports K in {16,32} and C in {16,32,64,128} "
                  "(C >= 32 for K = 32)");
  }
  int rc = check_basis_args("BasisProjGrads", basis_rows, num_basis, num_features, num_neighbors,
                            neighbors_rank, neighbors_cols);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(in_grads_rank == 3 && in_grads_dim0 == num_samples &&
                    in_grads_dim1 == num_features && in_grads_dim2 == num_basis,
                "BasisProjGrads expects gradients of shape [num_samples, num_features, num_basis]");
  MCCNN_REQUIRE(num_pts >= 0 && num_samples >= 0 && num_neighbors >= 0 &&
                    num_neighbors < ((int64_t)1 << 31),
                "BasisProjGrads expects sizes in [0, 2^31)");
  hipStream_t s = as_stream(stream);
  if (num_pts > 0 && (!gathered || num_samples == 0 || num_neighbors == 0)) {
    MCCNN_REQUIRE(feature_grads_out, "BasisProjGrads received a null tensor");
    rc = fill_zero(s, feature_grads_out, sizeof(float) * (size_t)num_pts * num_features);
    if (rc != MCCNN_OK) return rc;
  }
  if (num_samples == 0 || num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && basis && features && neighbors && in_grads && basis_grads_out,
                "BasisProjGrads received a null tensor");
  const int2 *nb = (const int2 *)neighbors;
  if (mfma_grads_supported(num_features, num_basis)) {
    MCCNN_REQUIRE(num_samples < ((int64_t)1 << 31), "BasisProjGrads launch too large");
    const dim3 grid(wave_grid(num_samples)), block(256);
#define MCCNN_BWD(KERNEL_, C_)                                                              \
  hipLaunchKernelGGL((KERNEL_<C_>), grid, block, 0, s, num_samples, basis, features, nb,   \
                     ranges, order, in_grads, basis_grads_out, feature_grads_out, pair_rows)
    if (num_basis == 32) {
      switch (num_features) {
        case 32: MCCNN_BWD(basis_proj_grads_mfma32_kernel, 32); break;
        case 64: MCCNN_BWD(basis_proj_grads_mfma32_kernel, 64); break;
        default: MCCNN_BWD(basis_proj_grads_mfma32_kernel, 128); break;
      }
    } else {
      switch (num_features) {
        case 16: MCCNN_BWD(basis_proj_grads_mfma16_kernel, 16); break;
        case 32: MCCNN_BWD(basis_proj_grads_mfma16_kernel, 32); break;
        case 64: MCCNN_BWD(basis_proj_grads_mfma16_kernel, 64); break;
        default: MCCNN_BWD(basis_proj_grads_mfma16_kernel, 128); break;
      }
    }
#undef MCCNN_BWD
    MCCNN_LAUNCH_CHECK();
    if (gathered)
      return launch_dfeat_gather(s, num_pts, num_features, point_ranges, pair_order, pair_rows,
                                 feature_grads_out);
    return MCCNN_OK;
  }
  const int chunks = generic_chunks(num_features, num_basis);
  if (chunks > 1) {
    rc = fill_zero(s, basis_grads_out, sizeof(float) * (size_t)num_neighbors * num_basis);
    if (rc != MCCNN_OK) return rc;
  }
  const int64_t waves = num_samples * chunks;
  MCCNN_REQUIRE(waves < ((int64_t)1 << 31), "BasisProjGrads launch too large");
  const unsigned grid = wave_grid(waves);
  MCCNN_BASIS_SWITCH(num_basis, hipLaunchKernelGGL(basis_proj_grads_generic_kernel<K>, dim3(grid),
                                                   dim3(256), 0, s, num_samples, num_features,
                                                   chunks, basis, features, nb, ranges, order,
                                                   in_grads,
                                                   basis_grads_out, feature_grads_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_basis_proj(mccnn_stream_t stream, int64_t basis_rows, int num_basis,
                                const float *basis, int64_t num_pts, int num_features,
                                const float *features, int64_t num_neighbors, int neighbors_rank,
                                int neighbors_cols, const int32_t *neighbors,
                                int64_t num_samples, const int32_t *ranges, float *out) {
  return mccnn_basis_proj_ordered(stream, basis_rows, num_basis, basis, num_pts, num_features,
                                  features, num_neighbors, neighbors_rank, neighbors_cols,
                                  neighbors, num_samples, ranges, nullptr, out);
}

extern "C" int mccnn_basis_proj_grads_ordered(
    mccnn_stream_t stream, int64_t basis_rows, int num_basis, const float *basis, int64_t num_pts,
    int num_features, const float *features, int64_t num_neighbors, int neighbors_rank,
    int neighbors_cols, const int32_t *neighbors, int64_t num_samples, const int32_t *ranges,
    const int32_t *centre_order, int in_grads_rank, int64_t in_grads_dim0, int64_t in_grads_dim1,
    int64_t in_grads_dim2, const float *in_grads, float *basis_grads_out,
    float *feature_grads_out) {
  return basis_proj_grads_impl(stream, basis_rows, num_basis, basis, num_pts, num_features,
                               features, num_neighbors, neighbors_rank, neighbors_cols, neighbors,
                               num_samples, ranges, centre_order, in_grads_rank, in_grads_dim0,
                               in_grads_dim1, in_grads_dim2, in_grads, nullptr, nullptr, nullptr,
                               basis_grads_out, feature_grads_out);
}

extern "C" int mccnn_basis_proj_grads_gathered(
    mccnn_stream_t stream, int64_t basis_rows, int num_basis, const float *basis, int64_t num_pts,
    int num_features, const float *features, int64_t num_neighbors, int neighbors_rank,
    int neighbors_cols, const int32_t *neighbors, int64_t num_samples, const int32_t *ranges,
    int in_grads_rank, int64_t in_grads_dim0, int64_t in_grads_dim1, int64_t in_grads_dim2,
    const float *in_grads, const int32_t *point_ranges, const int32_t *pair_order,
    float *pair_rows_workspace, float *basis_grads_out, float *feature_grads_out) {
  MCCNN_REQUIRE(pair_rows_workspace || num_neighbors == 0,
                "BasisProjGrads (gathered) needs a [num_neighbors, C] workspace");
  return basis_proj_grads_impl(stream, basis_rows, num_basis, basis, num_pts, num_features,
                               features, num_neighbors, neighbors_rank, neighbors_cols, neighbors,
                               num_samples, ranges, nullptr, in_grads_rank, in_grads_dim0,
                               in_grads_dim1, in_grads_dim2, in_grads, point_ranges, pair_order,
                               pair_rows_workspace, basis_grads_out, feature_grads_out);
}

extern "C" int mccnn_basis_proj_grads(mccnn_stream_t stream, int64_t basis_rows, int num_basis,
                                      const float *basis, int64_t num_pts, int num_features,
                                      const float *features, int64_t num_neighbors,
                                      int neighbors_rank, int neighbors_cols,
                                      const int32_t *neighbors, int64_t num_samples,
                                      const int32_t *ranges, int in_grads_rank,
                                      int64_t in_grads_dim0, int64_t in_grads_dim1,
                                      int64_t in_grads_dim2, const float *in_grads,
                                      float *basis_grads_out, float *feature_grads_out) {
  return basis_proj_grads_impl(stream, basis_rows, num_basis, basis, num_pts, num_features,
                               features, num_neighbors, neighbors_rank, neighbors_cols, neighbors,
                               num_samples, ranges, nullptr, in_grads_rank, in_grads_dim0,
                               in_grads_dim1, in_grads_dim2, in_grads, nullptr, nullptr, nullptr,
                               basis_grads_out, feature_grads_out);
}
