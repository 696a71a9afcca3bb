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

namespace mccnn {

constexpr int kAcc = 16;   // accumulators per lane in the generic kernels

template <int K>
__global__ void __launch_bounds__(256) basis_proj_generic_kernel(
    int64_t n_out, int C, int chunks, const float *__restrict__ basis,
    const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, float *__restrict__ out) {
  constexpr int kChanStep = kWave / K;            // channels covered by one j
  const int lane = lane_id();
  const int64_t wid =
      __builtin_amdgcn_readfirstlane((int)((blockIdx.x * (int64_t)blockDim.x + threadIdx.x) / kWave));
  const int64_t centre = wid / chunks;
  if (centre >= n_out) return;
  const int chunk = (int)(wid - centre * chunks);
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
    const int *__restrict__ ranges, const float *__restrict__ in_grad,
    float *__restrict__ dbasis, float *__restrict__ dfeat) {
  constexpr int kChanStep = kWave / K;
  const int lane = lane_id();
  const int64_t wid =
      __builtin_amdgcn_readfirstlane((int)((blockIdx.x * (int64_t)blockDim.x + threadIdx.x) / kWave));
  const int64_t centre = wid / chunks;
  if (centre >= n_out) return;
  const int chunk = (int)(wid - centre * chunks);
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

extern "C" int mccnn_basis_proj(mccnn_stream_t stream, int64_t basis_rows, int num_basis,
                                const float *basis, int64_t num_pts, int num_features,
                                const float *features, int64_t num_neighbors, int neighbors_rank,
                                int neighbors_cols, const int32_t *neighbors,
                                int64_t num_samples, const int32_t *ranges, float *out) {
  int rc = check_basis_args("BasisProj", basis_rows, num_basis, num_features, num_neighbors,
                            neighbors_rank, neighbors_cols);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(num_pts >= 0 && num_samples >= 0 && num_neighbors >= 0 &&
                    num_neighbors < ((int64_t)1 << 31),
                "BasisProj expects sizes in [0, 2^31)");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && out && (num_neighbors == 0 || (basis && features && neighbors)),
                "BasisProj received a null tensor");
  const int chunks = generic_chunks(num_features, num_basis);
  const int64_t waves = num_samples * chunks;
  MCCNN_REQUIRE(waves < ((int64_t)1 << 31), "BasisProj launch too large");
  const unsigned grid = blocks_for(waves, 256 / kWave);
  MCCNN_BASIS_SWITCH(num_basis,
                     hipLaunchKernelGGL(basis_proj_generic_kernel<K>, dim3(grid), dim3(256), 0,
                                        as_stream(stream), num_samples, num_features, chunks,
                                        basis, features, (const int2 *)neighbors, ranges, out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
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
  if (num_pts > 0) {
    MCCNN_REQUIRE(feature_grads_out, "BasisProjGrads received a null tensor");
    rc = fill_zero(s, feature_grads_out, sizeof(float) * (size_t)num_pts * num_features);
    if (rc != MCCNN_OK) return rc;
  }
  if (num_samples == 0 || num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && basis && features && neighbors && in_grads && basis_grads_out,
                "BasisProjGrads received a null tensor");
  const int chunks = generic_chunks(num_features, num_basis);
  if (chunks > 1) {
    rc = fill_zero(s, basis_grads_out, sizeof(float) * (size_t)num_neighbors * num_basis);
    if (rc != MCCNN_OK) return rc;
  }
  const int64_t waves = num_samples * chunks;
  MCCNN_REQUIRE(waves < ((int64_t)1 << 31), "BasisProjGrads launch too large");
  const unsigned grid = blocks_for(waves, 256 / kWave);
  MCCNN_BASIS_SWITCH(num_basis, hipLaunchKernelGGL(basis_proj_grads_generic_kernel<K>, dim3(grid),
                                                   dim3(256), 0, s, num_samples, num_features,
                                                   chunks, basis, features,
                                                   (const int2 *)neighbors, ranges, in_grads,
                                                   basis_grads_out, feature_grads_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
