// Helpers shared by the matrix-core kernels (basis projection and the fused
// Monte-Carlo convolution path).
#pragma once
#include "common.h"

namespace mccnn {

// Wave slot -> centre.  `order` (optional) is a permutation of the centres that
// fixes the visiting order; it is a scheduling hint only.  (Dealing contiguous
// slot ranges to the 8 XCDs and visiting the centres in cell order were both
// measured and left out: the feature rows already hit the memory-side cache,
// and concentrating the feature-gradient atomics of neighbouring centres in
// time made them slower.)
constexpr int kWavesPerBlock = 256 / kWave;

__device__ __forceinline__ int64_t wave_slot() {
  return __builtin_amdgcn_readfirstlane(
      (int)(blockIdx.x * kWavesPerBlock + threadIdx.x / kWave));
}

// The same with the blocks renumbered for the eight XCDs, each of which has its own L2:
// the hardware deals consecutive blocks to the XCDs in turn (block b runs on XCD b % 8),
// so plain numbering sends neighbouring centres -- which share most of their feature
// rows on a grid-ordered table -- to eight different caches, and each row is fetched from
// HBM up to eight times.  Here XCD x works through windows of kXcdWindow consecutive
// virtual blocks (x, x + 8, x + 16, ... in units of windows), so its resident blocks are
// neighbours.  Measured on the 763 k-point scene batch (projection kernel): read requests
// to the fabric 28.9 M -> 6.3 M per launch at equal run time (windows of 8 / 32 / 128 /
// 512 blocks: 14.3 / 10.1 / 6.3 / 6.6 M; one contiguous eighth per XCD is 10 % slower,
// the XCDs then finish at different times on clustered clouds).
constexpr unsigned kXcdWindow = 128;
__device__ __forceinline__ int64_t wave_slot_xcd() {
  const unsigned b = blockIdx.x;
  const unsigned full = gridDim.x / (8 * kXcdWindow) * (8 * kXcdWindow);   // the rest keeps its number
  const unsigned v = b < full ? ((b / (8 * kXcdWindow)) * 8 + b % 8) * kXcdWindow + (b / 8) % kXcdWindow : b;
  return __builtin_amdgcn_readfirstlane((int)(v * kWavesPerBlock + threadIdx.x / kWave));
}

__device__ __forceinline__ int64_t centre_of(int64_t slot_centre, const int *__restrict__ order) {
  return order ? (int64_t)__builtin_amdgcn_readfirstlane(order[slot_centre]) : slot_centre;
}

static unsigned wave_grid(int64_t waves) {
  const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
  return (unsigned)(blocks < 1 ? 1 : blocks);
}


// dfeat[n, :] = sum over the pairs listed for point n of pair_rows[pair, :]
// (defined in basis_proj.hip).
int launch_dfeat_gather(hipStream_t s, int64_t num_pts, int C, const int *point_ranges,
                        const int *pair_order, const float *pair_rows, float *dfeat);

// out = x * w for x [N, R], w [R, F] as a tiled product (defined in dense.hip): for weight
// matrices too large for the register-resident product of mc_layer.hip.
bool tile_product_supported(int R, int F);
int tile_product_rows(int F);
int launch_tile_product(hipStream_t s, int64_t n, int R, const float *x, int F, const float *w,
                        bool w_transposed, const int *out_rows, float *out);

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));

template <int N>
struct FVec {
  float v[N];
};

template <int N>
__device__ __forceinline__ FVec<N> load_vec(const float *__restrict__ p, bool valid) {
  FVec<N> r;
#pragma unroll
  for (int i = 0; i < N; ++i) r.v[i] = 0.0f;
  if (valid) {
    if constexpr (N % 4 == 0) {
#pragma unroll
      for (int i = 0; i < N / 4; ++i) {
        const float4 t = reinterpret_cast<const float4 *>(p)[i];
        r.v[4 * i] = t.x; r.v[4 * i + 1] = t.y; r.v[4 * i + 2] = t.z; r.v[4 * i + 3] = t.w;
      }
    } else if constexpr (N == 2) {
      const float2 t = *reinterpret_cast<const float2 *>(p);
      r.v[0] = t.x; r.v[1] = t.y;
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i) r.v[i] = p[i];
    }
  }
  return r;
}


}  // namespace mccnn
