// Shared host/device helpers of libmccnn_hip.so (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/mccnn_hip.h"

namespace mccnn {

constexpr int kWave = 64;
constexpr int kMaxDims = MCCNN_MAX_DIMENSIONS;

// Records the message returned by mccnn_last_error() for the calling thread.
void set_error(const char *fmt, ...);

inline hipStream_t as_stream(mccnn_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

#define MCCNN_REQUIRE(cond, ...)            \
  do {                                      \
    if (!(cond)) {                          \
      ::mccnn::set_error(__VA_ARGS__);      \
      return MCCNN_INVALID_ARGUMENT;        \
    }                                       \
  } while (0)

#define MCCNN_HIP_CHECK(expr)                                                   \
  do {                                                                          \
    hipError_t err_ = (expr);                                                   \
    if (err_ != hipSuccess) {                                                   \
      ::mccnn::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(err_), \
                         __FILE__, __LINE__);                                   \
      return MCCNN_HIP_ERROR;                                                   \
    }                                                                           \
  } while (0)

#define MCCNN_LAUNCH_CHECK() MCCNN_HIP_CHECK(hipGetLastError())

// Dispatch on the point dimension (2..6), the template parameter of most kernels.
#define MCCNN_DIM_SWITCH(D_, ...)                              \
  switch (D_) {                                                \
    case 2: { constexpr int D = 2; __VA_ARGS__; } break;       \
    case 3: { constexpr int D = 3; __VA_ARGS__; } break;       \
    case 4: { constexpr int D = 4; __VA_ARGS__; } break;       \
    case 5: { constexpr int D = 5; __VA_ARGS__; } break;       \
    case 6: { constexpr int D = 6; __VA_ARGS__; } break;       \
  }

inline bool valid_dims(int d) { return d >= MCCNN_MIN_DIMENSIONS && d <= MCCNN_MAX_DIMENSIONS; }

inline unsigned blocks_for(int64_t work, int block) {
  int64_t b = (work + block - 1) / block;
  return (unsigned)(b < 1 ? 1 : b);
}

// Round a byte count up to a 256-byte boundary (workspace carving).
inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

#ifdef __HIPCC__

template <int D>
struct GridShape {
  int n[D];
};

template <int D>
__device__ __forceinline__ GridShape<D> load_shape(const int *__restrict__ num_cells) {
  GridShape<D> g;
#pragma unroll
  for (int d = 0; d < D; ++d) g.n[d] = num_cells[d];
  return g;
}

template <int D>
__device__ __forceinline__ int64_t total_cells(const GridShape<D> &g) {
  int64_t t = 1;
#pragma unroll
  for (int d = 0; d < D; ++d) t *= g.n[d];
  return t;
}

// Row-major key of a cell with the batch id as the most significant digit.
template <int D>
__device__ __forceinline__ int64_t key_of_cell(const int *cell, const GridShape<D> &g, int b) {
  int64_t key = 0, accum = 1;
#pragma unroll
  for (int d = D - 1; d >= 0; --d) {
    key += (int64_t)cell[d] * accum;
    accum *= g.n[d];
  }
  return key + accum * (int64_t)b;
}

// cell = clamp(floor(p * inv_cell - smin), 0, n-1), each float op rounded once.
// Files that call this are compiled with -ffp-contract=off.
template <int D>
__device__ __forceinline__ void cell_of_point(const float *p, const float *smin,
                                              const float *inv_cell, const GridShape<D> &g,
                                              int *cell) {
#pragma unroll
  for (int d = 0; d < D; ++d) {
    float prod = p[d] * inv_cell[d];
    float rel = prod - smin[d];
    int c = (int)floorf(rel);
    c = c < 0 ? 0 : c;
    c = c > g.n[d] - 1 ? g.n[d] - 1 : c;
    cell[d] = c;
  }
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Orders the LDS traffic of one wavefront: what any lane wrote before the call
// is what every lane reads after it.  The hardware already serves the LDS
// accesses of a wavefront in program order; the call keeps the compiler from
// moving (or duplicating into divergent branches) loads and stores across it.
// Every lane of the wavefront must reach it.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Barrier of the block that orders its LDS traffic only: what any thread wrote to LDS
// before the call is what every thread reads after it.  Unlike __syncthreads() it does not
// wait for the wavefront's outstanding global loads and stores (a prefetch in flight,
// streamed stores whose acknowledgement takes microseconds).  Every thread must reach it.
__device__ __forceinline__ void block_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Inclusive prefix sum across the 64 lanes of a wave.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  const int lane = lane_id();
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    int t = __shfl_up(v, off, kWave);
    if (lane >= off) v += t;
  }
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// Activations of the kernel MLP (pylib/pc/layers/MCConv.py:27-31; leaky slope
// 0.2 and ELU alpha 1 are the TensorFlow defaults the reference relies on).
__device__ __forceinline__ float act_fwd(int act, float z) {
  if (act == MCCNN_ACT_RELU) return z > 0.0f ? z : 0.0f;
  if (act == MCCNN_ACT_LEAKY_RELU) return z > 0.0f ? z : 0.2f * z;
  return z > 0.0f ? z : expm1f(z);
}

__device__ __forceinline__ float act_bwd(int act, float z) {
  if (act == MCCNN_ACT_RELU) return z > 0.0f ? 1.0f : 0.0f;
  if (act == MCCNN_ACT_LEAKY_RELU) return z > 0.0f ? 1.0f : 0.2f;
  return z > 0.0f ? 1.0f : expf(z);
}

#endif  // __HIPCC__

}  // namespace mccnn
