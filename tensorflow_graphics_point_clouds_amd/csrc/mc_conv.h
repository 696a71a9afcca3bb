// Kernel-MLP parameters shared by the fused Monte-Carlo convolution kernels.
#pragma once
#include "common.h"
#include "mfma.h"

namespace mccnn {

constexpr int kFusedUnroll = 4;
constexpr int kFusedK = 16;

template <int D>
struct McParams {
  const float *pin;        // [N_in, D]
  const float *pout;       // [N_out, D]
  const float *inv_radii;  // [D]
  const float *weights;    // [L, D, H]
  const float *biases;     // [L*H]
  const float *pdf;        // [M]
  int hidden;              // H
  int act;
};

// Weight column j of the flattened [D, L*H] kernel matrix.
template <int D>
__device__ __forceinline__ void load_weight_column(const McParams<D> &p, int j, float *w,
                                                   float *bias) {
  const int l = j / p.hidden, h = j - l * p.hidden;
#pragma unroll
  for (int d = 0; d < D; ++d) w[d] = p.weights[(l * D + d) * p.hidden + h];
  *bias = p.biases[j];
}

// Per-wavefront LDS staging of one chunk of 64 pairs: lane n prepares pair n once
// (offset to the neighbour, 1/pdf, neighbour feature row), and every matrix-core
// step then fetches the four pairs it needs with two broadcast LDS reads instead
// of recomputing them in each of the 16 lanes of a quarter.
struct PairStage {
  float4 geo[kWave];      // delta * inv_radii in x, y, z (z = 0 for D = 2), 1 / pdf in w
  unsigned row[kWave];    // byte offset of the neighbour's feature row
  int aux[kWave];         // row of a per-centre side table (deformable kernel points)
};

// The activation is a template parameter of the fused kernels: with a run-time
// selector the compiler evaluates all three (including the exponential of ELU)
// for every pair and selects afterwards.
#define MCCNN_ACT_SWITCH(act_, ...)                                   \
  switch (act_) {                                                     \
    case MCCNN_ACT_RELU: { constexpr int ACT = MCCNN_ACT_RELU; __VA_ARGS__; } break;             \
    case MCCNN_ACT_LEAKY_RELU: { constexpr int ACT = MCCNN_ACT_LEAKY_RELU; __VA_ARGS__; } break; \
    default: { constexpr int ACT = MCCNN_ACT_ELU; __VA_ARGS__; } break;                          \
  }

// Per-lane basis functors: the value of basis column `col + 16 kt` (col = lane & 15)
// for a staged pair g = (delta * inv_radii, weight), weight = 1/pdf or 1 for a
// live pair and 0 for a padding slot.
template <int D, int kAct, int KT = 1>
struct MlpBasis {                  // act(delta . W[:, col] + b[col]) / pdf   (MCConv.py:163-171)
  float w[KT][3], b[KT];           // columns col, col + 16, ... of the flattened kernel matrix
  __device__ __forceinline__ MlpBasis(const McParams<D> &p) {
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      w[kt][0] = w[kt][1] = w[kt][2] = 0.0f;
      load_weight_column<D>(p, 16 * kt + (lane_id() & 15), w[kt], &b[kt]);
    }
  }
  static constexpr bool kUsesAux = false;
  __device__ __forceinline__ float operator()(const float4 &g, int kt = 0, int = 0) const {
    const float z = b[kt] + g.x * w[kt][0] + g.y * w[kt][1] + g.z * w[kt][2];
    return act_fwd(kAct, z) * g.w;
  }
};

template <int D, int kKind, int KT = 1>
struct KpBasis {                   // kernel-point correlation (KPConv.py:29-57, 193-213)
  float k[KT][3], sigma;
  bool live[KT];                   // columns past the last kernel point are zero padding
  __device__ __forceinline__ KpBasis(const float *__restrict__ kernel_points, int num_kp,
                                     float sigma_) : sigma(sigma_) {
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      const int col = 16 * kt + (lane_id() & 15);
      live[kt] = col < num_kp;
      k[kt][0] = k[kt][1] = k[kt][2] = 0.0f;
#pragma unroll
      for (int d = 0; d < D; ++d) k[kt][d] = live[kt] ? kernel_points[col * D + d] : 0.0f;
    }
  }
  static constexpr bool kUsesAux = false;
  __device__ __forceinline__ float operator()(const float4 &g, int kt = 0, int = 0) const {
    const float dx = g.x - k[kt][0], dy = g.y - k[kt][1], dz = g.z - k[kt][2];
    const float dist = sqrtf(dx * dx + dy * dy + dz * dz);
    float wgt;
    if (kKind == 0) {
      const float v = 1.0f - dist / sigma;
      wgt = v > 0.0f ? v : 0.0f;
    } else {
      const float q = dist / (sigma / 3.0f);
      wgt = expf(-(q * q));
    }
    return live[kt] ? wgt * g.w : 0.0f;
  }
};

// Correlation weight of the kernel-point convolution for a distance.
template <int kKind>
__device__ __forceinline__ float kp_weight(float dist, float sigma) {
  if (kKind == 0) {
    const float v = 1.0f - dist / sigma;
    return v > 0.0f ? v : 0.0f;
  }
  const float q = dist / (sigma / 3.0f);
  return expf(-(q * q));
}

// Deformable kernel points (KPConv.py:317-392): kernel point `col` of the centre of a
// pair is shifted by offsets[row, col, :], where `row` (the staged aux value) is the
// centre's row in the [N_centres, num_kp, D] offset table.  Up to 16 kernel points.
template <int D, int kKind>
struct KpDeformBasis {
  float k[3], sigma;
  const float *off;                // offsets + col * D, or null for a padding column
  int stride;                      // num_kp * D
  __device__ __forceinline__ KpDeformBasis(const float *__restrict__ kernel_points, int num_kp,
                                           float sigma_, const float *__restrict__ offsets)
      : sigma(sigma_), stride(num_kp * D) {
    const int col = lane_id() & 15;
    const bool live = col < num_kp;
    k[0] = k[1] = k[2] = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) k[d] = live ? kernel_points[col * D + d] : 0.0f;
    off = live ? offsets + col * D : nullptr;
  }
  static constexpr bool kUsesAux = true;
  __device__ __forceinline__ float operator()(const float4 &g, int, int aux) const {
    if (off == nullptr) return 0.0f;
    const float *o = off + (int64_t)aux * stride;
    float diff[3] = {g.x - k[0], g.y - k[1], g.z - k[2]};
    float sq = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      diff[d] -= o[d];
      sq += diff[d] * diff[d];
    }
    return kp_weight<kKind>(sqrtf(sq), sigma) * g.w;
  }
};

// acc[j] += projection of the pairs [a, b) of one centre for the channels
// col*kCPL + j (kStrided: col + 16*j) of the 16*kCPL-channel chunk starting at
// feat_base.  Rows are row_bytes apart; every byte offset fits 32 bits (checked by
// the host).  p.pdf may be null (weight 1).
template <int kCPL, int D, class Basis, bool kStrided = false>
__device__ __forceinline__ void project_pairs(const char *__restrict__ feat_base,
                                              unsigned row_bytes, const int2 *__restrict__ nbrs,
                                              int a, int b, const McParams<D> &p,
                                              const float *ctr, PairStage *stage,
                                              const Basis &basis, v4f *acc) {
  const int lane = lane_id(), quarter = lane >> 4, col = lane & 15;
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = p.inv_radii[d];
  const unsigned lane_off = kStrided ? col * 4 : col * kCPL * 4;
  for (int m0 = a; m0 < b; m0 += kWave) {
    const int cnt = b - m0 < kWave ? b - m0 : kWave;
    float4 g = {0.0f, 0.0f, 0.0f, 0.0f};
    unsigned row = 0;
    if (lane < cnt) {
      const int idx = nbrs[m0 + lane].x;
      float dl[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int d = 0; d < D; ++d) dl[d] = (p.pin[(int64_t)idx * D + d] - ctr[d]) * ir[d];
      g = make_float4(dl[0], dl[1], dl[2], p.pdf ? 1.0f / p.pdf[m0 + lane] : 1.0f);
      row = (unsigned)idx * row_bytes;
    }
    // unused slots of the last step point at the first pair's row with weight 0
    const unsigned row0 = __builtin_amdgcn_readfirstlane(row);
    stage->geo[lane] = g;
    stage->row[lane] = lane < cnt ? row : row0;
    wave_lds_sync();
    // Steps of 4 pairs, taken kFusedUnroll at a time without a branch: the slots
    // past the last pair hold weight 0 and a valid row, so the steps that round the
    // count up add exact zeros.
    const int steps = (cnt + 3) >> 2;
    for (int t = 0; t < steps; t += kFusedUnroll) {
      FVec<kCPL> f[kFusedUnroll];
      float w[kFusedUnroll];
#pragma unroll
      for (int u = 0; u < kFusedUnroll; ++u) {
        const int n = 4 * (t + u) + quarter;
        const float4 gn = stage->geo[n];
        const unsigned rn = stage->row[n];
        if constexpr (kStrided) {
#pragma unroll
          for (int j = 0; j < kCPL; ++j)
            f[u].v[j] = *reinterpret_cast<const float *>(feat_base + (size_t)(rn + lane_off) + j * 64);
        } else {
          f[u] = load_vec<kCPL>(reinterpret_cast<const float *>(feat_base + (size_t)(rn + lane_off)), true);
        }
        w[u] = basis(gn);
      }
#pragma unroll
      for (int u = 0; u < kFusedUnroll; ++u)
#pragma unroll
        for (int j = 0; j < kCPL; ++j)
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u], f[u].v[j], acc[j], 0, 0, 0);
    }
    wave_lds_sync();                        // the stage is free for the next chunk
  }
}

}  // namespace mccnn
