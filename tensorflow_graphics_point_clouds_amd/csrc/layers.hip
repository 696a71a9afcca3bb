// Per-pair basis functions of the convolution layers, evaluated in registers
// from the two point coordinates of a pair:
//   Monte-Carlo convolution  pylib/pc/layers/MCConv.py:163-171, 264-269
//   kernel-point convolution pylib/pc/layers/KPConv.py:29-57, 193-213
// One lane per (pair, basis column): the K lanes of a pair read the same two
// points (broadcast loads) and write one contiguous basis row.
#include <mutex>

#include "common.h"
#include "fill.h"

namespace mccnn {

// delta = (p_in[nbr] - p_out[ctr]) * inv_radii
template <int D>
__device__ __forceinline__ void pair_delta(const float *__restrict__ pin,
                                           const float *__restrict__ pout, int2 pr,
                                           const float *ir, float *delta) {
#pragma unroll
  for (int d = 0; d < D; ++d)
    delta[d] = (pin[(int64_t)pr.x * D + d] - pout[(int64_t)pr.y * D + d]) * ir[d];
}

// weights [L, D, H]: column j = l*H + h reads weights[(l*D + d)*H + h].
template <int D>
__global__ void __launch_bounds__(256) mc_basis_kernel(
    int64_t m_total, int K, int H, int act, const float *__restrict__ pin,
    const float *__restrict__ pout, const int2 *__restrict__ nbrs,
    const float *__restrict__ inv_radii, const float *__restrict__ weights,
    const float *__restrict__ biases, const float *__restrict__ pdf, float *__restrict__ basis) {
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = inv_radii[d];
  const int64_t total = m_total * K;
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < total;
       t += (int64_t)gridDim.x * blockDim.x) {
    const int64_t m = t / K;
    const int j = (int)(t - m * K);
    const int l = j / H, h = j - l * H;
    float delta[D];
    pair_delta<D>(pin, pout, nbrs[m], ir, delta);
    float z = biases[j];
#pragma unroll
    for (int d = 0; d < D; ++d) z += delta[d] * weights[(l * D + d) * H + h];
    basis[t] = act_fwd(act, z) / pdf[m];
  }
}

constexpr int kGradBlocks = 1024;

// Each block walks a strided share of the pairs; thread (row r, column j) keeps
// D weight partials and one bias partial, reduced over the rows in LDS and
// written to partials[block][(D+1)*K].
template <int D>
__global__ void __launch_bounds__(256) mc_basis_grads_kernel(
    int64_t m_total, int K, int H, int act, const float *__restrict__ pin,
    const float *__restrict__ pout, const int2 *__restrict__ nbrs,
    const float *__restrict__ inv_radii, const float *__restrict__ weights,
    const float *__restrict__ biases, const float *__restrict__ pdf,
    const float *__restrict__ dbasis, float *__restrict__ partials) {
  __shared__ float red[256 * (D + 1)];
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = inv_radii[d];
  const int rows = 256 / K;                 // pairs handled per step by this block
  const int j = threadIdx.x % K, r = threadIdx.x / K;
  const int l = j / H, h = j - l * H;
  float w[D], dw[D], db = 0.0f;
#pragma unroll
  for (int d = 0; d < D; ++d) {
    w[d] = weights[(l * D + d) * H + h];
    dw[d] = 0.0f;
  }
  const float bj = biases[j];
  for (int64_t m = (int64_t)blockIdx.x * rows + r; m < m_total; m += (int64_t)gridDim.x * rows) {
    float delta[D];
    pair_delta<D>(pin, pout, nbrs[m], ir, delta);
    float z = bj;
#pragma unroll
    for (int d = 0; d < D; ++d) z += delta[d] * w[d];
    const float dz = dbasis[m * K + j] * act_bwd(act, z) / pdf[m];
    db += dz;
#pragma unroll
    for (int d = 0; d < D; ++d) dw[d] += delta[d] * dz;
  }
#pragma unroll
  for (int d = 0; d < D; ++d) red[d * 256 + threadIdx.x] = dw[d];
  red[D * 256 + threadIdx.x] = db;
  __syncthreads();
  if (r == 0) {
    for (int q = 0; q <= D; ++q) {
      float s = 0.0f;
      for (int rr = 0; rr < rows; ++rr) s += red[q * 256 + rr * K + j];
      partials[((int64_t)blockIdx.x * (D + 1) + q) * K + j] = s;
    }
  }
}

// weight_grads [L, D, H], bias_grads [L, H] from partials [blocks][(D+1)][K]: one
// wavefront per output, lanes stride over the blocks, fixed summation order.
__global__ void __launch_bounds__(64) mc_basis_grads_reduce_kernel(
    int blocks, int D, int K, int H, const float *__restrict__ partials,
    float *__restrict__ dweights, float *__restrict__ dbiases) {
  const int t = blockIdx.x;
  const int q = t / K, j = t - q * K;
  float s = 0.0f;
  for (int b = threadIdx.x; b < blocks; b += kWave)
    s += partials[((int64_t)b * (D + 1) + q) * K + j];
  s = wave_sum(s);
  if (threadIdx.x != 0) return;
  const int l = j / H, h = j - l * H;
  if (q < D) dweights[(l * D + q) * H + h] = s;
  else dbiases[j] = s;
}

template <int D>
__global__ void __launch_bounds__(256) kp_basis_kernel(
    int64_t m_total, int KP, int K, int kind, float sigma, const float *__restrict__ pin,
    const float *__restrict__ pout, const int2 *__restrict__ nbrs,
    const float *__restrict__ inv_radii, const float *__restrict__ kpts,
    const float *__restrict__ offsets, float *__restrict__ basis, float *__restrict__ dist_out) {
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = inv_radii[d];
  const int64_t total = m_total * K;
  for (int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; t < total;
       t += (int64_t)gridDim.x * blockDim.x) {
    const int64_t m = t / K;
    const int k = (int)(t - m * K);
    float wgt = 0.0f;
    if (k < KP) {
      const int2 pr = nbrs[m];
      float delta[D];
      pair_delta<D>(pin, pout, pr, ir, delta);
      float sq = 0.0f;
#pragma unroll
      for (int d = 0; d < D; ++d) {
        float kp = kpts[k * D + d];
        if (offsets) kp += offsets[((int64_t)pr.y * KP + k) * D + d];
        const float diff = delta[d] - kp;
        sq += diff * diff;
      }
      const float dist = sqrtf(sq);
      if (dist_out) dist_out[m * KP + k] = dist;
      if (kind == 0) {
        const float v = 1.0f - dist / sigma;
        wgt = v > 0.0f ? v : 0.0f;
      } else {
        const float q = dist / (sigma / 3.0f);
        wgt = expf(-(q * q));
      }
    }
    basis[t] = wgt;
  }
}

// d(weight)/d(distance) of the kernel-point correlation.
__device__ __forceinline__ float kp_weight_slope(int kind, float sigma, float dist) {
  if (kind == 0) return dist < sigma ? -1.0f / sigma : 0.0f;
  const float s = sigma / 3.0f, q = dist / s;
  return -2.0f * q / s * expf(-(q * q));
}

// Gradient of the kernel-point weights with respect to the per-centre offsets:
//   doff[c, k, :] = sum over the pairs m of centre c of
//                   dbasis[m, k] * w'(dist) * d(dist)/d(off),  d(dist)/d(off) = -diff / dist.
// One thread per (centre, kernel point): the pairs of a centre are contiguous,
// so the sum needs no atomics and has a fixed order.
template <int D>
__global__ void __launch_bounds__(256) kp_basis_grads_kernel(
    int64_t n_out, int KP, int K, int kind, float sigma, const float *__restrict__ pin,
    const float *__restrict__ pout, const int2 *__restrict__ nbrs, const int *__restrict__ ranges,
    const float *__restrict__ inv_radii, const float *__restrict__ kpts,
    const float *__restrict__ offsets, const float *__restrict__ dbasis,
    float *__restrict__ doffsets) {
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = inv_radii[d];
  const int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (t >= n_out * KP) return;
  const int64_t c = t / KP;
  const int k = (int)(t - c * KP);
  float kp[D], acc[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    kp[d] = kpts[k * D + d] + (offsets ? offsets[t * D + d] : 0.0f);
    acc[d] = 0.0f;
  }
  const int a = c > 0 ? ranges[c - 1] : 0, b = ranges[c];
  for (int m = a; m < b; ++m) {
    const int2 pr = nbrs[m];
    float diff[D], sq = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      diff[d] = (pin[(int64_t)pr.x * D + d] - pout[c * D + d]) * ir[d] - kp[d];
      sq += diff[d] * diff[d];
    }
    const float dist = sqrtf(sq);
    if (dist > 0.0f) {
      const float g = dbasis[(int64_t)m * K + k] * kp_weight_slope(kind, sigma, dist) / dist;
#pragma unroll
      for (int d = 0; d < D; ++d) acc[d] -= g * diff[d];
    }
  }
#pragma unroll
  for (int d = 0; d < D; ++d) doffsets[t * D + d] = acc[d];
}

// Regularisation terms of the deformable kernel points (pylib/pc/layers/KPConv.py:394-429):
//   fit[c, k]  = min over the pairs of centre c of (dist[m, k] / sigma)^2, with the pair that
//                attains it in argmin[c, k] (-1 and 0 for a centre without pairs);
//   rep[c]     = sum over k != k' of weight(|kp'_k - kp'_k'|), kp' = kernel point + offset.
template <int D>
__global__ void __launch_bounds__(256) kp_regularization_kernel(
    int64_t n_out, int KP, int kind, float sigma, const float *__restrict__ pin,
    const float *__restrict__ pout, const int2 *__restrict__ nbrs, const int *__restrict__ ranges,
    const float *__restrict__ inv_radii, const float *__restrict__ kpts,
    const float *__restrict__ offsets, float *__restrict__ fit, int *__restrict__ argmin,
    float *__restrict__ rep) {
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = inv_radii[d];
  const int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (t >= n_out * KP) return;
  const int64_t c = t / KP;
  const int k = (int)(t - c * KP);
  float kp[D];
#pragma unroll
  for (int d = 0; d < D; ++d) kp[d] = kpts[k * D + d] + offsets[t * D + d];
  const int a = c > 0 ? ranges[c - 1] : 0, b = ranges[c];
  float best = 0.0f;
  int best_m = -1;
  for (int m = a; m < b; ++m) {
    const int2 pr = nbrs[m];
    float sq = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float diff = (pin[(int64_t)pr.x * D + d] - pout[c * D + d]) * ir[d] - kp[d];
      sq += diff * diff;
    }
    if (best_m < 0 || sq < best) {
      best = sq;
      best_m = m;
    }
  }
  fit[t] = best / (sigma * sigma);
  argmin[t] = best_m;
  // repulsion of this kernel point against the others of the same centre
  float r = 0.0f;
  for (int k2 = 0; k2 < KP; ++k2) {
    if (k2 == k) continue;
    float sq = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float diff = kp[d] - (kpts[k2 * D + d] + offsets[(c * KP + k2) * D + d]);
      sq += diff * diff;
    }
    const float dist = sqrtf(sq);
    if (kind == 0) {
      const float v = 1.0f - dist / sigma;
      r += v > 0.0f ? v : 0.0f;
    } else {
      const float q = dist / (sigma / 3.0f);
      r += expf(-(q * q));
    }
  }
  rep[t] = r;
}

// The same terms for up to 16 kernel points in 2 or 3 dimensions: the 16 lanes of a quarter of a wavefront take
// one centre, lane k kernel point k.  The quarter fetches 16 pairs of its centre at a time --
// lane j pair m0 + j: index, coordinates, scaled offset to the centre -- and parks them in
// LDS; every lane then runs over the parked offsets with one broadcast LDS read per pair,
// instead of one index load and D coordinate loads per pair in each of the KP threads of a
// centre (1.34 -> 0.54 ms on 825 274 centres, 32.3 M pairs, 15 kernel points).  Same
// operations in the same order per (centre, kernel point): same bits.
template <int D>
__global__ void __launch_bounds__(256) kp_regularization16_kernel(
    int64_t n_out, int KP, int kind, float sigma, const float *__restrict__ pin,
    const float *__restrict__ pout, const int2 *__restrict__ nbrs, const int *__restrict__ ranges,
    const float *__restrict__ inv_radii, const float *__restrict__ kpts,
    const float *__restrict__ offsets, float *__restrict__ fit, int *__restrict__ argmin,
    float *__restrict__ rep) {
  static_assert(D <= 3, "a parked offset is three floats");
  __shared__ float4 stage[256];
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = inv_radii[d];
  const int k = threadIdx.x & 15;
  float4 *mine = stage + (threadIdx.x & ~15);       // the 16 slots of this quarter
  const int64_t c = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 4;
  const bool centre = c < n_out, live = centre && k < KP;
  const int64_t t = c * KP + k;
  float kp[3] = {0.0f, 0.0f, 0.0f}, ctr[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int d = 0; d < D; ++d) {
    if (live) kp[d] = kpts[k * D + d] + offsets[t * D + d];
    if (centre) ctr[d] = pout[c * D + d];
  }
  const int a = centre ? (c > 0 ? ranges[c - 1] : 0) : 0, b = centre ? ranges[c] : 0;
  float best = 0.0f;
  int best_m = -1;
  for (int m0 = a; __any(m0 < b); m0 += 16) {        // every lane of the wavefront stays in step
    const int cnt = b - m0 < 16 ? b - m0 : 16;       // <= 0 for a quarter that has finished
    if (k < cnt) {
      const int idx = nbrs[m0 + k].x;
      float dl[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int d = 0; d < D; ++d) dl[d] = (pin[(int64_t)idx * D + d] - ctr[d]) * ir[d];
      mine[k] = make_float4(dl[0], dl[1], dl[2], 0.0f);
    }
    wave_lds_sync();
    for (int j = 0; j < cnt; ++j) {
      const float4 g = mine[j];
      const float dl[3] = {g.x, g.y, g.z};
      float sq = 0.0f;
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const float diff = dl[d] - kp[d];
        sq += diff * diff;
      }
      if (best_m < 0 || sq < best) {
        best = sq;
        best_m = m0 + j;
      }
    }
    wave_lds_sync();
  }
  // repulsion of this kernel point against the others of the same centre
  mine[k] = make_float4(kp[0], kp[1], kp[2], 0.0f);
  wave_lds_sync();
  float r = 0.0f;
  for (int k2 = 0; k2 < KP; ++k2) {
    if (k2 == k) continue;
    const float4 o = mine[k2];
    const float other[3] = {o.x, o.y, o.z};
    float sq = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float diff = kp[d] - other[d];
      sq += diff * diff;
    }
    const float dist = sqrtf(sq);
    if (kind == 0) {
      const float v = 1.0f - dist / sigma;
      r += v > 0.0f ? v : 0.0f;
    } else {
      const float q = dist / (sigma / 3.0f);
      r += expf(-(q * q));
    }
  }
  if (live) {
    fit[t] = best / (sigma * sigma);
    argmin[t] = best_m;
    rep[t] = r;
  }
}

// d(scale * (sum fit + sum rep)) / d(offsets).
template <int D>
__global__ void __launch_bounds__(256) kp_regularization_grads_kernel(
    int64_t n_out, int KP, int kind, float sigma, float scale, const float *__restrict__ pin,
    const float *__restrict__ pout, const int2 *__restrict__ nbrs,
    const float *__restrict__ inv_radii, const float *__restrict__ kpts,
    const float *__restrict__ offsets, const int *__restrict__ argmin,
    float *__restrict__ doffsets) {
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = inv_radii[d];
  const int64_t t = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (t >= n_out * KP) return;
  const int64_t c = t / KP;
  const int k = (int)(t - c * KP);
  float kp[D], g[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    kp[d] = kpts[k * D + d] + offsets[t * D + d];
    g[d] = 0.0f;
  }
  const int m = argmin[t];
  if (m >= 0) {       // fit: d/d(off) of |diff|^2 / sigma^2 = -2 diff / sigma^2
    const int2 pr = nbrs[m];
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float diff = (pin[(int64_t)pr.x * D + d] - pout[c * D + d]) * ir[d] - kp[d];
      g[d] -= 2.0f * diff / (sigma * sigma);
    }
  }
  // repulsion: the pair (k, k2) appears twice in the double sum
  for (int k2 = 0; k2 < KP; ++k2) {
    if (k2 == k) continue;
    float diff[D], sq = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      diff[d] = kp[d] - (kpts[k2 * D + d] + offsets[(c * KP + k2) * D + d]);
      sq += diff[d] * diff[d];
    }
    const float dist = sqrtf(sq);
    if (dist > 0.0f) {
      const float w = 2.0f * kp_weight_slope(kind, sigma, dist) / dist;
#pragma unroll
      for (int d = 0; d < D; ++d) g[d] += w * diff[d];
    }
  }
#pragma unroll
  for (int d = 0; d < D; ++d) doffsets[t * D + d] = scale * g[d];
}

static bool valid_basis_count(int k) { return k == 8 || k == 16 || k == 32 || k == 64; }

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_mc_basis(mccnn_stream_t stream, int64_t num_neighbors, int num_dims,
                              int num_basis, int activation, const float *points_in,
                              const float *points_out, const int32_t *neighbors,
                              const float *inv_radii, const float *weights, const float *biases,
                              int num_mlps, const float *pdf, float *basis_out) {
  MCCNN_REQUIRE(valid_dims(num_dims), "mc_basis expects a valid number of dimensions");
  MCCNN_REQUIRE(valid_basis_count(num_basis), "mc_basis expects 8, 16, 32 or 64 basis functions");
  MCCNN_REQUIRE(num_mlps > 0 && num_basis % num_mlps == 0,
                "mc_basis expects the number of basis functions to be divisible by the number of "
                "kernel MLPs");
  MCCNN_REQUIRE(activation >= 0 && activation <= 2, "mc_basis expects a known activation");
  MCCNN_REQUIRE(num_neighbors >= 0, "mc_basis expects a non-negative size");
  if (num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points_in && points_out && neighbors && inv_radii && weights && biases && pdf &&
                    basis_out,
                "mc_basis received a null tensor");
  int64_t work = num_neighbors * num_basis;
  if (work > (int64_t)1 << 26) work = (int64_t)1 << 26;
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(mc_basis_kernel<D>, dim3(blocks_for(work, 256)),
                                                dim3(256), 0, as_stream(stream), num_neighbors,
                                                num_basis, num_basis / num_mlps, activation,
                                                points_in, points_out, (const int2 *)neighbors,
                                                inv_radii, weights, biases, pdf, basis_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" size_t mccnn_mc_basis_grads_workspace_bytes(int num_dims, int num_basis) {
  if (!valid_dims(num_dims) || num_basis <= 0) return 0;
  return align256(sizeof(float) * (size_t)kGradBlocks * (num_dims + 1) * num_basis);
}

// Validation and the two launches shared by mccnn_mc_basis_grads (partials in the caller's
// workspace) and mccnn_mc_basis_grads_static (partials in this library's static array).
static int mc_basis_grads_run(const char *op, mccnn_stream_t stream, int64_t num_neighbors,
                              int num_dims, int num_basis, int activation,
                              const float *points_in, const float *points_out,
                              const int32_t *neighbors, const float *inv_radii,
                              const float *weights, const float *biases, int num_mlps,
                              const float *pdf, const float *basis_grads, float *partials,
                              size_t partials_bytes, float *weight_grads_out,
                              float *bias_grads_out) {
  MCCNN_REQUIRE(valid_dims(num_dims), "%s expects a valid number of dimensions", op);
  MCCNN_REQUIRE(valid_basis_count(num_basis), "%s expects 8, 16, 32 or 64 basis functions", op);
  MCCNN_REQUIRE(num_mlps > 0 && num_basis % num_mlps == 0,
                "%s expects the number of basis functions to be divisible by the number of "
                "kernel MLPs", op);
  MCCNN_REQUIRE(activation >= 0 && activation <= 2, "%s expects a known activation", op);
  MCCNN_REQUIRE(num_neighbors >= 0, "%s expects a non-negative size", op);
  MCCNN_REQUIRE(weight_grads_out && bias_grads_out && partials, "%s received a null tensor", op);
  MCCNN_REQUIRE(partials_bytes >= mccnn_mc_basis_grads_workspace_bytes(num_dims, num_basis),
                "%s: scratch of %zu bytes is too small for %d dimensions and %d basis "
                "functions (%zu bytes needed)", op, partials_bytes, num_dims, num_basis,
                mccnn_mc_basis_grads_workspace_bytes(num_dims, num_basis));
  MCCNN_REQUIRE(num_neighbors == 0 || (points_in && points_out && neighbors && inv_radii &&
                                       weights && biases && pdf && basis_grads),
                "%s received a null tensor", op);
  hipStream_t s = as_stream(stream);
  const int rows = 256 / num_basis;
  int blocks = (int)((num_neighbors + rows - 1) / rows);
  if (blocks > kGradBlocks) blocks = kGradBlocks;
  if (blocks < 1) blocks = 1;
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(mc_basis_grads_kernel<D>, dim3(blocks), dim3(256),
                                                0, s, num_neighbors, num_basis,
                                                num_basis / num_mlps, activation, points_in,
                                                points_out, (const int2 *)neighbors, inv_radii,
                                                weights, biases, pdf, basis_grads, partials));
  MCCNN_LAUNCH_CHECK();
  const int outs = (num_dims + 1) * num_basis;
  hipLaunchKernelGGL(mc_basis_grads_reduce_kernel, dim3(outs), dim3(kWave), 0, s,
                     blocks, num_dims, num_basis, num_basis / num_mlps,
                     (const float *)partials, weight_grads_out, bias_grads_out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_mc_basis_grads(mccnn_stream_t stream, int64_t num_neighbors, int num_dims,
                                    int num_basis, int activation, const float *points_in,
                                    const float *points_out, const int32_t *neighbors,
                                    const float *inv_radii, const float *weights,
                                    const float *biases, int num_mlps, const float *pdf,
                                    const float *basis_grads, void *workspace,
                                    size_t workspace_bytes, float *weight_grads_out,
                                    float *bias_grads_out) {
  return mc_basis_grads_run("mc_basis_grads", stream, num_neighbors, num_dims, num_basis,
                            activation, points_in, points_out, neighbors, inv_radii, weights,
                            biases, num_mlps, pdf, basis_grads, (float *)workspace,
                            workspace_bytes, weight_grads_out, bias_grads_out);
}

// Per-block partial sums of mccnn_mc_basis_grads_static: the largest shape the op accepts
// (6 dimensions, 64 basis functions) times the fixed number of blocks, 1.75 MiB.  Every
// device the library runs on holds its own copy until the process ends.  Host code never
// passes the array's name to a kernel (there it is a host-side stand-in, not a device
// address): it asks the runtime once per device for the address and uses that.
constexpr size_t kStaticScratchFloats = (size_t)kGradBlocks * (kMaxDims + 1) * 64;
static __device__ __align__(256) float scratch[kStaticScratchFloats];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static float *g_scratch_ptr[kMaxDevices];      // address of `scratch` on each device

// The current device's copy of `scratch` (looked up on the first call on that device).
static int static_scratch(float **out) {
  int device = -1;
  MCCNN_HIP_CHECK(hipGetDevice(&device));
  MCCNN_REQUIRE(device >= 0 && device < kMaxDevices,
                "mc_basis_grads_static supports device ordinals below %d (got %d)", kMaxDevices,
                device);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void *address = nullptr;
    MCCNN_HIP_CHECK(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
    MCCNN_REQUIRE(address != nullptr, "mc_basis_grads_static: no address for the static scratch");
    g_scratch_ptr[device] = static_cast<float *>(address);
  }
  *out = g_scratch_ptr[device];
  return MCCNN_OK;
}

extern "C" int mccnn_mc_basis_grads_static(mccnn_stream_t stream, int64_t num_neighbors,
                                           int num_dims, int num_basis, int activation,
                                           const float *points_in, const float *points_out,
                                           const int32_t *neighbors, const float *inv_radii,
                                           const float *weights, const float *biases,
                                           int num_mlps, const float *pdf,
                                           const float *basis_grads, float *weight_grads_out,
                                           float *bias_grads_out) {
  // sizes the static array cannot hold are refused before anything is launched
  MCCNN_REQUIRE(num_dims <= kMaxDims && num_basis <= 64,
                "mc_basis_grads_static holds partial sums for at most %d dimensions and 64 basis "
                "functions (got %d and %d); use mc_basis_grads with a workspace", kMaxDims,
                num_dims, num_basis);
  float *partials = nullptr;
  int rc = static_scratch(&partials);
  if (rc != MCCNN_OK) return rc;
  // Nothing in the array has to start at zero: every block that runs overwrites its own
  // slots and the reduction reads the slots of exactly those blocks.
  return mc_basis_grads_run("mc_basis_grads_static", stream, num_neighbors, num_dims, num_basis,
                            activation, points_in, points_out, neighbors, inv_radii, weights,
                            biases, num_mlps, pdf, basis_grads, partials,
                            sizeof(float) * kStaticScratchFloats, weight_grads_out,
                            bias_grads_out);
}

extern "C" int mccnn_kp_basis(mccnn_stream_t stream, int64_t num_neighbors, int num_dims,
                              int num_kernel_points, int num_basis, int kind, float sigma,
                              const float *points_in, const float *points_out,
                              const int32_t *neighbors, const float *inv_radii,
                              const float *kernel_points, const float *offsets, float *basis_out,
                              float *dist_out) {
  MCCNN_REQUIRE(valid_dims(num_dims), "kp_basis expects a valid number of dimensions");
  MCCNN_REQUIRE(valid_basis_count(num_basis), "kp_basis expects 8, 16, 32 or 64 basis columns");
  MCCNN_REQUIRE(num_kernel_points > 0 && num_kernel_points <= num_basis,
                "kp_basis expects 1 <= kernel points <= basis columns");
  MCCNN_REQUIRE(kind == 0 || kind == 1, "kp_basis expects kind 0 (linear) or 1 (gaussian)");
  MCCNN_REQUIRE(sigma > 0.0f, "kp_basis expects a positive sigma");
  MCCNN_REQUIRE(num_neighbors >= 0, "kp_basis expects a non-negative size");
  if (num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points_in && points_out && neighbors && inv_radii && kernel_points && basis_out,
                "kp_basis received a null tensor");
  int64_t work = num_neighbors * num_basis;
  if (work > (int64_t)1 << 26) work = (int64_t)1 << 26;
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(kp_basis_kernel<D>, dim3(blocks_for(work, 256)),
                                                dim3(256), 0, as_stream(stream), num_neighbors,
                                                num_kernel_points, num_basis, kind, sigma,
                                                points_in, points_out, (const int2 *)neighbors,
                                                inv_radii, kernel_points, offsets, basis_out,
                                                dist_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

static int check_kp_args(const char *op, int num_dims, int num_kernel_points, int kind,
                         float sigma, int64_t num_samples, int64_t num_neighbors) {
  MCCNN_REQUIRE(valid_dims(num_dims), "%s expects a valid number of dimensions", op);
  MCCNN_REQUIRE(num_kernel_points > 0 && num_kernel_points <= 64,
                "%s expects between 1 and 64 kernel points", op);
  MCCNN_REQUIRE(kind == 0 || kind == 1, "%s expects kind 0 (linear) or 1 (gaussian)", op);
  MCCNN_REQUIRE(sigma > 0.0f, "%s expects a positive sigma", op);
  MCCNN_REQUIRE(num_samples >= 0 && num_neighbors >= 0, "%s expects non-negative sizes", op);
  return MCCNN_OK;
}

extern "C" int mccnn_kp_basis_grads(mccnn_stream_t stream, int64_t num_neighbors, int num_dims,
                                    int num_kernel_points, int num_basis, int kind, float sigma,
                                    const float *points_in, const float *points_out,
                                    const int32_t *neighbors, int64_t num_samples,
                                    const int32_t *ranges, const float *inv_radii,
                                    const float *kernel_points, const float *offsets,
                                    const float *basis_grads, float *offsets_grads_out) {
  int rc = check_kp_args("kp_basis_grads", num_dims, num_kernel_points, kind, sigma, num_samples,
                         num_neighbors);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(valid_basis_count(num_basis) && num_kernel_points <= num_basis,
                "kp_basis_grads expects 8, 16, 32 or 64 basis columns, at least one per kernel "
                "point");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points_out && ranges && inv_radii && kernel_points && offsets_grads_out &&
                    (num_neighbors == 0 || (points_in && neighbors && basis_grads)),
                "kp_basis_grads received a null tensor");
  const int64_t work = num_samples * num_kernel_points;
  MCCNN_DIM_SWITCH(num_dims,
                   hipLaunchKernelGGL(kp_basis_grads_kernel<D>, dim3(blocks_for(work, 256)),
                                      dim3(256), 0, as_stream(stream), num_samples,
                                      num_kernel_points, num_basis, kind, sigma, points_in,
                                      points_out, (const int2 *)neighbors, ranges, inv_radii,
                                      kernel_points, offsets, basis_grads, offsets_grads_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_kp_regularization(mccnn_stream_t stream, int64_t num_neighbors, int num_dims,
                                       int num_kernel_points, int kind, float sigma,
                                       const float *points_in, const float *points_out,
                                       const int32_t *neighbors, int64_t num_samples,
                                       const int32_t *ranges, const float *inv_radii,
                                       const float *kernel_points, const float *offsets,
                                       float *fit_out, int32_t *argmin_out, float *repulsion_out) {
  int rc = check_kp_args("kp_regularization", num_dims, num_kernel_points, kind, sigma,
                         num_samples, num_neighbors);
  if (rc != MCCNN_OK) return rc;
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points_out && ranges && inv_radii && kernel_points && offsets && fit_out &&
                    argmin_out && repulsion_out && (num_neighbors == 0 || (points_in && neighbors)),
                "kp_regularization received a null tensor");
  if (num_kernel_points <= 16 && num_dims <= 3) {
    const dim3 grid(blocks_for(num_samples * 16, 256)), block(256);
    if (num_dims == 2)
      hipLaunchKernelGGL(kp_regularization16_kernel<2>, grid, block, 0, as_stream(stream),
                         num_samples, num_kernel_points, kind, sigma, points_in, points_out,
                         (const int2 *)neighbors, ranges, inv_radii, kernel_points, offsets,
                         fit_out, argmin_out, repulsion_out);
    else
      hipLaunchKernelGGL(kp_regularization16_kernel<3>, grid, block, 0, as_stream(stream),
                         num_samples, num_kernel_points, kind, sigma, points_in, points_out,
                         (const int2 *)neighbors, ranges, inv_radii, kernel_points, offsets,
                         fit_out, argmin_out, repulsion_out);
    MCCNN_LAUNCH_CHECK();
    return MCCNN_OK;
  }
  const int64_t work = num_samples * num_kernel_points;
  MCCNN_DIM_SWITCH(num_dims,
                   hipLaunchKernelGGL(kp_regularization_kernel<D>, dim3(blocks_for(work, 256)),
                                      dim3(256), 0, as_stream(stream), num_samples,
                                      num_kernel_points, kind, sigma, points_in, points_out,
                                      (const int2 *)neighbors, ranges, inv_radii, kernel_points,
                                      offsets, fit_out, argmin_out, repulsion_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_kp_regularization_grads(mccnn_stream_t stream, int64_t num_neighbors,
                                             int num_dims, int num_kernel_points, int kind,
                                             float sigma, float loss_grad,
                                             const float *points_in, const float *points_out,
                                             const int32_t *neighbors, int64_t num_samples,
                                             const float *inv_radii, const float *kernel_points,
                                             const float *offsets, const int32_t *argmin,
                                             float *offsets_grads_out) {
  int rc = check_kp_args("kp_regularization_grads", num_dims, num_kernel_points, kind, sigma,
                         num_samples, num_neighbors);
  if (rc != MCCNN_OK) return rc;
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points_out && inv_radii && kernel_points && offsets && argmin &&
                    offsets_grads_out && (num_neighbors == 0 || (points_in && neighbors)),
                "kp_regularization_grads received a null tensor");
  const int64_t work = num_samples * num_kernel_points;
  MCCNN_DIM_SWITCH(num_dims, hipLaunchKernelGGL(kp_regularization_grads_kernel<D>,
                                                dim3(blocks_for(work, 256)), dim3(256), 0,
                                                as_stream(stream), num_samples, num_kernel_points,
                                                kind, sigma, loss_grad, points_in, points_out,
                                                (const int2 *)neighbors, inv_radii, kernel_points,
                                                offsets, argmin, offsets_grads_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
