// Per-pair density transform of PointConv (pylib/pc/layers/PointConv.py:176-190):
//   rel[m] = pdf[point of pair m] / max_pdf[centre of pair m]
//   y[m]   = b2 + sum_j w2[j] * relu(rel[m] * w1[j] + b1[j]),   j < 16
// y takes the place of the density in the Monte-Carlo projection kernels (they
// scale the basis by 1 / y), so the [M, 16] hidden layer the reference writes with
// TensorFlow ops never exists.  The second kernel turns the gradient with respect
// to the pairs' scale 1 / y into the gradients of the 49 parameters.
#include "common.h"
#include "fill.h"

namespace mccnn {

constexpr int kPdfHidden = 16;                     // PointConv.py:118-141
constexpr int kPdfParams = 3 * kPdfHidden + 1;     // w1, b1, w2, b2
constexpr int kDensityThreads = 256;

struct DensityMlp {
  float w1[kPdfHidden], b1[kPdfHidden], w2[kPdfHidden], b2;
};

__device__ __forceinline__ DensityMlp load_density_mlp(const float *__restrict__ w1,
                                                       const float *__restrict__ b1,
                                                       const float *__restrict__ w2,
                                                       const float *__restrict__ b2) {
  DensityMlp p;
#pragma unroll
  for (int j = 0; j < kPdfHidden; ++j) {
    p.w1[j] = w1[j];
    p.b1[j] = b1[j];
    p.w2[j] = w2[j];
  }
  p.b2 = b2[0];
  return p;
}

// pairs[m][point_column] indexes pdf, the other column max_pdf.
__device__ __forceinline__ float relative_density(const int2 pair, int point_column,
                                                  const float *__restrict__ pdf,
                                                  const float *__restrict__ max_pdf) {
  const int pt = point_column == 0 ? pair.x : pair.y;
  const int ctr = point_column == 0 ? pair.y : pair.x;
  return pdf[pt] / max_pdf[ctr];
}

__global__ void __launch_bounds__(kDensityThreads) pointconv_density_kernel(
    int64_t m, const int2 *__restrict__ pairs, int point_column, const float *__restrict__ pdf,
    const float *__restrict__ max_pdf, const float *__restrict__ w1, const float *__restrict__ b1,
    const float *__restrict__ w2, const float *__restrict__ b2, float *__restrict__ out) {
  const DensityMlp p = load_density_mlp(w1, b1, w2, b2);
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < m;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float rel = relative_density(pairs[i], point_column, pdf, max_pdf);
    float y = p.b2;
#pragma unroll
    for (int j = 0; j < kPdfHidden; ++j) {
      const float u = rel * p.w1[j] + p.b1[j];
      y += p.w2[j] * (u > 0.0f ? u : 0.0f);
    }
    out[i] = y;
  }
}

// partials [blocks][49]: per block the sums over its pairs of
//   gy * d y / d theta,  gy = -(sum over slabs of scale_grads) / y^2,
// ordered w1[16], b1[16], w2[16], b2.
__global__ void __launch_bounds__(kDensityThreads) pointconv_density_grads_kernel(
    int64_t m, const int2 *__restrict__ pairs, int point_column, const float *__restrict__ pdf,
    const float *__restrict__ max_pdf, const float *__restrict__ w1, const float *__restrict__ b1,
    const float *__restrict__ w2, const float *__restrict__ b2, const float *__restrict__ y,
    int slabs, const float *__restrict__ scale_grads, float *__restrict__ partials) {
  __shared__ float red[kDensityThreads / kWave][kPdfParams];
  const DensityMlp p = load_density_mlp(w1, b1, w2, b2);
  float g[kPdfParams];
#pragma unroll
  for (int j = 0; j < kPdfParams; ++j) g[j] = 0.0f;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < m;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float rel = relative_density(pairs[i], point_column, pdf, max_pdf);
    float t = 0.0f;
    for (int s = 0; s < slabs; ++s) t += scale_grads[(int64_t)s * m + i];
    const float yi = y[i];
    const float gy = -t / (yi * yi);
#pragma unroll
    for (int j = 0; j < kPdfHidden; ++j) {
      const float u = rel * p.w1[j] + p.b1[j];
      const float live = u > 0.0f ? gy : 0.0f;
      g[j] += live * p.w2[j] * rel;
      g[kPdfHidden + j] += live * p.w2[j];
      g[2 * kPdfHidden + j] += u > 0.0f ? gy * u : 0.0f;
    }
    g[3 * kPdfHidden] += gy;
  }
  const int lane = lane_id(), wave = threadIdx.x / kWave;
#pragma unroll
  for (int j = 0; j < kPdfParams; ++j) {
    const float s = wave_sum(g[j]);
    if (lane == 0) red[wave][j] = s;
  }
  __syncthreads();
  if (threadIdx.x < kPdfParams) {
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < kDensityThreads / kWave; ++w) s += red[w][threadIdx.x];
    partials[(int64_t)blockIdx.x * kPdfParams + threadIdx.x] = s;
  }
}

__global__ void __launch_bounds__(kDensityThreads) pointconv_density_reduce_kernel(
    int blocks, const float *__restrict__ partials, float *__restrict__ out) {
  __shared__ float red[kDensityThreads / kWave];
  const int j = blockIdx.x;
  float s = 0.0f;
  for (int b = threadIdx.x; b < blocks; b += kDensityThreads) s += partials[b * kPdfParams + j];
  s = wave_sum(s);
  if (lane_id() == 0) red[threadIdx.x / kWave] = s;
  __syncthreads();
  if (threadIdx.x != 0) return;
  s = 0.0f;
#pragma unroll
  for (int w = 0; w < kDensityThreads / kWave; ++w) s += red[w];
  out[j] = s;
}

static unsigned density_blocks(int64_t m) {
  const int64_t b = (m + kDensityThreads * 8 - 1) / (kDensityThreads * 8);
  return (unsigned)(b < 1 ? 1 : b > 2048 ? 2048 : b);
}

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_pointconv_density(mccnn_stream_t stream, int64_t num_neighbors,
                                       const int32_t *neighbors, int point_column,
                                       const float *pdf, const float *max_pdf,
                                       const float *weights_1, const float *biases_1,
                                       const float *weights_2, const float *biases_2,
                                       float *density_out) {
  MCCNN_REQUIRE(num_neighbors >= 0 && num_neighbors < ((int64_t)1 << 31),
                "pointconv_density expects a pair count in [0, 2^31)");
  MCCNN_REQUIRE(point_column == 0 || point_column == 1,
                "pointconv_density expects point_column 0 or 1");
  if (num_neighbors == 0) return MCCNN_OK;
  MCCNN_REQUIRE(neighbors && pdf && max_pdf && weights_1 && biases_1 && weights_2 && biases_2 &&
                    density_out,
                "pointconv_density received a null tensor");
  hipLaunchKernelGGL(pointconv_density_kernel, dim3(density_blocks(num_neighbors)),
                     dim3(kDensityThreads), 0, as_stream(stream), num_neighbors,
                     (const int2 *)neighbors, point_column, pdf, max_pdf, weights_1, biases_1,
                     weights_2, biases_2, density_out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" size_t mccnn_pointconv_density_grads_workspace_bytes(int64_t num_neighbors) {
  if (num_neighbors < 0) num_neighbors = 0;
  return align256(sizeof(float) * (size_t)density_blocks(num_neighbors) * kPdfParams);
}

extern "C" int mccnn_pointconv_density_grads(
    mccnn_stream_t stream, int64_t num_neighbors, const int32_t *neighbors, int point_column,
    const float *pdf, const float *max_pdf, const float *weights_1, const float *biases_1,
    const float *weights_2, const float *biases_2, const float *density, int num_slabs,
    const float *pair_scale_grads, void *workspace, size_t workspace_bytes,
    float *param_grads_out) {
  MCCNN_REQUIRE(num_neighbors >= 0 && num_neighbors < ((int64_t)1 << 31),
                "pointconv_density_grads expects a pair count in [0, 2^31)");
  MCCNN_REQUIRE(point_column == 0 || point_column == 1,
                "pointconv_density_grads expects point_column 0 or 1");
  MCCNN_REQUIRE(num_slabs >= 1 && num_slabs <= 4,
                "pointconv_density_grads expects 1 to 4 slabs of scale gradients");
  MCCNN_REQUIRE(param_grads_out && workspace, "pointconv_density_grads received a null output");
  MCCNN_REQUIRE(workspace_bytes >= mccnn_pointconv_density_grads_workspace_bytes(num_neighbors),
                "pointconv_density_grads workspace too small");
  hipStream_t s = as_stream(stream);
  if (num_neighbors == 0)
    return fill_zero(s, param_grads_out, sizeof(float) * kPdfParams);
  MCCNN_REQUIRE(neighbors && pdf && max_pdf && weights_1 && biases_1 && weights_2 && biases_2 &&
                    density && pair_scale_grads,
                "pointconv_density_grads received a null tensor");
  const unsigned blocks = density_blocks(num_neighbors);
  hipLaunchKernelGGL(pointconv_density_grads_kernel, dim3(blocks), dim3(kDensityThreads), 0, s,
                     num_neighbors, (const int2 *)neighbors, point_column, pdf, max_pdf,
                     weights_1, biases_1, weights_2, biases_2, density, num_slabs,
                     pair_scale_grads, (float *)workspace);
  MCCNN_LAUNCH_CHECK();
  hipLaunchKernelGGL(pointconv_density_reduce_kernel, dim3(kPdfParams), dim3(kDensityThreads), 0,
                     s, (int)blocks, (const float *)workspace, param_grads_out);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
