// One layer of a kernel MLP evaluated per neighbour pair (pylib/pc/layers/MCConv.py:163-168,
// PointConv.py:168-190): y[m, :] = act(x[m, :] * W + b) for x [M, I] with M in the tens of
// millions and I, O <= 64, and its gradients.  Memory-bound: every kernel reads or writes
// the per-pair tensors once; the weights sit in LDS.  Used for kernel MLPs with more than
// one layer and wherever the kernel input must stay differentiable (gradients with respect
// to point coordinates), where the [M, K] basis is materialised as in the reference.
#include "common.h"
#include "fill.h"

namespace mccnn {

constexpr int kPairDenseMax = 64;        // largest layer width
constexpr int kPairDenseRows = 32;       // rows per LDS tile of the weight-gradient kernel

// activation codes of this file: -1 identity, otherwise MCCNN_ACT_*
__device__ __forceinline__ float pd_act(int act, float z) { return act < 0 ? z : act_fwd(act, z); }

// derivative of the activation from its OUTPUT y = act(z) (all three are invertible in sign:
// relu / leaky relu keep the sign of z, ELU gives y + 1 = exp(z) for z <= 0)
__device__ __forceinline__ float pd_slope(int act, float y) {
  if (act < 0) return 1.0f;
  if (act == MCCNN_ACT_RELU) return y > 0.0f ? 1.0f : 0.0f;
  if (act == MCCNN_ACT_LEAKY_RELU) return y > 0.0f ? 1.0f : 0.2f;
  return y > 0.0f ? 1.0f : y + 1.0f;
}

// thread per (row, output column)
__global__ void __launch_bounds__(256) pair_dense_kernel(int64_t rows, int I, int O,
                                                         const float *__restrict__ x,
                                                         const float *__restrict__ w,
                                                         const float *__restrict__ b, int act,
                                                         float *__restrict__ y) {
  __shared__ float wl[kPairDenseMax * kPairDenseMax + kPairDenseMax];
  for (int e = threadIdx.x; e < I * O; e += blockDim.x) wl[e] = w[e];
  for (int e = threadIdx.x; e < O; e += blockDim.x) wl[I * O + e] = b ? b[e] : 0.0f;
  __syncthreads();
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows * O) return;
  const int64_t m = t / O;
  const int o = (int)(t - m * O);
  const float *xr = x + m * I;
  float z = wl[I * O + o];
  for (int i = 0; i < I; ++i) z += xr[i] * wl[i * O + o];
  y[t] = pd_act(act, z);
}

// dx[m, i] = sum_o dy[m, o] act'(y[m, o]) W[i, o]: thread per (row, input column)
__global__ void __launch_bounds__(256) pair_dense_dx_kernel(int64_t rows, int I, int O,
                                                            const float *__restrict__ w,
                                                            const float *__restrict__ y,
                                                            const float *__restrict__ dy, int act,
                                                            float *__restrict__ dx) {
  __shared__ float wl[kPairDenseMax * kPairDenseMax];
  for (int e = threadIdx.x; e < I * O; e += blockDim.x) wl[e] = w[e];
  __syncthreads();
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= rows * I) return;
  const int64_t m = t / I;
  const int i = (int)(t - m * I);
  const float *yr = y + m * O, *dr = dy + m * O;
  float s = 0.0f;
  for (int o = 0; o < O; ++o) s += dr[o] * pd_slope(act, yr[o]) * wl[i * O + o];
  dx[t] = s;
}

// Per-slice partial sums of dW[i, o] = sum_m x[m, i] dz[m, o] and db[o] = sum_m dz[m, o],
// dz = dy * act'(y): a block walks its slice of the rows in tiles of 32 (x and dz staged in
// LDS), every thread owns kEPT of the I * O + O sums in registers.  The partial sums are
// added over the slices in a fixed order afterwards: bit-reproducible.
template <int kEPT>
__global__ void __launch_bounds__(256) pair_dense_dw_kernel(int64_t rows, int I, int O,
                                                            const float *__restrict__ x,
                                                            const float *__restrict__ y,
                                                            const float *__restrict__ dy, int act,
                                                            int slices,
                                                            float *__restrict__ partials) {
  __shared__ float xs[kPairDenseRows][kPairDenseMax + 1];
  __shared__ float zs[kPairDenseRows][kPairDenseMax + 1];
  const int t = threadIdx.x, elems = I * O + O;
  const int64_t tiles_total = (rows + kPairDenseRows - 1) / kPairDenseRows;
  const int64_t per = (tiles_total + slices - 1) / slices;
  const int64_t t0 = blockIdx.x * per;
  const int64_t t1 = t0 + per < tiles_total ? t0 + per : tiles_total;
  int ei[kEPT], eo[kEPT];          // element -> (input column or -1 for the bias, output column)
  float acc[kEPT];
#pragma unroll
  for (int u = 0; u < kEPT; ++u) {
    const int e = t + 256 * u;
    acc[u] = 0.0f;
    if (e < I * O) {
      ei[u] = e / O;
      eo[u] = e - ei[u] * O;
    } else {
      ei[u] = -1;
      eo[u] = e < elems ? e - I * O : -1;
    }
  }
  for (int64_t tile = t0; tile < t1; ++tile) {
    const int64_t m0 = tile * kPairDenseRows;
    __syncthreads();
    for (int e = t; e < kPairDenseRows * I; e += 256) {
      const int r = e / I, i = e - r * I;
      xs[r][i] = m0 + r < rows ? x[(m0 + r) * I + i] : 0.0f;
    }
    for (int e = t; e < kPairDenseRows * O; e += 256) {
      const int r = e / O, o = e - r * O;
      const int64_t at = (m0 + r) * O + o;
      zs[r][o] = m0 + r < rows ? dy[at] * pd_slope(act, y[at]) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kEPT; ++u) {
      if (eo[u] < 0) continue;
      float s = acc[u];
      if (ei[u] >= 0) {
#pragma unroll 8
        for (int r = 0; r < kPairDenseRows; ++r) s += xs[r][ei[u]] * zs[r][eo[u]];
      } else {
#pragma unroll 8
        for (int r = 0; r < kPairDenseRows; ++r) s += zs[r][eo[u]];
      }
      acc[u] = s;
    }
  }
#pragma unroll
  for (int u = 0; u < kEPT; ++u) {
    const int e = t + 256 * u;
    if (e < elems) partials[(int64_t)blockIdx.x * elems + e] = acc[u];
  }
}

__global__ void __launch_bounds__(256) pair_dense_reduce_kernel(int elems, int split, int slices,
                                                                const float *__restrict__ partials,
                                                                float *__restrict__ dw,
                                                                float *__restrict__ db) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= elems) return;
  float s = 0.0f;
  for (int k = 0; k < slices; ++k) s += partials[(int64_t)k * elems + e];
  if (e < split) dw[e] = s;
  else if (db) db[e - split] = s;
}

static int pair_dense_slices(int64_t rows) {
  const int64_t by_size = (rows + 4 * kPairDenseRows - 1) / (4 * kPairDenseRows);
  return (int)(by_size < 1 ? 1 : by_size > 1024 ? 1024 : by_size);
}

static bool pair_dense_shape_ok(int I, int O) {
  return I >= 1 && I <= kPairDenseMax && O >= 1 && O <= kPairDenseMax;
}

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_pair_dense(mccnn_stream_t stream, int64_t num_rows, int num_cols_in,
                                const float *x, int num_cols_out, const float *weights,
                                const float *biases, int activation, float *y) {
  MCCNN_REQUIRE(pair_dense_shape_ok(num_cols_in, num_cols_out),
                "pair_dense supports 1..64 input and output columns (got %d -> %d)", num_cols_in,
                num_cols_out);
  MCCNN_REQUIRE(activation >= -1 && activation <= 2,
                "pair_dense expects activation -1 (none), 0 (relu), 1 (leaky relu) or 2 (elu)");
  MCCNN_REQUIRE(num_rows >= 0 && num_rows * num_cols_out < ((int64_t)1 << 40) &&
                    num_rows * num_cols_in < ((int64_t)1 << 40),
                "pair_dense expects a non-negative row count");
  if (num_rows == 0) return MCCNN_OK;
  MCCNN_REQUIRE(x && weights && y, "pair_dense received a null tensor");
  hipLaunchKernelGGL(pair_dense_kernel, dim3(blocks_for(num_rows * num_cols_out, 256)), dim3(256),
                     0, as_stream(stream), num_rows, num_cols_in, num_cols_out, x, weights, biases,
                     activation, y);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" size_t mccnn_pair_dense_grads_workspace_bytes(int64_t num_rows, int num_cols_in,
                                                         int num_cols_out) {
  if (!pair_dense_shape_ok(num_cols_in, num_cols_out) || num_rows < 0) return 0;
  return align256(sizeof(float) * (size_t)pair_dense_slices(num_rows) *
                  ((size_t)num_cols_in * num_cols_out + num_cols_out));
}

extern "C" int mccnn_pair_dense_grads(mccnn_stream_t stream, int64_t num_rows, int num_cols_in,
                                      const float *x, int num_cols_out, const float *weights,
                                      const float *y, const float *dy, int activation,
                                      void *workspace, size_t workspace_bytes, float *dx,
                                      float *dweights, float *dbiases) {
  MCCNN_REQUIRE(pair_dense_shape_ok(num_cols_in, num_cols_out),
                "pair_dense_grads supports 1..64 input and output columns (got %d -> %d)",
                num_cols_in, num_cols_out);
  MCCNN_REQUIRE(activation >= -1 && activation <= 2,
                "pair_dense_grads expects activation -1 (none), 0 (relu), 1 (leaky relu) or 2 (elu)");
  MCCNN_REQUIRE(num_rows >= 0, "pair_dense_grads expects a non-negative row count");
  MCCNN_REQUIRE(dweights, "pair_dense_grads received a null tensor");
  const int I = num_cols_in, O = num_cols_out, elems = I * O + O;
  hipStream_t s = as_stream(stream);
  if (num_rows == 0) {
    int rc = fill_zero(s, dweights, sizeof(float) * (size_t)I * O);
    if (rc == MCCNN_OK && dbiases) rc = fill_zero(s, dbiases, sizeof(float) * (size_t)O);
    return rc;
  }
  MCCNN_REQUIRE(x && weights && y && dy && workspace, "pair_dense_grads received a null tensor");
  MCCNN_REQUIRE(workspace_bytes >= mccnn_pair_dense_grads_workspace_bytes(num_rows, I, O),
                "pair_dense_grads workspace too small");
  if (dx) {
    hipLaunchKernelGGL(pair_dense_dx_kernel, dim3(blocks_for(num_rows * I, 256)), dim3(256), 0, s,
                       num_rows, I, O, weights, y, dy, activation, dx);
    MCCNN_LAUNCH_CHECK();
  }
  const int slices = pair_dense_slices(num_rows);
  float *partials = (float *)workspace;
  const int ept = (elems + 255) / 256;
#define MCCNN_PD_LAUNCH(E_)                                                                     \
  hipLaunchKernelGGL(pair_dense_dw_kernel<E_>, dim3(slices), dim3(256), 0, s, num_rows, I, O, x, \
                     y, dy, activation, slices, partials)
  if (ept <= 1) MCCNN_PD_LAUNCH(1);
  else if (ept <= 2) MCCNN_PD_LAUNCH(2);
  else if (ept <= 4) MCCNN_PD_LAUNCH(4);
  else if (ept <= 8) MCCNN_PD_LAUNCH(8);
  else MCCNN_PD_LAUNCH(17);
#undef MCCNN_PD_LAUNCH
  MCCNN_LAUNCH_CHECK();
  hipLaunchKernelGGL(pair_dense_reduce_kernel, dim3(blocks_for(elems, 256)), dim3(256), 0, s,
                     elems, I * O, slices, partials, dweights, dbiases);
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
