// Whole Monte-Carlo convolution in one kernel (pylib/pc/layers/MCConv.py:137-194):
//     out[i, f] = sum_{c,k} proj[i, c, k] * W[c*K + k, f],
//     proj[i, c, k] = sum_{m in nbh(i)} feat[nbr_m, c] * act(delta_m . A[:, k] + b[k]) / pdf[m]
// A block of 16 wavefronts owns 16 consecutive centres.  Phase 1: each wavefront
// accumulates the [C, 16] projection of one centre on the matrix cores exactly as
// the projection kernel does and parks it in LDS.  Phase 2: the 16 x (C*16) tile
// in LDS is the A operand of the product with the final weights; the wavefronts
// split the F/16 column tiles and the reduction range among themselves, stream
// their slice of the (pre-permuted) weights from L2 and combine their partial
// tiles through LDS.  The [N_out, C, K] projection never reaches HBM unless the
// caller asks for it (the layer backward does, for the weight gradient).
// K = 16, D in {2, 3}, C and F in {16, 32, 64, 128}.
#include "common.h"
#include "fill.h"
#include "mfma.h"
#include "mc_conv.h"

namespace mccnn {

constexpr int kLayerWaves = 16;          // wavefronts (= centres) per block
constexpr int kLayerPad = 17;            // LDS row stride of the tile, in floats

static bool layer_supported(int D, int C, int K, int F) {
  auto ok = [](int x) { return x == 16 || x == 32 || x == 64 || x == 128; };
  return (D == 2 || D == 3) && K == kFusedK && ok(C) && ok(F);
}

// Row of the LDS tile -> row of the [C*16, F] weight matrix.  Phase 1 leaves
// proj[c = col*kCPL + j][k = 4*quarter + r] of lane (quarter, col) in tile row
// (j*4 + r)*64 + lane, which makes its LDS stores conflict-free.
__host__ __device__ inline int tile_row_to_weight_row(int row, int cpl) {
  const int lane = row & 63, jr = row >> 6;
  const int j = jr >> 2, r = jr & 3, col = lane & 15, quarter = lane >> 4;
  return (col * cpl + j) * kFusedK + 4 * quarter + r;
}

// packed[((wave * (steps/4) + s/4) * 64 + lane) * 4 + s%4] = the B-operand value
// of `lane` at reduction step `s` of wavefront `wave` (column tile ct = wave /
// split, reduction slice sp = wave % split).
__global__ void __launch_bounds__(256) pack_final_weights_kernel(int C, int F,
                                                                 const float *__restrict__ w,
                                                                 float *__restrict__ packed) {
  const int R = C * kFusedK, cpl = C / 16;
  const int split = kLayerWaves / (F / 16), steps = R / 4 / split;
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= R * F) return;
  const int i = t & 3, lane = (t >> 2) & 63;
  const int rest = t >> 8;                 // wave * (steps/4) + s/4
  const int s4 = rest % (steps / 4), wave = rest / (steps / 4);
  const int ct = wave / split, sp = wave - ct * split;
  const int row = sp * (R / split) + 4 * (4 * s4 + i) + (lane >> 4);
  packed[t] = w[(int64_t)tile_row_to_weight_row(row, cpl) * F + ct * 16 + (lane & 15)];
}

template <int kCPL, int D, int kAct>
__global__ void __launch_bounds__(1024) mc_conv_layer16_kernel(
    int64_t n_out, int F, const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, McParams<D> p, const float4 *__restrict__ packed_w,
    float *__restrict__ proj_out, float *__restrict__ out) {
  constexpr int K = kFusedK;
  constexpr int C = 16 * kCPL;
  constexpr int R = C * K;
  extern __shared__ float tile[];          // [R][kLayerPad]; later [split][16][F] partial sums
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
  const int64_t centre0 = (int64_t)blockIdx.x * kLayerWaves;
  const int64_t centre = centre0 + wave;
  const int quarter = lane >> 4, col = lane & 15;

  // ---- phase 1: projection of this wavefront's centre --------------------
  // (the pair staging areas live in the tile region, which is not written
  //  before every wavefront has left phase 1)
  v4f acc[kCPL];
#pragma unroll
  for (int j = 0; j < kCPL; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[j][r] = 0.0f;
  if (centre < n_out) {
    const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
    float ctr[D];
#pragma unroll
    for (int d = 0; d < D; ++d) ctr[d] = p.pout[centre * D + d];
    const MlpBasis<D, kAct> basis(p);
    project_pairs<kCPL, D>(reinterpret_cast<const char *>(feat), (unsigned)C * 4, nbrs, a, b, p,
                           ctr, reinterpret_cast<PairStage *>(tile) + wave, basis, acc);
    if (proj_out) {
      float *o = proj_out + centre * (int64_t)C * K + 4 * quarter;
#pragma unroll
      for (int j = 0; j < kCPL; ++j)
        *reinterpret_cast<v4f *>(o + (col * kCPL + j) * K) = acc[j];
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kCPL; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) tile[((j * 4 + r) * 64 + lane) * kLayerPad + wave] = acc[j][r];

  // ---- phase 2: [16 centres x R] (LDS) times [R x F] (packed weights) ----
  const int split = kLayerWaves / (F >> 4);
  const int ct = wave / split, sp = wave - ct * split;
  const int groups = R / 16 / split;       // float4 loads (= 4 reduction steps each) per lane
  const float4 *wp = packed_w + (int64_t)wave * groups * 64 + lane;
  float4 b0 = wp[0];
  float4 b1 = groups > 1 ? wp[64] : b0;
  __syncthreads();
  const float *arow = tile + (sp * (R / split) + quarter) * kLayerPad + col;
  v4f o = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int g = 0; g < groups; ++g) {
    const float4 b2 = g + 2 < groups ? wp[(int64_t)(g + 2) * 64] : b0;
    const float *ar = arow + g * 16 * kLayerPad;
    o = __builtin_amdgcn_mfma_f32_16x16x4f32(ar[0], b0.x, o, 0, 0, 0);
    o = __builtin_amdgcn_mfma_f32_16x16x4f32(ar[4 * kLayerPad], b0.y, o, 0, 0, 0);
    o = __builtin_amdgcn_mfma_f32_16x16x4f32(ar[8 * kLayerPad], b0.z, o, 0, 0, 0);
    o = __builtin_amdgcn_mfma_f32_16x16x4f32(ar[12 * kLayerPad], b0.w, o, 0, 0, 0);
    b0 = b1;
    b1 = b2;
  }
  __syncthreads();                          // every wavefront has finished reading the tile
  // o[r] = partial out[centre0 + 4*quarter + r][ct*16 + col] of reduction slice sp
#pragma unroll
  for (int r = 0; r < 4; ++r) tile[(sp * 16 + 4 * quarter + r) * F + ct * 16 + col] = o[r];
  __syncthreads();
  for (int t = threadIdx.x; t < 16 * F; t += 1024) {
    const int ce = t / F;
    float s = 0.0f;
    for (int q = 0; q < split; ++q) s += tile[q * 16 * F + t];
    if (centre0 + ce < n_out) out[(centre0 + ce) * F + (t - ce * F)] = s;
  }
}

template <int kCPL, int D, int ACT>
static int launch_layer(hipStream_t s, dim3 grid, dim3 block, size_t lds, int64_t num_samples,
                        int F, const float *features, const int2 *nb, const int *ranges,
                        const McParams<D> &prm, const float4 *packed, float *proj_out,
                        float *out) {
  auto kernel = mc_conv_layer16_kernel<kCPL, D, ACT>;
  MCCNN_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kernel, grid, block, lds, s, num_samples, F, features, nb, ranges, prm,
                     packed, proj_out, out);
  return MCCNN_OK;
}

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_mc_conv_layer_supported(int num_dims, int num_features, int num_basis,
                                             int num_out_features) {
  return layer_supported(num_dims, num_features, num_basis, num_out_features) ? 1 : 0;
}

extern "C" size_t mccnn_mc_conv_layer_workspace_bytes(int num_features, int num_basis,
                                                      int num_out_features) {
  if (num_features <= 0 || num_basis <= 0 || num_out_features <= 0) return 0;
  return align256(sizeof(float) * (size_t)num_features * num_basis * num_out_features);
}

extern "C" int mccnn_mc_conv_layer(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                                   const float *points_in, int num_features,
                                   const float *features, int64_t num_samples,
                                   const float *points_out, int64_t num_neighbors,
                                   const int32_t *neighbors, const int32_t *ranges,
                                   const float *inv_radii, int num_basis, int num_mlps,
                                   int activation, const float *weights, const float *biases,
                                   const float *pdf, int num_out_features,
                                   const float *final_weights, void *workspace,
                                   size_t workspace_bytes, float *proj_out, float *out) {
  MCCNN_REQUIRE(layer_supported(num_dims, num_features, num_basis, num_out_features),
                "mc_conv_layer supports D in {2,3}, K = 16 and C, F in {16,32,64,128} (got D=%d, "
                "K=%d, C=%d, F=%d)", num_dims, num_basis, num_features, num_out_features);
  MCCNN_REQUIRE(num_mlps > 0 && num_basis % num_mlps == 0,
                "mc_conv_layer expects the number of basis functions to be divisible by the "
                "number of kernel MLPs");
  MCCNN_REQUIRE(activation >= 0 && activation <= 2, "mc_conv_layer expects a known activation");
  MCCNN_REQUIRE(num_pts * num_features < ((int64_t)1 << 30),
                "mc_conv_layer expects a feature table of fewer than 2^30 elements");
  MCCNN_REQUIRE(num_pts >= 0 && num_neighbors >= 0 && num_neighbors < ((int64_t)1 << 31) &&
                    num_samples >= 0 && num_samples < ((int64_t)1 << 31),
                "mc_conv_layer expects sizes in [0, 2^31)");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && out && points_out && inv_radii && weights && biases &&
                    final_weights && workspace &&
                    (num_neighbors == 0 || (points_in && features && neighbors && pdf)),
                "mc_conv_layer received a null tensor");
  MCCNN_REQUIRE(workspace_bytes >= mccnn_mc_conv_layer_workspace_bytes(num_features, num_basis,
                                                                       num_out_features),
                "mc_conv_layer workspace too small");
  hipStream_t s = as_stream(stream);
  const int C = num_features, F = num_out_features, R = C * kFusedK;
  hipLaunchKernelGGL(pack_final_weights_kernel, dim3(blocks_for((int64_t)R * F, 256)), dim3(256),
                     0, s, C, F, final_weights, (float *)workspace);
  MCCNN_LAUNCH_CHECK();
  const size_t lds_tile = sizeof(float) * (size_t)R * kLayerPad;
  const size_t lds_red = sizeof(float) * 16 * (size_t)F * (kLayerWaves / (F / 16));
  size_t lds = lds_tile > lds_red ? lds_tile : lds_red;
  if (lds < sizeof(PairStage) * kLayerWaves) lds = sizeof(PairStage) * kLayerWaves;
  const dim3 grid(blocks_for(num_samples, kLayerWaves)), block(kLayerWaves * kWave);
  const int2 *nb = (const int2 *)neighbors;
  int rc = MCCNN_OK;
#define MCCNN_LAYER(CPL_, D_)                                                                  \
  {                                                                                            \
    McParams<D_> prm{points_in, points_out, inv_radii, weights, biases, pdf,                   \
                     num_basis / num_mlps, activation};                                        \
    MCCNN_ACT_SWITCH(activation,                                                               \
                     rc = (launch_layer<CPL_, D_, ACT>(s, grid, block, lds, num_samples, F,    \
                                                       features, nb, ranges, prm,              \
                                                       (const float4 *)workspace, proj_out,    \
                                                       out)));                                 \
  }
#define MCCNN_LAYER_D(CPL_) \
  if (num_dims == 3) MCCNN_LAYER(CPL_, 3) else MCCNN_LAYER(CPL_, 2)
  switch (C / 16) {
    case 8: MCCNN_LAYER_D(8); break;
    case 4: MCCNN_LAYER_D(4); break;
    case 2: MCCNN_LAYER_D(2); break;
    default: MCCNN_LAYER_D(1); break;
  }
#undef MCCNN_LAYER_D
#undef MCCNN_LAYER
  if (rc != MCCNN_OK) return rc;
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
