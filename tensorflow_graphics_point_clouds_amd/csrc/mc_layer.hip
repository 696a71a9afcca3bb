// Whole convolution layer in one kernel (pylib/pc/layers/MCConv.py:137-194,
// KPConv.py:165-232):
//     out[i, f] = sum_{c,k} proj[i, c, k] * W[c*16 + k, f],
//     proj[i, c, k] = sum_{m in nbh(i)} feat[nbr_m, c] * basis_k(pair m)
// with the [N, C*16] projection handed from the matrix-core accumulators to the
// product with the final weights through LDS, so that it reaches HBM only when the
// caller asks for it (the layer backward does, for the final-weight gradient).
//
// One block of 16 wavefronts per compute unit walks over tiles of 16 consecutive
// centres.  The whole [C*16, F] weight matrix lives in the block's registers for the
// life of the kernel (wavefront (slice, column tile) keeps its rows x 16 columns as
// B operands, at most 64 registers per lane), so the weights are read once per
// block rather than once per tile.  Per tile:
//   1. each wavefront projects one centre as the projection kernel does and parks
//      its [C, 16] accumulators in its row of the LDS tile (natural c*16 + k order,
//      written as contiguous kilobytes);
//   2. (optional) the block copies the tile to proj_out with coalesced streaming stores;
//   3. every wavefront multiplies the 16 x rows slice of the tile (A operand, read
//      from LDS 16 bytes at a time) with its registers: four independent
//      accumulator chains, summed in a fixed order;
//   4. the per-slice partial tiles are added through LDS in a fixed order and the
//      16 x F result rows leave as contiguous rows.
// Two block-wide barriers per tile.  Results are bit-reproducible.
#include "common.h"
#include "fill.h"
#include "mfma.h"
#include "mc_conv.h"

namespace mccnn {

constexpr int kLayerWaves = 16;          // wavefronts per block = centres per tile
constexpr int kLayerThreads = kLayerWaves * kWave;

// C*16*F <= 65536 floats fit the registers of one block; the LDS tile holds C <= 64.
static bool layer_supported(int D, int C, int K, int F) {
  const bool c_ok = C == 16 || C == 32 || C == 64;
  const bool f_ok = F == 16 || F == 32 || F == 64 || F == 128;
  return (D == 2 || D == 3) && K == kFusedK && c_ok && f_ok && C * K * F <= 65536;
}

template <int kCPL, int FT>
struct LayerShape {
  static constexpr int C = 16 * kCPL;
  static constexpr int R = C * kFusedK;          // reduction length of the final product
  static constexpr int F = 16 * FT;
  static constexpr int kSlices = kLayerWaves / FT;   // reduction slices (FT <= 16)
  static constexpr int kSliceRows = R / kSlices;
  static constexpr int kSteps = kSliceRows / 4;  // matrix steps (= weight registers) per lane
  static constexpr int kTileStride = R + 4;      // floats; rows 16 bytes apart in the banks
  static constexpr size_t kTileFloats = (size_t)kLayerWaves * kTileStride;
  static constexpr size_t kPartialFloats = (size_t)kSlices * 16 * F;
  static constexpr size_t kLdsBytes =
      sizeof(float) * (kTileFloats + kPartialFloats) + sizeof(PairStage) * kLayerWaves;
};

// Row strides (in floats) of the dense product's operands when they are blocks of larger
// matrices: x [N, ldx], W [., ldw], out [N, ldo]; `accumulate` adds to what `out` holds.
// Zero means "the block is the whole matrix" (R, F and F).
struct DenseStrides {
  int64_t ldx = 0, ldw = 0, ldo = 0;
  int r_total = 0;       // reduction length of the whole product, walked in blocks of R
  int f_block = 0;       // columns per blockIdx.y
};

template <int kCPL, int FT, int D, class Basis, bool kDense = false>
__device__ __forceinline__ void layer_body(int64_t n_out, const float *__restrict__ feat,
                                           const int2 *__restrict__ nbrs,
                                           const int *__restrict__ ranges, const McParams<D> &p,
                                           const Basis &basis, const float *__restrict__ w,
                                           const int *__restrict__ out_rows,
                                           float *__restrict__ proj_out, float *__restrict__ out,
                                           float *lds, const DenseStrides ld = DenseStrides{}) {
  using S = LayerShape<kCPL, FT>;
  constexpr int C = S::C, R = S::R, F = S::F, kSteps = S::kSteps;
  float *tile = lds;
  float *partial = tile + S::kTileFloats;
  PairStage *stages = reinterpret_cast<PairStage *>(partial + S::kPartialFloats);
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
  const int quarter = lane >> 4, col = lane & 15;
  const int slice = wave / FT, ft = wave - slice * FT;

  // B operands of this wavefront: step s of lane (quarter, col) multiplies tile column
  // slice*kSliceRows + quarter*kSteps + s with W[that row][16 ft + col]
  const int64_t ldx = kDense && ld.ldx ? ld.ldx : R, ldw = kDense && ld.ldw ? ld.ldw : F;
  const int64_t ldo = kDense && ld.ldo ? ld.ldo : F;
  const int r_total = kDense && ld.r_total ? ld.r_total : R;
  if constexpr (kDense) {           // this block's columns of a wider product
    w += (int64_t)blockIdx.y * ld.f_block;
    out += (int64_t)blockIdx.y * ld.f_block;
  }
  const float *arow = tile + col * S::kTileStride + slice * S::kSliceRows + quarter * kSteps;
  const int64_t tiles = (n_out + kLayerWaves - 1) / kLayerWaves;
  // A product whose weights exceed the block's registers walks the reduction in blocks of
  // R rows of w: the block's tiles are visited once per block of rows, the later visits
  // adding to what the earlier ones wrote (the same thread owns an output element in every
  // visit, so the sum has a fixed order and needs no fence).
  for (int r0 = 0; r0 < r_total; r0 += R, feat += kDense ? R : 0, w += (int64_t)R * ldw) {
  float wreg[kSteps];
  {
    const float *wl = w + (int64_t)(slice * S::kSliceRows + quarter * kSteps) * ldw + 16 * ft + col;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) wreg[s] = wl[(int64_t)s * ldw];
  }

  // dense producer: the wavefront's row of x, fetched one tile ahead (R / 256 loads of 16
  // bytes per lane, each covering one contiguous kilobyte of the row)
  constexpr int kRowLoads = R / 256;
  v4f xrow[kDense ? kRowLoads : 1];
  auto fetch_row = [&](int64_t tile_id) {
    if constexpr (kDense) {
      const int64_t row = tile_id * kLayerWaves + wave;
      const bool live = tile_id < tiles && row < n_out;
#pragma unroll
      for (int i = 0; i < kRowLoads; ++i)
        xrow[i] = live ? __builtin_nontemporal_load(reinterpret_cast<const v4f *>(
                             feat + row * ldx + 4 * (i * 64 + lane)))
                       : v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
  };
  fetch_row(blockIdx.x);
  for (int64_t t = blockIdx.x; t < tiles; t += gridDim.x) {
    const int64_t centre0 = t * kLayerWaves;
    const int64_t centre = centre0 + wave;
    if constexpr (kDense) {
      // ---- 1 (dense): this wavefront's row of x into the tile
#pragma unroll
      for (int i = 0; i < kRowLoads; ++i)
        *reinterpret_cast<v4f *>(tile + wave * S::kTileStride + 4 * (i * 64 + lane)) = xrow[i];
      __syncthreads();
      fetch_row(t + gridDim.x);               // in flight during the product
    } else {
      // ---- 1: projection of this wavefront's centre
      v4f acc[kCPL];
#pragma unroll
      for (int j = 0; j < kCPL; ++j) acc[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
      if (centre < n_out) {
        const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
        float ctr[D];
#pragma unroll
        for (int d = 0; d < D; ++d) ctr[d] = p.pout[centre * D + d];
        project_pairs<kCPL, D, Basis, true>(reinterpret_cast<const char *>(feat), (unsigned)C * 4,
                                            nbrs, a, b, p, ctr, stages + wave, basis, acc);
      }
      // acc[j][r] = proj[c = col + 16 j][k = 4 quarter + r]: for one j the wavefront's 64
      // stores of 16 bytes cover one contiguous kilobyte of the row
#pragma unroll
      for (int j = 0; j < kCPL; ++j)
        *reinterpret_cast<v4f *>(tile + wave * S::kTileStride + j * 256 + col * 16 +
                                 4 * quarter) = acc[j];
      __syncthreads();
    }
    // ---- 2: the tile as rows of proj_out
    if (!kDense && proj_out) {
      constexpr int kChunksPerRow = R / 4;
#pragma unroll
      for (int i = 0; i < kLayerWaves * kChunksPerRow / kLayerThreads; ++i) {
        const int chunk = threadIdx.x + kLayerThreads * i;
        const int row = chunk / kChunksPerRow, c4 = chunk - row * kChunksPerRow;
        if (centre0 + row < n_out) {
          const int64_t orow = out_rows ? out_rows[centre0 + row] : centre0 + row;
          const v4f v = *reinterpret_cast<const v4f *>(tile + row * S::kTileStride + 4 * c4);
          __builtin_nontemporal_store(v, reinterpret_cast<v4f *>(proj_out + orow * R + 4 * c4));
        }
      }
    }
    // ---- 3: [16 centres x slice rows] (LDS) times [slice rows x 16] (registers)
    v4f o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int s4 = 0; s4 < kSteps / 4; ++s4) {
      const float4 a = *reinterpret_cast<const float4 *>(arow + 4 * s4);
      o[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, wreg[4 * s4], o[0], 0, 0, 0);
      o[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, wreg[4 * s4 + 1], o[1], 0, 0, 0);
      o[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, wreg[4 * s4 + 2], o[2], 0, 0, 0);
      o[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, wreg[4 * s4 + 3], o[3], 0, 0, 0);
    }
    // o[.][r]: partial out[centre0 + 4 quarter + r][16 ft + col] of this slice
#pragma unroll
    for (int r = 0; r < 4; ++r)
      partial[(slice * 16 + 4 * quarter + r) * F + 16 * ft + col] =
          (o[0][r] + o[1][r]) + (o[2][r] + o[3][r]);
    __syncthreads();
    // ---- 4: sum of the slices, rows out
    for (int e = threadIdx.x; e < 16 * F; e += kLayerThreads) {
      const int ce = e / F;
      float s = 0.0f;
#pragma unroll
      for (int q = 0; q < S::kSlices; ++q) s += partial[q * 16 * F + e];
      if (centre0 + ce < n_out) {
        const int64_t orow = out_rows ? out_rows[centre0 + ce] : centre0 + ce;
        float *dst = out + orow * ldo + (e - ce * F);
        if (kDense && r0 > 0) s += *dst;
        *dst = s;
      }
    }
    // The next tile's rows are written after this barrier pair: every wavefront has
    // left step 3 (second barrier) before any row of the tile changes, and every
    // thread has left step 4 before it reaches the next first barrier, after which
    // the partial sums change.
  }
  if (r0 + R < r_total) __syncthreads();   // step 4 of the last tile has read the partial sums
  }
}

template <int kCPL, int FT, int D, int kAct>
__global__ void __launch_bounds__(kLayerThreads) mc_conv_layer16_kernel(
    int64_t n_out, const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, McParams<D> p, const float *__restrict__ w,
    const int *__restrict__ out_rows, float *__restrict__ proj_out, float *__restrict__ out) {
  extern __shared__ __align__(16) float lds[];
  const MlpBasis<D, kAct> basis(p);
  layer_body<kCPL, FT, D>(n_out, feat, nbrs, ranges, p, basis, w, out_rows, proj_out, out, lds);
}

template <int kCPL, int FT, int D, int kKind>
__global__ void __launch_bounds__(kLayerThreads) kp_conv_layer16_kernel(
    int64_t n_out, const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, McParams<D> p, const float *__restrict__ kernel_points,
    int num_kp, float sigma, const float *__restrict__ w, const int *__restrict__ out_rows,
    float *__restrict__ proj_out, float *__restrict__ out) {
  extern __shared__ __align__(16) float lds[];
  const KpBasis<D, kKind> basis(kernel_points, num_kp, sigma);
  layer_body<kCPL, FT, D>(n_out, feat, nbrs, ranges, p, basis, w, out_rows, proj_out, out, lds);
}

// The product alone: out[n, :] = x[n, :] * W for x [N, R] in HBM (the projection written by
// the projection kernels, or its transposed counterpart in the layer backward).  Same
// tiles, registers and summation order as above; x is read exactly once.
struct NoBasis {};

template <int kCPL, int FT>
__global__ void __launch_bounds__(kLayerThreads) final_product_kernel(
    int64_t n, const float *__restrict__ x, const float *__restrict__ w,
    const int *__restrict__ out_rows, float *__restrict__ out, DenseStrides ld) {
  extern __shared__ __align__(16) float lds[];
  const McParams<3> none{};
  layer_body<kCPL, FT, 3, NoBasis, true>(n, x, nullptr, nullptr, none, NoBasis{}, w, out_rows,
                                         nullptr, out, lds, ld);
}

// One block per compute unit (the LDS tile and 1024 threads fill it), fewer if
// there are fewer tiles.
static int layer_grid(int64_t num_samples, unsigned *blocks) {
  int device = 0, cus = 0;
  MCCNN_HIP_CHECK(hipGetDevice(&device));
  MCCNN_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  const int64_t tiles = (num_samples + kLayerWaves - 1) / kLayerWaves;
  *blocks = (unsigned)(tiles < cus ? (tiles < 1 ? 1 : tiles) : cus);
  return MCCNN_OK;
}

template <class Kernel, class... Args>
static int launch_layer(Kernel kernel, hipStream_t s, dim3 blocks, size_t lds, Args... args) {
  MCCNN_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kernel, blocks, dim3(kLayerThreads), lds, s, args...);
  return MCCNN_OK;
}

static int check_layer_args(const char *op, int num_dims, int num_features, int num_basis,
                            int num_out_features, int64_t num_pts, int64_t num_neighbors,
                            int64_t num_samples) {
  MCCNN_REQUIRE(layer_supported(num_dims, num_features, num_basis, num_out_features),
                "%s supports D in {2,3}, 16 basis columns, C in {16,32,64} and F in "
                "{16,32,64,128} with C*16*F <= 65536 (got D=%d, K=%d, C=%d, F=%d)", op, num_dims,
                num_basis, num_features, num_out_features);
  MCCNN_REQUIRE(num_pts >= 0 && num_pts * num_features < ((int64_t)1 << 30),
                "%s expects a feature table of fewer than 2^30 elements", op);
  MCCNN_REQUIRE(num_neighbors >= 0 && num_neighbors < ((int64_t)1 << 31) && num_samples >= 0 &&
                    num_samples < ((int64_t)1 << 31),
                "%s expects sizes in [0, 2^31)", op);
  return MCCNN_OK;
}

static int zero_outputs(hipStream_t s, int64_t num_samples, int C, int F, float *proj_out,
                        float *out) {
  int rc = fill_zero(s, out, sizeof(float) * (size_t)num_samples * F);
  if (rc == MCCNN_OK && proj_out)
    rc = fill_zero(s, proj_out, sizeof(float) * (size_t)num_samples * C * kFusedK);
  return rc;
}

// Expands BODY for the (channels per lane, column tiles) pair of a covered shape.
#define MCCNN_LAYER_SHAPE_SWITCH(C_, F_, BODY)                                  \
  switch (((C_) / 16) * 100 + (F_) / 16) {                                      \
    case 101: { constexpr int CPL = 1, FT = 1; BODY; } break;                   \
    case 102: { constexpr int CPL = 1, FT = 2; BODY; } break;                   \
    case 104: { constexpr int CPL = 1, FT = 4; BODY; } break;                   \
    case 108: { constexpr int CPL = 1, FT = 8; BODY; } break;                   \
    case 201: { constexpr int CPL = 2, FT = 1; BODY; } break;                   \
    case 202: { constexpr int CPL = 2, FT = 2; BODY; } break;                   \
    case 204: { constexpr int CPL = 2, FT = 4; BODY; } break;                   \
    case 208: { constexpr int CPL = 2, FT = 8; BODY; } break;                   \
    case 401: { constexpr int CPL = 4, FT = 1; BODY; } break;                   \
    case 402: { constexpr int CPL = 4, FT = 2; BODY; } break;                   \
    default: { constexpr int CPL = 4, FT = 4; BODY; } break;                    \
  }

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_mc_conv_layer_supported(int num_dims, int num_features, int num_basis,
                                             int num_out_features) {
  return layer_supported(num_dims, num_features, num_basis, num_out_features) ? 1 : 0;
}

extern "C" int mccnn_mc_conv_layer(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                                   const float *points_in, int num_features,
                                   const float *features, int64_t num_samples,
                                   const float *points_out, int64_t num_neighbors,
                                   const int32_t *neighbors, const int32_t *ranges,
                                   const float *inv_radii, int num_basis, int num_mlps,
                                   int activation, const float *weights, const float *biases,
                                   const float *pdf, int num_out_features,
                                   const float *final_weights, const int32_t *out_rows,
                                   float *proj_out, float *out) {
  int rc = check_layer_args("mc_conv_layer", num_dims, num_features, num_basis,
                            num_out_features, num_pts, num_neighbors, num_samples);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(num_mlps > 0 && num_basis % num_mlps == 0,
                "mc_conv_layer expects the number of basis functions to be divisible by the "
                "number of kernel MLPs");
  MCCNN_REQUIRE(activation >= 0 && activation <= 2, "mc_conv_layer expects a known activation");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && out && points_out && inv_radii && weights && biases &&
                    final_weights &&
                    (num_neighbors == 0 || (points_in && features && neighbors && pdf)),
                "mc_conv_layer received a null tensor");
  hipStream_t s = as_stream(stream);
  if (num_neighbors == 0)       // no pairs: zero rows (the kernel assumes a feature table)
    return zero_outputs(s, num_samples, num_features, num_out_features, proj_out, out);
  unsigned blocks = 1;
  rc = layer_grid(num_samples, &blocks);
  if (rc != MCCNN_OK) return rc;
  const int2 *nb = (const int2 *)neighbors;
#define MCCNN_LAYER_D(D_)                                                                      \
  {                                                                                            \
    McParams<D_> prm{points_in, points_out, inv_radii, weights, biases, pdf,                   \
                     num_basis / num_mlps, activation};                                        \
    MCCNN_ACT_SWITCH(activation,                                                               \
                     rc = launch_layer(mc_conv_layer16_kernel<CPL, FT, D_, ACT>, s, blocks,    \
                                       LayerShape<CPL, FT>::kLdsBytes, num_samples, features,  \
                                       nb, ranges, prm, final_weights, out_rows, proj_out,     \
                                       out));                                                  \
  }
  MCCNN_LAYER_SHAPE_SWITCH(num_features, num_out_features,
                           if (num_dims == 3) MCCNN_LAYER_D(3) else MCCNN_LAYER_D(2));
#undef MCCNN_LAYER_D
  if (rc != MCCNN_OK) return rc;
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_kp_conv_layer(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                                   const float *points_in, int num_features,
                                   const float *features, int64_t num_samples,
                                   const float *points_out, int64_t num_neighbors,
                                   const int32_t *neighbors, const int32_t *ranges,
                                   const float *inv_radii, int num_kernel_points,
                                   const float *kernel_points, int kind, float sigma,
                                   int num_out_features, const float *final_weights,
                                   const int32_t *out_rows, float *proj_out, float *out) {
  int rc = check_layer_args("kp_conv_layer", num_dims, num_features, kFusedK, num_out_features,
                            num_pts, num_neighbors, num_samples);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(num_kernel_points > 0 && num_kernel_points <= kFusedK,
                "kp_conv_layer expects 1..16 kernel points (got %d)", num_kernel_points);
  MCCNN_REQUIRE(kind == 0 || kind == 1, "kp_conv_layer expects kind 0 (linear) or 1 (gaussian)");
  MCCNN_REQUIRE(sigma > 0.0f, "kp_conv_layer expects a positive sigma");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && out && points_out && inv_radii && kernel_points && final_weights &&
                    (num_neighbors == 0 || (points_in && features && neighbors)),
                "kp_conv_layer received a null tensor");
  hipStream_t s = as_stream(stream);
  if (num_neighbors == 0)       // no pairs: zero rows (the kernel assumes a feature table)
    return zero_outputs(s, num_samples, num_features, num_out_features, proj_out, out);
  unsigned blocks = 1;
  rc = layer_grid(num_samples, &blocks);
  if (rc != MCCNN_OK) return rc;
  const int2 *nb = (const int2 *)neighbors;
#define MCCNN_LAYER_DK(D_, KIND_)                                                              \
  {                                                                                            \
    McParams<D_> prm{points_in, points_out, inv_radii, nullptr, nullptr, nullptr, 0, 0};       \
    rc = launch_layer(kp_conv_layer16_kernel<CPL, FT, D_, KIND_>, s, blocks,                   \
                      LayerShape<CPL, FT>::kLdsBytes, num_samples, features, nb, ranges, prm,  \
                      kernel_points, num_kernel_points, sigma, final_weights, out_rows,        \
                      proj_out, out);                                                          \
  }
#define MCCNN_LAYER_D(D_) \
  if (kind == 0) MCCNN_LAYER_DK(D_, 0) else MCCNN_LAYER_DK(D_, 1)
  MCCNN_LAYER_SHAPE_SWITCH(num_features, num_out_features,
                           if (num_dims == 3) MCCNN_LAYER_D(3) else MCCNN_LAYER_D(2));
#undef MCCNN_LAYER_D
#undef MCCNN_LAYER_DK
  if (rc != MCCNN_OK) return rc;
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

// Blocks of the reduction and of the output columns that one launch covers: the
// largest column block first (x is read once per column block), then the longest
// reduction block whose weights still fit the registers of a block of wavefronts.
static bool product_blocks(int R, int F, int *rb, int *fb) {
  if (R < 256 || R % 256 != 0 || F < 16 || F % 16 != 0) return false;
  for (int f = 128; f >= 16; f >>= 1) {
    if (F % f != 0) continue;
    for (int r = 1024; r >= 256; r >>= 1)
      if (R % r == 0 && r * f <= 65536) {
        *rb = r;
        *fb = f;
        return true;
      }
  }
  return false;
}

extern "C" int mccnn_final_product_supported(int num_cols_in, int num_cols_out) {
  int rb = 0, fb = 0;
  return num_cols_in <= 8192 && num_cols_out <= 1024 &&
                 product_blocks(num_cols_in, num_cols_out, &rb, &fb)
             ? 1 : 0;
}

extern "C" int mccnn_final_product(mccnn_stream_t stream, int64_t num_rows, int num_cols_in,
                                   const float *x, int num_cols_out, const float *w,
                                   const int32_t *out_rows, float *out) {
  MCCNN_REQUIRE(mccnn_final_product_supported(num_cols_in, num_cols_out),
                "final_product supports a multiple of 256 (at most 8192) input columns and a "
                "multiple of 16 (at most 1024) output columns (got %d x %d)", num_cols_in,
                num_cols_out);
  MCCNN_REQUIRE(num_rows >= 0 && num_rows < ((int64_t)1 << 31),
                "final_product expects a size in [0, 2^31)");
  if (num_rows == 0) return MCCNN_OK;
  MCCNN_REQUIRE(x && w && out, "final_product received a null tensor");
  hipStream_t s = as_stream(stream);
  int device = 0, cus = 0, rc = MCCNN_OK;
  MCCNN_HIP_CHECK(hipGetDevice(&device));
  MCCNN_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  const int R = num_cols_in, F = num_cols_out;
  const int64_t tiles = (num_rows + kLayerWaves - 1) / kLayerWaves;
  // weights beyond a block's registers: the tiled product, once its 128- or 256-row tiles give
  // every compute unit a block (below that a launch is a few blocks walking the whole
  // reduction alone: 170 us for 400 rows x 4096 x 256 against 20 us for the blocked
  // register-resident product, whose tiles are 16 rows)
  if ((int64_t)R * F > 65536 && tile_product_supported(R, F) &&
      (num_rows + tile_product_rows(F) - 1) / tile_product_rows(F) *
              (F / (F % 128 == 0 ? 128 : 64)) >= cus)
    return launch_tile_product(s, num_rows, R, x, F, w, false, out_rows, out);
  int rb = 0, fb = 0;
  product_blocks(R, F, &rb, &fb);
  // A small input leaves compute units idle: narrower column blocks with longer reduction
  // blocks then give more blocks of threads, each walking fewer blocks of the reduction
  // (1500 rows x 4096 x 256: 8 visits of 512 rows of w per block of threads become 4 of 1024)
  while (fb > 16 && rb < 1024 && R % (2 * rb) == 0 && tiles * (F / (fb / 2)) <= cus) {
    fb /= 2;
    rb *= 2;
  }
  // out[:, f0:f0+fb] = sum over the reduction blocks r0 of x[:, r0:r0+rb] W[r0:r0+rb, f0:f0+fb]:
  // one launch, column block f0 = blockIdx.y * fb, every block walking the reduction blocks
  // in order for its own tiles
  DenseStrides ld;
  ld.ldx = R;
  ld.ldw = F;
  ld.ldo = F;
  ld.r_total = R;
  ld.f_block = fb;
  const int col_blocks = F / fb;
  // one block per compute unit in all (the register-resident weights and the LDS tile
  // fill it), shared among the column blocks; never more blocks than tiles
  int64_t per = cus / col_blocks < 1 ? 1 : cus / col_blocks;
  if (per > tiles) per = tiles;
  const unsigned blocks = (unsigned)per;
  MCCNN_LAYER_SHAPE_SWITCH(rb / kFusedK, fb,
                           rc = launch_layer(final_product_kernel<CPL, FT>, s,
                                             dim3(blocks, (unsigned)col_blocks),
                                             LayerShape<CPL, FT>::kLdsBytes, num_rows, x, w,
                                             out_rows, out, ld));
  if (rc != MCCNN_OK) return rc;
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

// The same product with the weights given transposed, wt [F, R] (rows of w^T are
// contiguous along the reduction, like the rows of x): the layout the tiled product
// fetches without a transposing pass through LDS.
extern "C" int mccnn_final_product_wt_supported(int num_cols_in, int num_cols_out) {
  return tile_product_supported(num_cols_in, num_cols_out) ? 1 : 0;
}

extern "C" int mccnn_final_product_wt(mccnn_stream_t stream, int64_t num_rows, int num_cols_in,
                                      const float *x, int num_cols_out, const float *wt,
                                      const int32_t *out_rows, float *out) {
  MCCNN_REQUIRE(tile_product_supported(num_cols_in, num_cols_out),
                "final_product_wt supports a multiple of 32 input columns and a multiple of 64 "
                "output columns (got %d x %d)", num_cols_in, num_cols_out);
  MCCNN_REQUIRE(num_rows >= 0 && num_rows < ((int64_t)1 << 31),
                "final_product_wt expects a size in [0, 2^31)");
  if (num_rows == 0) return MCCNN_OK;
  MCCNN_REQUIRE(x && wt && out, "final_product_wt received a null tensor");
  return launch_tile_product(as_stream(stream), num_rows, num_cols_in, x, num_cols_out, wt, true,
                             out_rows, out);
}
