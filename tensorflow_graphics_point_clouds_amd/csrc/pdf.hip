// Gaussian kernel density per point over its neighbour list and the gradient
// with respect to the point coordinates
// (custom_ops/tfg_custom_ops/compute_pdf/cc/kernels/compute_pdf_kernels.cu.cc:72-215).
//
// 4, 8 or 16 lanes share a centre and stride over its pairs; the pair table is read
// coalesced, neighbour coordinates are gathered (they sit close together in the
// sorted array, so the gathers hit L2).  The product over dimensions of
// exp(-u_d^2/2) is evaluated as one exponential of the summed exponent.
#include "common.h"
#include "fill.h"

namespace mccnn {

constexpr int kPdfThreads = 256;
constexpr float kInvSqrt2Pi = 0.39894228f;

template <int D>
struct PdfScale {
  float s[D];     // bw_d * inv_radii_d
  float norm;     // prod_d bw_d * 0.39894228
};

template <int D>
__device__ __forceinline__ PdfScale<D> load_pdf_scale(const float *__restrict__ inv_bw,
                                                      const float *__restrict__ inv_r, int mode,
                                                      int64_t n) {
  PdfScale<D> sc;
  sc.norm = 1.0f;
#pragma unroll
  for (int d = 0; d < D; ++d) {
    const float bw = mode == 0 ? inv_bw[d] : sqrtf((float)n);
    sc.s[d] = bw * inv_r[d];
    sc.norm *= bw * kInvSqrt2Pi;
  }
  return sc;
}

// G lanes share a centre.  The kernel is bound by the chain of dependent loads of a centre
// (list bounds, pair indices, coordinates) times the centres a compute unit holds in flight,
// so short lists want few lanes per centre (more centres per wavefront) and long lists many:
// 4 x 200k points, 7.5 / 52 / 170 pairs per point: 0.027 / 0.134 / 0.486 ms with 4 lanes,
// 0.041 / 0.115 / 0.355 ms with 8, 0.074 / 0.133 / 0.315 ms with 16.
template <int D, int G>
__global__ void __launch_bounds__(kPdfThreads) compute_pdf_kernel(
    int64_t n, const float *__restrict__ pts, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, const float *__restrict__ inv_bw,
    const float *__restrict__ inv_r, int mode, float *__restrict__ pdf) {
  const PdfScale<D> sc = load_pdf_scale<D>(inv_bw, inv_r, mode, n);
  const int sub = threadIdx.x & (G - 1);
  const int64_t c = (int64_t)blockIdx.x * (kPdfThreads / G) + threadIdx.x / G;
  if (c >= n) return;
  float p[D];
#pragma unroll
  for (int d = 0; d < D; ++d) p[d] = pts[c * D + d];
  const int64_t a = c > 0 ? ranges[c - 1] : 0, b = ranges[c];
  // four pairs per lane and trip: their index loads, then their coordinate gathers, are
  // in flight together (the sums keep the order of a one-pair-per-trip loop)
  float acc = 0.0f;
  for (int64_t m = a + sub; m < b; m += 4 * G) {
    int64_t j[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) j[q] = m + q * G < b ? nbrs[m + q * G].x : -1;
    float e[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      e[q] = 0.0f;
      const int64_t jj = j[q] < 0 ? c : j[q];
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const float u = (pts[jj * D + d] - p[d]) * sc.s[d];
        e[q] += u * u;
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) acc += j[q] < 0 ? 0.0f : expf(-0.5f * e[q]);
  }
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, kWave);
  if (sub == 0) pdf[c] = acc * sc.norm;
}

#ifdef MCCNN_PROBE_STAGED_PDF
// Measurement probe (correct results, built by `make probes` only): the same density with the
// neighbours' coordinates staged in LDS.  A block takes 32 consecutive centres, 8 lanes each.
// It finds the span of point indices its pairs touch, marks the chunks of 32 consecutive
// points that occur in a direct-mapped table (index span of up to 65 536 points, no hashing),
// gives every marked chunk a slot, copies the chunks' coordinates into LDS with coalesced
// loads, and then evaluates the pairs with the coordinates read from LDS.  Pairs whose chunk
// found no slot (more than kStageSlots chunks) and blocks whose span exceeds the table read
// their coordinates from memory as the shipped kernel does.
constexpr int kStageChunk = 32;
constexpr int kStageMaxChunks = 2048;
constexpr int kStageSlots = 48;

template <int D>
__global__ void __launch_bounds__(kPdfThreads) compute_pdf_staged_kernel(
    int64_t n, const float *__restrict__ pts, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, const float *__restrict__ inv_bw,
    const float *__restrict__ inv_r, int mode, float *__restrict__ pdf) {
  constexpr int G = 8, kCentres = kPdfThreads / G;
  constexpr unsigned short kUntouched = 0xffff, kTouched = 0xfffe;
  __shared__ unsigned short slot_of[kStageMaxChunks];
  __shared__ unsigned short chunk_of[kStageSlots];
  __shared__ float staged[kStageSlots * kStageChunk * D];
  __shared__ int s_min, s_max, s_count;
  const PdfScale<D> sc = load_pdf_scale<D>(inv_bw, inv_r, mode, n);
  const int sub = threadIdx.x & (G - 1);
  const int64_t c = (int64_t)blockIdx.x * kCentres + threadIdx.x / G;
  const bool live = c < n;
  float p[D];
#pragma unroll
  for (int d = 0; d < D; ++d) p[d] = live ? pts[c * D + d] : 0.0f;
  const int64_t a = live ? (c > 0 ? ranges[c - 1] : 0) : 0, b = live ? ranges[c] : 0;
  if (threadIdx.x == 0) {
    s_min = 0x7fffffff;
    s_max = -1;
    s_count = 0;
  }
  __syncthreads();
  int lo = 0x7fffffff, hi = -1;
  for (int64_t m = a + sub; m < b; m += G) {
    const int j = nbrs[m].x;
    lo = j < lo ? j : lo;
    hi = j > hi ? j : hi;
  }
  if (hi >= 0) {
    atomicMin(&s_min, lo);
    atomicMax(&s_max, hi);
  }
  __syncthreads();
  const int base = s_min;
  const int chunks = s_max >= 0 ? (s_max - base) / kStageChunk + 1 : 0;
  const bool table = chunks > 0 && chunks <= kStageMaxChunks;     // the same for the whole block
  if (table) {
    for (int i = threadIdx.x; i < chunks; i += kPdfThreads) slot_of[i] = kUntouched;
    __syncthreads();
    for (int64_t m = a + sub; m < b; m += G) slot_of[(nbrs[m].x - base) / kStageChunk] = kTouched;
    __syncthreads();
    for (int i = threadIdx.x; i < chunks; i += kPdfThreads)
      if (slot_of[i] == kTouched) {
        const int slot = atomicAdd(&s_count, 1);
        if (slot < kStageSlots) {
          slot_of[i] = (unsigned short)slot;
          chunk_of[slot] = (unsigned short)i;
        }
      }
    __syncthreads();
    const int slots = s_count < kStageSlots ? s_count : kStageSlots;
    for (int i = threadIdx.x; i < slots * kStageChunk * D; i += kPdfThreads) {
      const int slot = i / (kStageChunk * D), r = i - slot * (kStageChunk * D);
      const int64_t src = ((int64_t)base + (int64_t)chunk_of[slot] * kStageChunk) * D + r;
      staged[i] = src < n * D ? pts[src] : 0.0f;
    }
    __syncthreads();
  }
  float acc = 0.0f;
  for (int64_t m = a + sub; m < b; m += G) {
    const int j = nbrs[m].x;
    float q[D];
    unsigned slot = kUntouched;
    if (table) slot = slot_of[(j - base) / kStageChunk];
    if (slot < (unsigned)kStageSlots) {
      const float *src = &staged[(slot * kStageChunk + (j - base) % kStageChunk) * D];
#pragma unroll
      for (int d = 0; d < D; ++d) q[d] = src[d];
    } else {
#pragma unroll
      for (int d = 0; d < D; ++d) q[d] = pts[(int64_t)j * D + d];
    }
    float e = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float u = (q[d] - p[d]) * sc.s[d];
      e += u * u;
    }
    acc += expf(-0.5f * e);
  }
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, kWave);
  if (live && sub == 0) pdf[c] = acc * sc.norm;
}
#endif  // MCCNN_PROBE_STAGED_PDF

// grad[i] += g, grad[j] -= g with g_d = pdf_grad_i * pdf_ij * u_d * s_d
// (compute_pdf_kernels.cu.cc:133-215 scatters both halves with atomics).
// The gradient for an arbitrary pair table with as few atomics as the table allows.
// The term a pair (j in N(c)) sends to grad[j] equals the term that centre j would
// gather for its own pair (c in N(j)) with pdf_grad_c in place of pdf_grad_j (see the
// symmetric kernel below).  So centre c looks c up in the list of j: if it is there,
// c adds the reverse pair's term to its own register sum and nobody scatters; if it is
// not (a list cut by max_neighs, a hand-made table), c sends the term to grad[j] with
// an atomic.  Lists written by find_neighbors ascend by point index, so the look-up is a
// binary search; a miss is confirmed by a linear scan, which keeps tables in any order
// correct.  Preconditions: centre c is point c (the op requires num_samples == num_pts)
// and no pair occurs twice in the table.  Every centre adds its register sum once (grads
// are zero-filled first).  An
// untruncated self-neighbourhood takes no scatter at all: 41.8 M pairs in 1.06 ms where
// scattering every pair's term with atomics takes 3.4 ms.
template <int D, int G>
__global__ void __launch_bounds__(kPdfThreads) compute_pdf_grads_lookup_kernel(
    int64_t n, const float *__restrict__ pts, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, const float *__restrict__ inv_bw,
    const float *__restrict__ inv_r, const float *__restrict__ pdf_grads, int mode,
    float *__restrict__ grads) {
  const PdfScale<D> sc = load_pdf_scale<D>(inv_bw, inv_r, mode, n);
  const int sub = threadIdx.x & (G - 1);
  const int64_t c = (int64_t)blockIdx.x * (kPdfThreads / G) + threadIdx.x / G;
  if (c >= n) return;
  float p[D], own[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    p[d] = pts[c * D + d];
    own[d] = 0.0f;
  }
  const float up = pdf_grads[c];
  const int64_t a = c > 0 ? ranges[c - 1] : 0, b = ranges[c];
  for (int64_t m = a + sub; m < b; m += G) {
    const int64_t j = nbrs[m].x;
    if (j == c) continue;                     // zero offset: no gradient either way
    float u[D], e = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      u[d] = (pts[j * D + d] - p[d]) * sc.s[d];
      e += u[d] * u[d];
    }
    const float kern = sc.norm * expf(-0.5f * e);
    // is c among the neighbours of j?
    const int aj = j > 0 ? ranges[j - 1] : 0, bj = ranges[j];
    int lo = aj, hi = bj;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (nbrs[mid].x < (int)c) lo = mid + 1; else hi = mid;
    }
    bool found = lo < bj && nbrs[lo].x == (int)c;
    if (!found)
      for (int t = aj; t < bj && !found; ++t) found = nbrs[t].x == (int)c;
    const float mine = up * kern, theirs = found ? pdf_grads[j] * kern : 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const float w = u[d] * sc.s[d];
      own[d] += w * (mine + theirs);
      if (!found) unsafeAtomicAdd(&grads[j * D + d], -(w * mine));
    }
  }
#pragma unroll
  for (int d = 0; d < D; ++d) {
    float v = own[d];
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    if (sub == 0) unsafeAtomicAdd(&grads[c * D + d], v);
  }
}

// The same gradient when the pair table is symmetric (j in N(c) <=> c in N(j), as
// in an untruncated self-neighbourhood: the distance test is exact under
// negation).  The term centre j adds to grad[c] through its pair (c, j) equals
// pdf_grad_j * k_cj * u_cj * s, so
//   grad[c] = sum_{j in N(c)} (pdf_grad_c + pdf_grad_j) * k_cj * u_cj * s
// is a pure gather: no atomics, no zero fill, fixed summation order.
template <int D, int G>
__global__ void __launch_bounds__(kPdfThreads) compute_pdf_grads_symmetric_kernel(
    int64_t n, const float *__restrict__ pts, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, const float *__restrict__ inv_bw,
    const float *__restrict__ inv_r, const float *__restrict__ pdf_grads, int mode,
    float *__restrict__ grads) {
  const PdfScale<D> sc = load_pdf_scale<D>(inv_bw, inv_r, mode, n);
  const int sub = threadIdx.x & (G - 1);
  const int64_t c = (int64_t)blockIdx.x * (kPdfThreads / G) + threadIdx.x / G;
  if (c >= n) return;
  float p[D], own[D];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    p[d] = pts[c * D + d];
    own[d] = 0.0f;
  }
  const float up = pdf_grads[c];
  const int64_t a = c > 0 ? ranges[c - 1] : 0, b = ranges[c];
  for (int64_t m = a + sub; m < b; m += G) {
    const int64_t j = nbrs[m].x;
    float u[D], e = 0.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) {
      u[d] = (pts[j * D + d] - p[d]) * sc.s[d];
      e += u[d] * u[d];
    }
    const float local = (up + pdf_grads[j]) * sc.norm * expf(-0.5f * e);
#pragma unroll
    for (int d = 0; d < D; ++d) own[d] += u[d] * sc.s[d] * local;
  }
#pragma unroll
  for (int d = 0; d < D; ++d) {
    float v = own[d];
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    if (sub == 0) grads[c * D + d] = v;
  }
}

static int check_pdf_args(const char *op, int64_t num_pts, int num_dims, int neighbors_rank,
                          int neighbors_cols, int64_t num_samples, int inv_bandwidth_len,
                          int inv_radii_len, int mode) {
  MCCNN_REQUIRE(mode >= 0 && mode < 2, "%s requires a mode between 0 and 1", op);
  MCCNN_REQUIRE(num_samples == num_pts, "%s expects the same points as samples", op);
  MCCNN_REQUIRE(valid_dims(num_dims), "%s expects a valid number of dimensions", op);
  MCCNN_REQUIRE(inv_bandwidth_len == num_dims,
                "%s expects a number of dimensions in inv_bandwidth equal to the number of "
                "dimensions in the input points", op);
  MCCNN_REQUIRE(inv_radii_len == num_dims,
                "%s expects a number of dimensions in inv_radii equal to the number of dimensions "
                "in the input points", op);
  MCCNN_REQUIRE(neighbors_rank == 2 && neighbors_cols == 2,
                "%s expects a neighbor tensor with 2 dimensions and 2 indices per neighbor", op);
  return MCCNN_OK;
}

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_compute_pdf(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                                 const float *points, int64_t num_neighbors, int neighbors_rank,
                                 int neighbors_cols, const int32_t *neighbors,
                                 int64_t num_samples, const int32_t *ranges,
                                 int inv_bandwidth_len, const float *inv_bandwidth,
                                 int inv_radii_len, const float *inv_radii, int mode,
                                 float *pdf_out) {
  int rc = check_pdf_args("ComputePdf", num_pts, num_dims, neighbors_rank, neighbors_cols,
                          num_samples, inv_bandwidth_len, inv_radii_len, mode);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(num_pts >= 0 && num_neighbors >= 0, "ComputePdf expects non-negative sizes");
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points && ranges && inv_bandwidth && inv_radii && pdf_out &&
                    (neighbors || num_neighbors == 0),
                "ComputePdf received a null tensor");
#ifdef MCCNN_PROBE_STAGED_PDF
  MCCNN_DIM_SWITCH(num_dims,
                   hipLaunchKernelGGL(compute_pdf_staged_kernel<D>,
                                      dim3(blocks_for(num_pts, kPdfThreads / 8)),
                                      dim3(kPdfThreads), 0, as_stream(stream), num_pts, points,
                                      (const int2 *)neighbors, ranges, inv_bandwidth, inv_radii,
                                      mode, pdf_out));
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
#endif
  // lanes per centre by the mean length of a list
  const int64_t mean = num_neighbors / num_pts;
#define MCCNN_PDF_LAUNCH(G_)                                                                   \
  MCCNN_DIM_SWITCH(num_dims,                                                                   \
                   hipLaunchKernelGGL((compute_pdf_kernel<D, G_>),                             \
                                      dim3(blocks_for(num_pts, kPdfThreads / G_)),             \
                                      dim3(kPdfThreads), 0, as_stream(stream), num_pts, points, \
                                      (const int2 *)neighbors, ranges, inv_bandwidth,          \
                                      inv_radii, mode, pdf_out))
  if (mean <= 16) {
    MCCNN_PDF_LAUNCH(4);
  } else if (mean <= 96) {
    MCCNN_PDF_LAUNCH(8);
  } else {
    MCCNN_PDF_LAUNCH(16);
  }
#undef MCCNN_PDF_LAUNCH
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

static int pdf_pt_grads_impl(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                             const float *points, int64_t num_neighbors, int neighbors_rank,
                             int neighbors_cols, const int32_t *neighbors, int64_t num_samples,
                             const int32_t *ranges, int inv_bandwidth_len,
                             const float *inv_bandwidth, int inv_radii_len,
                             const float *inv_radii, int64_t pdf_grads_len,
                             const float *pdf_grads, int mode, bool symmetric,
                             float *pt_grads_out) {
  int rc = check_pdf_args("ComputePdfPtGrads", num_pts, num_dims, neighbors_rank, neighbors_cols,
                          num_samples, inv_bandwidth_len, inv_radii_len, mode);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(pdf_grads_len == num_samples,
                "ComputePdfPtGrads expects a number of pdf gradients equal to the number of "
                "samples");
  MCCNN_REQUIRE(num_pts >= 0 && num_neighbors >= 0, "ComputePdfPtGrads expects non-negative sizes");
  if (num_pts == 0) return MCCNN_OK;
  MCCNN_REQUIRE(points && ranges && inv_bandwidth && inv_radii && pdf_grads && pt_grads_out &&
                    (neighbors || num_neighbors == 0),
                "ComputePdfPtGrads received a null tensor");
  hipStream_t s = as_stream(stream);
  // lanes per centre by the mean length of a list, as in compute_pdf
  const int64_t mean = num_neighbors / num_pts;
  const int lanes = mean <= 16 ? 4 : mean <= 96 ? 8 : 16;
#define MCCNN_PDF_GRADS_LAUNCH(KERNEL_, G_)                                                    \
  MCCNN_DIM_SWITCH(num_dims,                                                                   \
                   hipLaunchKernelGGL((KERNEL_<D, G_>),                                        \
                                      dim3(blocks_for(num_pts, kPdfThreads / G_)),             \
                                      dim3(kPdfThreads), 0, s, num_pts, points,                \
                                      (const int2 *)neighbors, ranges, inv_bandwidth,          \
                                      inv_radii, pdf_grads, mode, pt_grads_out))
  if (symmetric) {
    if (lanes == 4) {
      MCCNN_PDF_GRADS_LAUNCH(compute_pdf_grads_symmetric_kernel, 4);
    } else if (lanes == 8) {
      MCCNN_PDF_GRADS_LAUNCH(compute_pdf_grads_symmetric_kernel, 8);
    } else {
      MCCNN_PDF_GRADS_LAUNCH(compute_pdf_grads_symmetric_kernel, 16);
    }
    MCCNN_LAUNCH_CHECK();
    return MCCNN_OK;
  }
  rc = fill_zero(s, pt_grads_out, sizeof(float) * (size_t)num_pts * num_dims);
  if (rc != MCCNN_OK) return rc;
  // the look-ups dominate here: 16 lanes stay the better choice for all but short lists
  // (7.5 / 52 pairs per point: 0.108 / 1.148 ms with 4 / 8 lanes, 0.138 / 1.055 ms with 16)
  if (lanes == 4) {
    MCCNN_PDF_GRADS_LAUNCH(compute_pdf_grads_lookup_kernel, 4);
  } else {
    MCCNN_PDF_GRADS_LAUNCH(compute_pdf_grads_lookup_kernel, 16);
  }
#undef MCCNN_PDF_GRADS_LAUNCH
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_compute_pdf_pt_grads(mccnn_stream_t stream, int64_t num_pts, int num_dims,
                                          const float *points, int64_t num_neighbors,
                                          int neighbors_rank, int neighbors_cols,
                                          const int32_t *neighbors, int64_t num_samples,
                                          const int32_t *ranges, int inv_bandwidth_len,
                                          const float *inv_bandwidth, int inv_radii_len,
                                          const float *inv_radii, int64_t pdf_grads_len,
                                          const float *pdf_grads, int mode,
                                          float *pt_grads_out) {
  return pdf_pt_grads_impl(stream, num_pts, num_dims, points, num_neighbors, neighbors_rank,
                           neighbors_cols, neighbors, num_samples, ranges, inv_bandwidth_len,
                           inv_bandwidth, inv_radii_len, inv_radii, pdf_grads_len, pdf_grads, mode,
                           false, pt_grads_out);
}

extern "C" int mccnn_compute_pdf_pt_grads_symmetric(
    mccnn_stream_t stream, int64_t num_pts, int num_dims, const float *points,
    int64_t num_neighbors, int neighbors_rank, int neighbors_cols, const int32_t *neighbors,
    int64_t num_samples, const int32_t *ranges, int inv_bandwidth_len,
    const float *inv_bandwidth, int inv_radii_len, const float *inv_radii,
    int64_t pdf_grads_len, const float *pdf_grads, int mode, float *pt_grads_out) {
  return pdf_pt_grads_impl(stream, num_pts, num_dims, points, num_neighbors, neighbors_rank,
                           neighbors_cols, neighbors, num_samples, ranges, inv_bandwidth_len,
                           inv_bandwidth, inv_radii_len, inv_radii, pdf_grads_len, pdf_grads, mode,
                           true, pt_grads_out);
}
