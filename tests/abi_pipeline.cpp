// Drives the C-ABI of libmccnn_hip.so from plain C++ with hipMalloc'd buffers (no
// Python, no torch): bounding boxes and grid shape, keys, sort, gathers, grid
// table, neighbour search, densities and basis projection on a seeded cloud, each
// stage compared with the CPU oracle (liboracle: test infrastructure, linked only
// here).  Integer outputs must agree exactly, floats within 1e-5 of the magnitude
// sum.  Prints one line per stage and exits non-zero on the first mismatch.
//
// Built by tests/Makefile (from __graft_entry__.build()); run by tests/test_zz_abi_cpp_pipeline.py.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <numeric>
#include <vector>

#include "mccnn_hip.h"

extern "C" {
void orc_compute_keys(int D, int64_t n, const float *pts, const int *bids, const float *saabb_min,
                      const int *nc, const float *inv_cell, int64_t *keys);
void orc_build_grid_ds(int D, int64_t n, const int64_t *sorted_keys, const int *nc,
                       int batch_size, int *ds);
int64_t orc_find_neighbors_count(int D, int64_t ns, const float *samples, const int *sbids,
                                 int64_t n, const float *pts, const int64_t *keys, const int *ds,
                                 const int *nc, const float *saabb_min, const float *inv_cell,
                                 const float *inv_r, int max_neighs, int *ranges);
void orc_find_neighbors_fill(int D, int64_t ns, const float *samples, const int *sbids, int64_t n,
                             const float *pts, const int64_t *keys, const int *ds, const int *nc,
                             const float *saabb_min, const float *inv_cell, const float *inv_r,
                             int max_neighs, const int *ranges, int *nbrs);
void orc_compute_pdf(int D, int64_t n, const float *pts, const int *nbrs, const int *ranges,
                     const float *inv_bw, const float *inv_r, int mode, double *pdf);
void orc_basis_proj(int64_t n_out, int C, int K, const float *basis, const float *feat,
                    const int *nbrs, const int *ranges, double *out, double *mag);
}

#define HIP_OK(x)                                                                      \
  do {                                                                                 \
    hipError_t e_ = (x);                                                               \
    if (e_ != hipSuccess) {                                                            \
      std::printf("FAILED %s: %s (line %d)\n", #x, hipGetErrorString(e_), __LINE__);   \
      std::exit(2);                                                                    \
    }                                                                                  \
  } while (0)
#define OP_OK(x)                                                                       \
  do {                                                                                 \
    int rc_ = (x);                                                                     \
    if (rc_ != 0) {                                                                    \
      std::printf("FAILED %s: status %d, %s (line %d)\n", #x, rc_, mccnn_last_error(), \
                  __LINE__);                                                           \
      std::exit(2);                                                                    \
    }                                                                                  \
  } while (0)

template <class T>
static T *to_device(const std::vector<T> &v) {
  T *p = nullptr;
  HIP_OK(hipMalloc(&p, std::max<size_t>(v.size(), 1) * sizeof(T)));
  if (!v.empty()) HIP_OK(hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  return p;
}
template <class T>
static T *device_alloc(size_t n) {
  T *p = nullptr;
  HIP_OK(hipMalloc(&p, std::max<size_t>(n, 1) * sizeof(T)));
  return p;
}
template <class T>
static std::vector<T> to_host(const T *p, size_t n) {
  std::vector<T> v(n);
  if (n) HIP_OK(hipMemcpy(v.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
  return v;
}

template <class T>
static void expect_equal(const char *stage, const std::vector<T> &got, const std::vector<T> &want) {
  if (got.size() != want.size()) {
    std::printf("MISMATCH %s: %zu values, expected %zu\n", stage, got.size(), want.size());
    std::exit(1);
  }
  for (size_t i = 0; i < got.size(); ++i)
    if (got[i] != want[i]) {
      std::printf("MISMATCH %s at %zu: %lld, expected %lld\n", stage, i, (long long)got[i],
                  (long long)want[i]);
      std::exit(1);
    }
  std::printf("%-22s %10zu values bit-exact\n", stage, got.size());
}

static void expect_close(const char *stage, const std::vector<float> &got,
                         const std::vector<double> &want, const std::vector<double> &mag) {
  double worst = 0.0;
  for (size_t i = 0; i < got.size(); ++i) {
    const double m = mag.empty() ? std::fabs(want[i]) : mag[i];
    const double err = std::fabs((double)got[i] - want[i]);
    if (err > 1e-5 * m + 1e-30) {
      std::printf("MISMATCH %s at %zu: %.9g, expected %.9g (magnitude %.3g)\n", stage, i,
                  (double)got[i], want[i], m);
      std::exit(1);
    }
    if (m > 0.0) worst = std::max(worst, err / m);
  }
  std::printf("%-22s %10zu values, worst relative error %.2e\n", stage, got.size(), worst);
}

int main() {
  const int D = 3, B = 3, C = 16, K = 16;
  const int64_t N = 30000;
  const float radius = 0.07f;
  if (mccnn_abi_version() != 1) { std::printf("unexpected ABI version\n"); return 1; }

  // seeded cloud: uniform points, clouds of unequal size, some exact duplicates
  uint64_t state = 0x9E3779B97F4A7C15ull;
  auto rnd = [&]() {
    state = state * 6364136223846793005ull + 1442695040888963407ull;
    return (uint32_t)(state >> 40);                       // 24 bits
  };
  std::vector<float> pts(N * D), feat(N * C);
  std::vector<int> bids(N);
  for (int64_t i = 0; i < N; ++i) {
    bids[i] = i < B ? (int)i : (int)(rnd() % 4 % B);      // clouds of about 1/2, 1/4, 1/4 of the points
    for (int d = 0; d < D; ++d) pts[i * D + d] = (float)rnd() / 16777216.0f;
  }
  for (int64_t i = 100; i < 120; ++i)
    for (int d = 0; d < D; ++d) pts[i * D + d] = pts[(i - 50) * D + d];
  for (auto &f : feat) f = (float)rnd() / 8388608.0f - 1.0f;

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  float *d_pts = to_device(pts);
  int *d_bids = to_device(bids);
  std::vector<float> cell(D, radius), inv_r(D, 1.0f / radius), inv_bw(D, 1.0f / 0.2f);
  float *d_cell = to_device(cell), *d_inv_r = to_device(inv_r), *d_inv_bw = to_device(inv_bw);

  // ---- bounding boxes and grid shape
  float *d_amin = device_alloc<float>(B * D), *d_amax = device_alloc<float>(B * D);
  float *d_smin = device_alloc<float>(B * D), *d_inv_cell = device_alloc<float>(D);
  int *d_nc = device_alloc<int>(D);
  OP_OK(mccnn_grid_setup(stream, N, D, d_pts, d_bids, B, d_cell, d_amin, d_amax, d_nc, d_smin,
                         d_inv_cell));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<int> nc = to_host(d_nc, D);
  std::vector<float> smin = to_host(d_smin, B * D), inv_cell = to_host(d_inv_cell, D);
  {
    // PointCloud.py:38-43, Grid.py:44-48, custom_ops_wrapper.py:37-43 on the host
    std::vector<float> lo(B * D, INFINITY), hi(B * D, -INFINITY);
    for (int64_t i = 0; i < N; ++i)
      for (int d = 0; d < D; ++d) {
        lo[bids[i] * D + d] = std::min(lo[bids[i] * D + d], pts[i * D + d]);
        hi[bids[i] * D + d] = std::max(hi[bids[i] * D + d], pts[i * D + d]);
      }
    std::vector<int> want_nc(D, 1);
    std::vector<float> want_smin(B * D), want_inv(D);
    for (int b = 0; b < B; ++b)
      for (int d = 0; d < D; ++d) {
        const float mn = lo[b * D + d] - 1e-9f, mx = hi[b * D + d] + 1e-9f;
        want_nc[d] = std::max(want_nc[d], (int)std::ceil((mx - mn) / cell[d]));
        want_smin[b * D + d] = mn / cell[d];
      }
    for (int d = 0; d < D; ++d) want_inv[d] = 1.0f / cell[d];
    expect_equal("num_cells", nc, want_nc);
    expect_equal("scaled_aabb_min bits",
                 std::vector<int32_t>((int32_t *)smin.data(), (int32_t *)smin.data() + B * D),
                 std::vector<int32_t>((int32_t *)want_smin.data(),
                                      (int32_t *)want_smin.data() + B * D));
    expect_equal("inv_cell_sizes bits",
                 std::vector<int32_t>((int32_t *)inv_cell.data(), (int32_t *)inv_cell.data() + D),
                 std::vector<int32_t>((int32_t *)want_inv.data(), (int32_t *)want_inv.data() + D));
  }

  // ---- keys
  int64_t *d_keys = device_alloc<int64_t>(N);
  OP_OK(mccnn_compute_keys(stream, N, D, d_pts, N, d_bids, B, D, d_smin, D, d_nc, D, d_inv_cell,
                           d_keys));
  std::vector<int64_t> want_keys(N);
  orc_compute_keys(D, N, pts.data(), bids.data(), smin.data(), nc.data(), inv_cell.data(),
                   want_keys.data());
  HIP_OK(hipStreamSynchronize(stream));
  expect_equal("compute_keys", to_host(d_keys, N), want_keys);

  // ---- stable descending sort and the gathers
  int64_t total_cells = B;
  for (int d = 0; d < D; ++d) total_cells *= nc[d];
  int key_bits = 1;
  while (key_bits < 64 && (total_cells >> key_bits) != 0) ++key_bits;
  int64_t *d_skeys = device_alloc<int64_t>(N);
  int *d_sidx = device_alloc<int>(N);
  const size_t sort_bytes = mccnn_sort_keys_workspace_bytes(N);
  void *d_sort_ws = device_alloc<char>(sort_bytes);
  OP_OK(mccnn_sort_keys_descending(stream, N, key_bits, d_keys, d_skeys, d_sidx, d_sort_ws,
                                   sort_bytes));
  float *d_spts = device_alloc<float>(N * D);
  int *d_sbids = device_alloc<int>(N);
  OP_OK(mccnn_gather_points(stream, N, D, d_pts, d_bids, d_sidx, d_spts, d_sbids));
  std::vector<int> order(N);
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(),
                   [&](int a, int b) { return want_keys[a] > want_keys[b]; });
  std::vector<int64_t> skeys(N);
  std::vector<float> spts(N * D);
  std::vector<int> sbids(N);
  for (int64_t i = 0; i < N; ++i) {
    skeys[i] = want_keys[order[i]];
    sbids[i] = bids[order[i]];
    for (int d = 0; d < D; ++d) spts[i * D + d] = pts[(int64_t)order[i] * D + d];
  }
  HIP_OK(hipStreamSynchronize(stream));
  expect_equal("sorted_indices", to_host(d_sidx, N), order);
  expect_equal("sorted_keys", to_host(d_skeys, N), skeys);
  expect_equal("sorted_batch_ids", to_host(d_sbids, N), sbids);

  // ---- grid table
  const size_t ds_len = (size_t)B * nc[0] * nc[1] * 2;
  int *d_ds = device_alloc<int>(ds_len);
  OP_OK(mccnn_build_grid_ds(stream, N, d_skeys, D, d_nc, D, nc.data(), B, d_ds));
  std::vector<int> ds(ds_len);
  orc_build_grid_ds(D, N, skeys.data(), nc.data(), B, ds.data());
  HIP_OK(hipStreamSynchronize(stream));
  expect_equal("build_grid_ds", to_host(d_ds, ds_len), ds);

  // ---- neighbours of the sorted points among themselves
  const size_t nb_bytes = mccnn_find_neighbors_workspace_bytes(D, N);
  void *d_nb_ws = device_alloc<char>(nb_bytes);
  int *d_ranges = device_alloc<int>(N);
  int64_t M = -1;
  OP_OK(mccnn_find_neighbors_count(stream, N, D, d_spts, N, d_sbids, N, D, d_spts, N, d_skeys, 4,
                                   B, nc[0], nc[1], 2, d_ds, D, d_nc, D, d_smin, D, d_inv_cell, D,
                                   d_inv_r, 0, d_nb_ws, nb_bytes, d_ranges, &M));
  std::vector<int> ranges(N);
  const int64_t want_m = orc_find_neighbors_count(D, N, spts.data(), sbids.data(), N, spts.data(),
                                                  skeys.data(), ds.data(), nc.data(), smin.data(),
                                                  inv_cell.data(), inv_r.data(), 0, ranges.data());
  if (M != want_m) { std::printf("MISMATCH pair count %lld, expected %lld\n", (long long)M, (long long)want_m); return 1; }
  int *d_nbrs = device_alloc<int>(2 * M);
  OP_OK(mccnn_find_neighbors_fill(stream, N, D, d_spts, d_sbids, N, d_spts, d_skeys, d_ds, d_nc,
                                  d_smin, d_inv_cell, d_inv_r, 0, d_nb_ws, nb_bytes, d_ranges, M,
                                  d_nbrs));
  std::vector<int> nbrs(2 * M);
  orc_find_neighbors_fill(D, N, spts.data(), sbids.data(), N, spts.data(), skeys.data(), ds.data(),
                          nc.data(), smin.data(), inv_cell.data(), inv_r.data(), 0, ranges.data(),
                          nbrs.data());
  HIP_OK(hipStreamSynchronize(stream));
  expect_equal("neighbour ranges", to_host(d_ranges, N), ranges);
  expect_equal("neighbour pairs", to_host(d_nbrs, 2 * M), nbrs);

  // ---- densities
  float *d_pdf = device_alloc<float>(N);
  OP_OK(mccnn_compute_pdf(stream, N, D, d_spts, M, 2, 2, d_nbrs, N, d_ranges, D, d_inv_bw, D,
                          d_inv_r, 0, d_pdf));
  std::vector<double> pdf(N);
  orc_compute_pdf(D, N, spts.data(), nbrs.data(), ranges.data(), inv_bw.data(), inv_r.data(), 0,
                  pdf.data());
  HIP_OK(hipStreamSynchronize(stream));
  expect_close("compute_pdf", to_host(d_pdf, N), pdf, {});

  // ---- basis projection (features addressed by sorted index here)
  std::vector<float> basis(M * K);
  for (auto &w : basis) w = (float)rnd() / 8388608.0f - 1.0f;
  float *d_basis = to_device(basis), *d_feat = to_device(feat);
  float *d_out = device_alloc<float>(N * C * K);
  OP_OK(mccnn_basis_proj(stream, M, K, d_basis, N, C, d_feat, M, 2, 2, d_nbrs, N, d_ranges, d_out));
  std::vector<double> want_out(N * C * K), mag(N * C * K);
  orc_basis_proj(N, C, K, basis.data(), feat.data(), nbrs.data(), ranges.data(), want_out.data(),
                 mag.data());
  HIP_OK(hipStreamSynchronize(stream));
  expect_close("basis_proj", to_host(d_out, N * C * K), want_out, mag);

  // an invalid call comes back as a status with a message, and the library keeps working
  if (mccnn_basis_proj(stream, M, 12, d_basis, N, C, d_feat, M, 2, 2, d_nbrs, N, d_ranges, d_out) != 1) {
    std::printf("MISMATCH: K = 12 was not refused\n");
    return 1;
  }
  std::printf("refused call reports: %s\n", mccnn_last_error());
  HIP_OK(hipStreamDestroy(stream));
  std::printf("abi_pipeline ok: %lld points, %lld pairs\n", (long long)N, (long long)M);
  return 0;
}
