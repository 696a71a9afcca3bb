/*
 * CPU oracle for the MCCNN custom-op path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithms of the reference's native
 * ops (custom_ops/tfg_custom_ops/...) and the ordering rules of its pure-TF
 * fall-backs (pylib/pc/custom_ops/custom_ops_tf.py).  It exists so that the
 * HIP kernels can be checked against it and so that a host-CPU figure can be
 * reported beside the GPU one.  Nothing that ships may call into it: only the
 * test-suite, the smoke check and the cpu-baseline leg of the benchmark do.
 *
 * Conventions
 *   - all arrays are row-major and contiguous; keys are int64, indices int32.
 *   - "ranges" are the inclusive END offsets per centre (find_neighbors_ops.cpp
 *     output 0): the pairs of centre i are [ranges[i-1], ranges[i]) with
 *     ranges[-1] == 0.
 *   - integer-deciding float expressions are evaluated in fp32 with one
 *     rounding per operation (compile with -ffp-contract=off).
 *   - float-valued results (pdf, basis projection, gradients) are accumulated
 *     in double from the fp32 inputs; tests compare the fp32 GPU results against
 *     them with a stated tolerance.
 *
 * Pinning of each function (what independent check fixes it) is listed in the
 * comment above the function; the checks live in tests/test_oracle_*.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_MAX_D 6

/* ------------------------------------------------------------------------- */
/* grid arithmetic: shared/cc/kernels/grid_utils.h:63-143                     */
/* ------------------------------------------------------------------------- */

/* grid_utils.h:63-74 : rel = p*invCell - sMin (two roundings), floorf, clamp
 * to [0, n-1]. */
static void orc_cell_of_point(int D, const float *p, const float *smin,
                              const int *nc, const float *inv_cell, int *cell) {
  for (int d = 0; d < D; ++d) {
    float prod = p[d] * inv_cell[d];
    float rel = prod - smin[d];
    int c = (int)floorf(rel);
    if (c < 0) c = 0;
    if (c > nc[d] - 1) c = nc[d] - 1;
    cell[d] = c;
  }
}

/* grid_utils.h:85-100 : row-major key with the batch id as the top digit. */
static int64_t orc_key_of_cell(int D, const int *cell, const int *nc, int b) {
  int64_t key = 0, accum = 1;
  for (int d = D - 1; d >= 0; --d) {
    key += (int64_t)cell[d] * accum;
    accum *= nc[d];
  }
  return key + accum * (int64_t)b;
}

/* grid_utils.h:109-125 : out[0] = batch id, out[1..D] = cell. */
static void orc_cell_of_key(int D, int64_t key, const int *nc, int *out) {
  int64_t aux = key;
  for (int d = D - 1; d >= 0; --d) {
    out[d + 1] = (int)(aux % nc[d]);
    aux = aux / nc[d];
  }
  out[0] = (int)aux;
}

static int64_t orc_total_cells(int D, const int *nc) {
  int64_t t = 1;
  for (int d = 0; d < D; ++d) t *= nc[d];
  return t;
}

/* compute_keys_kernels.cu.cc:40-71.
 * Pinned by: the numpy formula of compute_keys_tf_test.py:59-70 on inputs with
 * dyadic cell sizes, the invariants 0 <= key < B*prod(n) and key / prod(n) ==
 * batch id, and hand-computed keys. */
void orc_compute_keys(int D, int64_t n, const float *pts, const int *bids,
                      const float *saabb_min, const int *nc,
                      const float *inv_cell, int64_t *keys) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    int cell[ORC_MAX_D];
    int b = bids[i];
    orc_cell_of_point(D, pts + i * D, saabb_min + (int64_t)b * D, nc, inv_cell,
                      cell);
    keys[i] = orc_key_of_cell(D, cell, nc, b);
  }
}

/* build_grid_ds_kernels.cu.cc:37-71 (after the memset of :104).
 * ds is [B, n0, n1, 2]; (first, last+1) per column, (0,0) when empty.
 * Pinned by: the numpy loop of build_grid_ds_tf_test.py:61-93. */
void orc_build_grid_ds(int D, int64_t n, const int64_t *sorted_keys,
                       const int *nc, int batch_size, int *ds) {
  int64_t div = 1;
  for (int d = 2; d < D; ++d) div *= nc[d];
  int64_t ncol = (int64_t)batch_size * nc[0] * nc[1];
  memset(ds, 0, sizeof(int) * 2 * (size_t)ncol);
  for (int64_t i = 0; i < n; ++i) {
    int64_t col = sorted_keys[i] / div;
    if (i > 0 && sorted_keys[i - 1] / div != col) ds[2 * col] = (int)i;
    if (i + 1 == n || sorted_keys[i + 1] / div != col)
      ds[2 * col + 1] = (int)(i + 1);
  }
}

/* ------------------------------------------------------------------------- */
/* find_neighbors                                                             */
/* ------------------------------------------------------------------------- */

/* count_neighbors_kernels.cu.cc:83-86 with math_helper.h:311-327:
 * length((s - p) * invRadii) < 1.0f, dot accumulated in dimension order. */
static int orc_within(int D, const float *s, const float *p,
                      const float *inv_r) {
  float acc = 0.0f;
  for (int d = 0; d < D; ++d) {
    float diff = s[d] - p[d];
    float sc = diff * inv_r[d];
    float sq = sc * sc;
    acc = acc + sq;
  }
  return sqrtf(acc) < 1.0f;
}

/* Candidate index range of one offset for one centre.
 * find_ranges_grid_ds_kernels.cu.cc:48-169 (D > 2) and :184-235 (D == 2):
 * the column (b, c0, c1) of the 2-D table, narrowed (D > 2) to the keys of the
 * last-dimension cells w-1..w+1 of that row.  Keys are sorted in descending
 * order.  Returns 0 when the range is empty. */
static int orc_offset_range(int D, const int *ccell /*D+1: b,cell*/,
                            const int *off, const int64_t *keys, const int *ds,
                            const int *nc, int64_t total_cells, int *lo,
                            int *hi) {
  int cell[ORC_MAX_D + 1];
  cell[0] = ccell[0];
  for (int d = 0; d < D; ++d) cell[d + 1] = ccell[d + 1] + off[d];
  int ndim_check = (D > 2) ? D - 1 : D;
  for (int d = 0; d < ndim_check; ++d)
    if (cell[d + 1] < 0 || cell[d + 1] >= nc[d]) return 0;
  int64_t col = (int64_t)cell[0] * nc[0] * nc[1] + (int64_t)cell[1] * nc[1] +
                cell[2];
  int x = ds[2 * col], y = ds[2 * col + 1];
  if (y - x - 1 < 0) return 0;
  if (D == 2) {
    *lo = x;
    *hi = y;
    return 1;
  }
  /* The reference searches the keys in [aux-1, aux+1] clipped to the batch
   * (:101-107).  Inside a column that is the last-dimension cells w-1..w+1,
   * except that at w == 0 or w == n-1 the +-1 step leaves the row: for D == 3
   * it leaves the column too (no effect), for D > 3 it would pick up a
   * non-adjacent cell of the same column, and with n_last <= 2 the same cell
   * twice.  The step is therefore clamped to the row here; identical to the
   * reference for D <= 3 and for D > 3 whenever cell size >= radius and
   * n_last > 2. */
  int64_t aux = orc_key_of_cell(D, cell + 1, nc, cell[0]);
  int w = cell[D];
  int64_t maxk = aux + (w < nc[D - 1] - 1 ? 1 : 0);
  int64_t mink = aux - (w > 0 ? 1 : 0);
  (void)total_cells;
  /* first index in [x,y) with key <= maxk */
  int a = x, b = y;
  while (a < b) {
    int m = a + (b - a) / 2;
    if (keys[m] > maxk) a = m + 1; else b = m;
  }
  int first = a;
  /* first index in [x,y) with key < mink */
  a = first; b = y;
  while (a < b) {
    int m = a + (b - a) / 2;
    if (keys[m] >= mink) a = m + 1; else b = m;
  }
  if (a <= first) return 0;
  *lo = first;
  *hi = a;
  return 1;
}

/* Number of offsets and the offsets themselves, ordered so that the candidate
 * ranges come out in ascending index order of the (descending-key) sorted
 * array: lexicographically descending in (o_0, o_1, ...).  The offset set is
 * the one of computeTotalNumOffsets (find_ranges_grid_ds_kernels.cu.cc:303-335):
 * {-1,0,1} on dims 0..max(D-2,1), zero on the last dim when D != 2. */
static int orc_offsets(int D, int *offs /* [243][ORC_MAX_D] */) {
  int nd = (D - 2 > 1 ? D - 2 : 1) + 1;
  int total = 1;
  for (int i = 0; i < nd; ++i) total *= 3;
  for (int i = 0; i < total; ++i) {
    int aux = i;
    int *o = offs + i * ORC_MAX_D;
    for (int d = 0; d < ORC_MAX_D; ++d) o[d] = 0;
    for (int d = nd - 1; d >= 0; --d) {
      o[d] = 1 - (aux % 3);
      aux /= 3;
    }
  }
  return total;
}

static int orc_visit_neighbors(int D, const float *s, int sb,
                               const float *pts, const int64_t *keys,
                               const int *ds, const int *nc,
                               const float *saabb_min, const float *inv_cell,
                               const float *inv_r, const int *offs, int noffs,
                               int64_t total_cells, int limit, int *out,
                               int centre) {
  int cell[ORC_MAX_D], ccell[ORC_MAX_D + 1];
  orc_cell_of_point(D, s, saabb_min + (int64_t)sb * D, nc, inv_cell, cell);
  /* the reference goes through the key and back (find_neighbors_ops.cpp:172-175,
   * find_ranges_grid_ds_kernels.cu.cc:79-80): identical for valid batch ids. */
  int64_t key = orc_key_of_cell(D, cell, nc, sb);
  orc_cell_of_key(D, key, nc, ccell);
  int count = 0;
  for (int o = 0; o < noffs; ++o) {
    int lo, hi;
    if (!orc_offset_range(D, ccell, offs + o * ORC_MAX_D, keys, ds, nc,
                          total_cells, &lo, &hi))
      continue;
    for (int j = lo; j < hi; ++j) {
      if (orc_within(D, s, pts + (int64_t)j * D, inv_r)) {
        if (limit > 0 && count >= limit) return count;
        if (out) {
          out[2 * count] = j;
          out[2 * count + 1] = centre;
        }
        ++count;
      }
    }
  }
  return count;
}

/* find_neighbors_ops.cpp:86-250 (keys of the centres, ranges, count, clamp,
 * scan).  Writes the inclusive end offsets into `ranges` and returns M.
 * max_neighs > 0 keeps the FIRST max_neighs neighbours in canonical order (the
 * reference's choice is seeded by the wall clock, store_neighbors_kernels.cu.cc:216).
 * Pinned by: the lattice known-answer test 1/7/19/27 of
 * find_neighbors_tf_test.py:28-61, brute force over all pairs, and
 * scipy.spatial.cKDTree on boundary-safe inputs. */
int64_t orc_find_neighbors_count(int D, int64_t ns, const float *samples,
                                 const int *sbids, int64_t n, const float *pts,
                                 const int64_t *keys, const int *ds,
                                 const int *nc, const float *saabb_min,
                                 const float *inv_cell, const float *inv_r,
                                 int max_neighs, int *ranges) {
  (void)n;
  int offs[243 * ORC_MAX_D];
  int noffs = orc_offsets(D, offs);
  int64_t total_cells = orc_total_cells(D, nc);
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < ns; ++i)
    ranges[i] = orc_visit_neighbors(D, samples + i * D, sbids[i], pts, keys, ds,
                                    nc, saabb_min, inv_cell, inv_r, offs, noffs,
                                    total_cells, max_neighs, NULL, (int)i);
  int64_t acc = 0;
  for (int64_t i = 0; i < ns; ++i) {
    acc += ranges[i];
    ranges[i] = (int)acc;
  }
  return acc;
}

/* store_neighbors_kernels.cu.cc:127-169, with the within-centre order fixed to
 * ascending sorted-point index (custom_ops_tf.py:201-205). nbrs is [M,2] rows
 * (sorted point index, centre index). */
void orc_find_neighbors_fill(int D, int64_t ns, const float *samples,
                             const int *sbids, int64_t n, const float *pts,
                             const int64_t *keys, const int *ds, const int *nc,
                             const float *saabb_min, const float *inv_cell,
                             const float *inv_r, int max_neighs,
                             const int *ranges, int *nbrs) {
  (void)n;
  int offs[243 * ORC_MAX_D];
  int noffs = orc_offsets(D, offs);
  int64_t total_cells = orc_total_cells(D, nc);
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < ns; ++i) {
    int64_t start = i ? ranges[i - 1] : 0;
    orc_visit_neighbors(D, samples + i * D, sbids[i], pts, keys, ds, nc,
                        saabb_min, inv_cell, inv_r, offs, noffs, total_cells,
                        max_neighs, nbrs + 2 * start, (int)i);
  }
}

/* ------------------------------------------------------------------------- */
/* compute_pdf                                                                */
/* ------------------------------------------------------------------------- */

/* compute_pdf_kernels.cu.cc:72-130.  mode 0: bandwidth = inv_bw; mode 1: the
 * reference passes the number of samples, so bandwidth = sqrt(n) in every
 * dimension (:56, :102).  Result in double.
 * Pinned by: sklearn.neighbors.KernelDensity as in compute_pdf_test.py:76-108,
 * and the closed form for a two-point cloud. */
void orc_compute_pdf(int D, int64_t n, const float *pts, const int *nbrs,
                     const int *ranges, const float *inv_bw, const float *inv_r,
                     int mode, double *pdf) {
  double bw[ORC_MAX_D];
  for (int d = 0; d < D; ++d)
    bw[d] = mode == 0 ? (double)inv_bw[d] : (double)sqrtf((float)n);
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t i = 0; i < n; ++i) {
    int64_t a = i ? ranges[i - 1] : 0, b = ranges[i];
    double acc = 0.0;
    for (int64_t m = a; m < b; ++m) {
      const float *q = pts + (int64_t)nbrs[2 * m] * D;
      double local = 1.0;
      for (int d = 0; d < D; ++d) {
        double u = ((double)q[d] - (double)pts[i * D + d]) * bw[d] *
                   (double)inv_r[d];
        local *= bw[d] * exp(-0.5 * u * u) * 0.3989422804014327;
      }
      acc += local;
    }
    pdf[i] = acc;
  }
}

/* compute_pdf_kernels.cu.cc:148-215: grad[i] += g, grad[j] -= g with
 * g_d = pdf_grad_i * pdf_ij * u_d * bw_d * inv_r_d.  Result in double [n,D].
 * Pinned by: central differences of orc_compute_pdf and autograd of a float64
 * torch restatement of the KDE sum. */
void orc_compute_pdf_pt_grads(int D, int64_t n, const float *pts,
                              const int *nbrs, const int *ranges,
                              const float *inv_bw, const float *inv_r,
                              const float *pdf_grads, int mode, double *grads) {
  double bw[ORC_MAX_D];
  for (int d = 0; d < D; ++d)
    bw[d] = mode == 0 ? (double)inv_bw[d] : (double)sqrtf((float)n);
  memset(grads, 0, sizeof(double) * (size_t)n * D);
  for (int64_t i = 0; i < n; ++i) {
    int64_t a = i ? ranges[i - 1] : 0, b = ranges[i];
    for (int64_t m = a; m < b; ++m) {
      int64_t j = nbrs[2 * m];
      double u[ORC_MAX_D], local = (double)pdf_grads[i];
      for (int d = 0; d < D; ++d) {
        u[d] = ((double)pts[j * D + d] - (double)pts[i * D + d]) * bw[d] *
               (double)inv_r[d];
        local *= bw[d] * exp(-0.5 * u[d] * u[d]) * 0.3989422804014327;
      }
      for (int d = 0; d < D; ++d) {
        double g = u[d] * bw[d] * (double)inv_r[d] * local;
        grads[i * D + d] += g;
        grads[j * D + d] -= g;
      }
    }
  }
}

/* ------------------------------------------------------------------------- */
/* basis_proj                                                                 */
/* ------------------------------------------------------------------------- */

/* basis_proj_kernels.cu.cc:29-127: out[i,c,k] = sum_m feat[nbr_m,c]*basis[m,k].
 * `mag` (may be NULL) receives sum_m |feat*basis|, the scale against which a
 * relative error of an fp32 sum is meaningful.
 * Pinned by: the numpy segment sum of basis_proj_test.py:88-111 and
 * numpy.einsum on padded neighbourhoods. */
void orc_basis_proj(int64_t n_out, int C, int K, const float *basis,
                    const float *feat, const int *nbrs, const int *ranges,
                    double *out, double *mag) {
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t i = 0; i < n_out; ++i) {
    int64_t a = i ? ranges[i - 1] : 0, b = ranges[i];
    double *o = out + i * C * K;
    double *g = mag ? mag + i * C * K : NULL;
    for (int e = 0; e < C * K; ++e) o[e] = 0.0;
    if (g) for (int e = 0; e < C * K; ++e) g[e] = 0.0;
    for (int64_t m = a; m < b; ++m) {
      const float *f = feat + (int64_t)nbrs[2 * m] * C;
      const float *w = basis + m * K;
      for (int c = 0; c < C; ++c)
        for (int k = 0; k < K; ++k) {
          double t = (double)f[c] * (double)w[k];
          o[c * K + k] += t;
          if (g) g[c * K + k] += fabs(t);
        }
    }
  }
}

/* basis_proj_grads_kernels.cu.cc:29-151:
 *   dbasis[m,k] = sum_c g[i,c,k]*feat[nbr_m,c]
 *   dfeat[n,c]  = sum_{m: nbr_m == n} sum_k g[i,c,k]*basis[m,k]
 * Pinned by: torch.autograd of a float64 restatement of the forward sum and by
 * the adjoint identity <g, proj(basis,feat)> == <dbasis, basis> == <dfeat, feat>. */
void orc_basis_proj_grads(int64_t n_in, int64_t n_out, int C, int K,
                          const float *basis, const float *feat,
                          const int *nbrs, const int *ranges,
                          const float *in_grad, double *dbasis,
                          double *dfeat) {
  memset(dfeat, 0, sizeof(double) * (size_t)n_in * C);
  for (int64_t i = 0; i < n_out; ++i) {
    int64_t a = i ? ranges[i - 1] : 0, b = ranges[i];
    const float *g = in_grad + i * C * K;
    for (int64_t m = a; m < b; ++m) {
      int64_t nb = nbrs[2 * m];
      const float *f = feat + nb * C;
      const float *w = basis + m * K;
      double *db = dbasis + m * K;
      for (int k = 0; k < K; ++k) db[k] = 0.0;
      for (int c = 0; c < C; ++c) {
        double s = 0.0;
        for (int k = 0; k < K; ++k) {
          db[k] += (double)g[c * K + k] * (double)f[c];
          s += (double)g[c * K + k] * (double)w[k];
        }
        dfeat[nb * C + c] += s;
      }
    }
  }
}

/* fp32 forms of the two functions above, multi-threaded, used as the host-CPU
 * figure reported beside the GPU one (same arithmetic type as the GPU path). */
void orc_basis_proj_f32(int64_t n_out, int C, int K, const float *basis,
                        const float *feat, const int *nbrs, const int *ranges,
                        float *out) {
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t i = 0; i < n_out; ++i) {
    int64_t a = i ? ranges[i - 1] : 0, b = ranges[i];
    float *o = out + i * C * K;
    for (int e = 0; e < C * K; ++e) o[e] = 0.0f;
    for (int64_t m = a; m < b; ++m) {
      const float *f = feat + (int64_t)nbrs[2 * m] * C;
      const float *w = basis + m * K;
      for (int c = 0; c < C; ++c) {
        float fc = f[c];
        for (int k = 0; k < K; ++k) o[c * K + k] += fc * w[k];
      }
    }
  }
}

void orc_basis_proj_grads_f32(int64_t n_in, int64_t n_out, int C, int K,
                              const float *basis, const float *feat,
                              const int *nbrs, const int *ranges,
                              const float *in_grad, float *dbasis,
                              float *dfeat) {
  memset(dfeat, 0, sizeof(float) * (size_t)n_in * C);
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t i = 0; i < n_out; ++i) {
    int64_t a = i ? ranges[i - 1] : 0, b = ranges[i];
    const float *g = in_grad + i * C * K;
    for (int64_t m = a; m < b; ++m) {
      int64_t nb = nbrs[2 * m];
      const float *f = feat + nb * C;
      const float *w = basis + m * K;
      float *db = dbasis + m * K;
      for (int k = 0; k < K; ++k) db[k] = 0.0f;
      for (int c = 0; c < C; ++c) {
        float s = 0.0f, fc = f[c];
        for (int k = 0; k < K; ++k) {
          db[k] += g[c * K + k] * fc;
          s += g[c * K + k] * w[k];
        }
#pragma omp atomic
        dfeat[nb * C + c] += s;
      }
    }
  }
}

/* ------------------------------------------------------------------------- */
/* sampling                                                                   */
/* ------------------------------------------------------------------------- */

/* count_unique_keys_kernels.cu.cc:34-68 + store_unique_keys_kernels.cu.cc:36-56,
 * with the cells kept in sorted order (custom_ops_tf.py:313-320).  first_idx
 * may be NULL to count only. */
int64_t orc_unique_keys(int64_t n, const int64_t *sorted_keys, int *first_idx) {
  int64_t u = 0;
  for (int64_t i = 0; i < n; ++i)
    if (i == 0 || sorted_keys[i] != sorted_keys[i - 1]) {
      if (first_idx) first_idx[u] = (int)i;
      ++u;
    }
  return u;
}

/* sampling_avg_kernels.cu.cc:42-88: per occupied cell the fp32 sum of its
 * points in sorted order divided by (float)count; batch id = key / prod(n).
 * Pinned by: the numpy loop of sample_test.py:101-125. */
void orc_sampling_avg(int D, int64_t n, int64_t n_cells, const float *pts,
                      const int64_t *sorted_keys, const int *nc,
                      const int *first_idx, float *out_pts, int *out_bids) {
  int64_t total = orc_total_cells(D, nc);
  for (int64_t u = 0; u < n_cells; ++u) {
    int64_t i = first_idx[u];
    int64_t key = sorted_keys[i];
    float acc[ORC_MAX_D] = {0};
    int cnt = 0;
    while (i < n && sorted_keys[i] == key) {
      for (int d = 0; d < D; ++d) acc[d] = acc[d] + pts[i * D + d];
      ++cnt;
      ++i;
    }
    for (int d = 0; d < D; ++d) out_pts[u * D + d] = acc[d] / (float)cnt;
    out_bids[u] = (int)(key / total);
  }
}

/* count_sampling_pd_kernels.cu.cc:41-108 and the host loop :156-181: 2^D passes,
 * pass `call` handles the cells whose index parity in dim i equals bit i of
 * `call`; inside a cell the points are visited in sorted order and a point is
 * selected iff none of its neighbours is already selected.  `used` is [n],
 * zeroed here; returns the number of selected points.
 * Pinned by: the collinear known-answer test n*n/2 of sample_test.py:61-78 and
 * the Poisson-disk invariants (pairwise separation, maximality). */
int64_t orc_sampling_poisson(int D, int64_t n, int64_t n_cells,
                             const int64_t *sorted_keys, const int *nc,
                             const int *nbrs, const int *ranges,
                             const int *first_idx, int *used) {
  memset(used, 0, sizeof(int) * (size_t)n);
  int64_t selected = 0;
  int calls = 1 << D;
  for (int call = 0; call < calls; ++call) {
    for (int64_t u = 0; u < n_cells; ++u) {
      int64_t i = first_idx[u];
      int64_t key = sorted_keys[i];
      int cell[ORC_MAX_D + 1];
      orc_cell_of_key(D, key, nc, cell);
      int valid_cell = 1;
      for (int d = 0; d < D; ++d)
        valid_cell = valid_cell && ((cell[d + 1] % 2) == ((call >> d) & 1));
      if (!valid_cell) continue;
      while (i < n && sorted_keys[i] == key) {
        int64_t a = i ? ranges[i - 1] : 0, b = ranges[i];
        int ok = 1;
        for (int64_t m = a; m < b; ++m) ok = ok && (used[nbrs[2 * m]] == 0);
        if (ok) {
          used[i] = 1;
          ++selected;
        }
        ++i;
      }
    }
  }
  return selected;
}
