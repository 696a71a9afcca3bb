// Fused Monte-Carlo convolution projection (pylib/pc/layers/MCConv.py:137-177,
// 264-269): the per-pair kernel-MLP basis
//     basis[m, j] = act(delta_m . W[:, j] + b[j]) / pdf[m],
//     delta_m = (p_in[nbr_m] - p_out[centre]) * inv_radii
// is evaluated in registers inside the matrix-core projection kernels, so the
// [M, K] basis tensor and its gradient never reach HBM.  Forward produces the
// same [N_out, C, K] projection as mc_basis + basis_proj; backward produces the
// feature gradient and the kernel-MLP weight / bias gradients from the upstream
// [N_out, C, K] gradient.  K in {16, 32, 64} (tiles of v_mfma_f32_16x16x4f32),
// D = 2 or 3, C a multiple of 16 (forward) or in {16, 32, 64, 128} (kernel-MLP
// gradients); other shapes use the separate kernels.
#include "common.h"
#include "fill.h"
#include "mfma.h"
#include "mc_conv.h"

namespace mccnn {

constexpr int kProjRun = 8;        // consecutive centres per wavefront
constexpr int kGradRun = 8;        // the same in the gradient kernels

// One wavefront per (run of kProjRun consecutive centres, chunk of 16*kCPL channels):
// projection of the centres' pairs with the basis evaluated in registers, rows
// written to out_rows[centre] (or centre).  Lane (quarter, col) owns channels
// col, col + 16, ... of the chunk, so that each of its kCPL stores lands in one
// contiguous kilobyte of the wavefront; the stores are non-temporal (the tile is
// read next by another kernel, and 3 GB of output would otherwise push the
// feature rows out of L2: 1.34 ms against 1.45 ms on 763 k centres x 64 channels).
// The run's pairs are
// one contiguous stretch of the table, which is walked in chunks of 64 pairs
// regardless of where the centres begin and end: lane n stages pair n of the
// chunk (offset to its own centre, 1/pdf, feature row) in LDS, and the pair
// indices and coordinates of the following chunks are already in flight while
// the current one is multiplied.  Matrix-core steps take 4 staged pairs each; a
// step that holds the last pair of a centre is run once per centre with the
// other centres' pairs weighted 0, the finished accumulators are stored and
// cleared, and the walk goes on.  Centres without pairs get their zeros the
// same way.
template <int kCPL, int D, int KT, class Basis>
__device__ __forceinline__ void project_run_body(
    int64_t n_out, int C, int chunks, const float *__restrict__ feat,
    const int2 *__restrict__ nbrs, const int *__restrict__ ranges, const McParams<D> &p,
    const Basis &basis, const int *__restrict__ out_rows, float *__restrict__ out,
    PairStage *stage, bool aux_is_point = false) {
  constexpr int K = kFusedK * KT;          // basis columns, KT tiles of 16
  constexpr int kCW = 16 * kCPL;
  const int lane = lane_id();
  const int64_t wid = wave_slot_xcd();
  const int64_t run = wid / chunks;
  const int64_t c0 = run * kProjRun;
  if (c0 >= n_out) return;
  const int chunk = (int)(wid - run * chunks);
  const int nc = (int)(n_out - c0 < kProjRun ? n_out - c0 : kProjRun);
  const int quarter = lane >> 4, col = lane & 15;
  // lane i < nc: end offset and output row of centre c0 + i
  int my_end = 0, my_row = 0;
  if (lane < nc) {
    my_end = ranges[c0 + lane];
    my_row = out_rows ? out_rows[c0 + lane] : (int)(c0 + lane);
  }
  const int begin = c0 > 0 ? ranges[c0 - 1] : 0;
  int ends[kProjRun];
#pragma unroll
  for (int i = 0; i < kProjRun; ++i)
    ends[i] = __builtin_amdgcn_readlane(my_end, i < nc ? i : nc - 1);
  const int total_end = ends[kProjRun - 1];
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = p.inv_radii[d];
  const char *feat_base = reinterpret_cast<const char *>(feat + chunk * kCW);
  const unsigned row_bytes = (unsigned)C * 4, lane_off = col * 4;
  float *out_base = out + (int64_t)chunk * kCW * K + 4 * quarter;

  // in flight for one chunk: the pair, its centre's and its neighbour's coordinates, its density
  struct Pending {
    int idx, aux;
    float ctr[D], pt[D], pdf;
  };
  auto fetch_index = [&](int m0) { return m0 + lane < total_end ? nbrs[m0 + lane].x : 0; };
  auto fetch_rest = [&](int m0, int idx) {
    Pending q;
    q.idx = idx;
    q.aux = 0;
    q.pdf = 1.0f;
#pragma unroll
    for (int d = 0; d < D; ++d) q.ctr[d] = q.pt[d] = 0.0f;
    const int m = m0 + lane;
    if (m < total_end) {
      int ci = 0;                       // centre of pair m inside the run
#pragma unroll
      for (int i = 0; i < kProjRun - 1; ++i) ci += m >= ends[i] ? 1 : 0;
#pragma unroll
      for (int d = 0; d < D; ++d) {
        q.ctr[d] = p.pout[(c0 + ci) * D + d];
        q.pt[d] = p.pin[(int64_t)idx * D + d];
      }
      if (p.pdf) q.pdf = p.pdf[m];
      // row of the per-centre side table: the pair's centre, or (transposed table) the
      // gathered point, which is the centre of the original direction
      if constexpr (Basis::kUsesAux) q.aux = aux_is_point ? idx : (int)(c0 + ci);
    }
    return q;
  };

  v4f acc[kCPL][KT];
#pragma unroll
  for (int j = 0; j < kCPL; ++j)
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) acc[j][kt] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  int cur = 0, cur_start = begin, cur_end = ends[0];
  auto finish_centre = [&]() {          // store and clear the accumulators, move to the next centre
    const int64_t row = __builtin_amdgcn_readlane(my_row, cur);
    float *o = out_base + row * (int64_t)C * K;
    // The tile leaves from copies of the accumulators: a store fetches its data from the
    // register file only when the memory pipeline gets to it, and a matrix instruction
    // that overwrites a register with a store pending on it waits for that fetch (in a
    // micro-benchmark of 80 MFMAs + a 4 KB tile per round, storing the accumulators
    // themselves takes 1.19 ms, storing copies 0.92 ms, the MFMAs alone 0.84 ms).
    v4f tile[kCPL][KT];
#pragma unroll
    for (int j = 0; j < kCPL; ++j)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        tile[j][kt] = acc[j][kt];
        asm volatile("" : "+v"(tile[j][kt]));
        acc[j][kt] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
      }
#ifdef MCCNN_PROBE_NO_TILE_STORES
    if (row == -7)          // measurement probe (no output): the kernel without its write-out
#endif
#pragma unroll
    for (int j = 0; j < kCPL; ++j)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
        __builtin_nontemporal_store(tile[j][kt],
                                    reinterpret_cast<v4f *>(o + (j * 16 + col) * K + 16 * kt));
    ++cur;
    cur_start = cur_end;
    cur_end = __builtin_amdgcn_readlane(my_end, cur < nc ? cur : nc - 1);
  };

  Pending pend = fetch_rest(begin, fetch_index(begin));
  int next_idx = fetch_index(begin + kWave);
  for (int m0 = begin; m0 < total_end; m0 += kWave) {
    const int cnt = total_end - m0 < kWave ? total_end - m0 : kWave;
    float dl[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int d = 0; d < D; ++d) dl[d] = (pend.pt[d] - pend.ctr[d]) * ir[d];
    const bool live = lane < cnt;
    const float4 g = make_float4(dl[0], dl[1], dl[2], live ? 1.0f / pend.pdf : 0.0f);
    const unsigned row = (unsigned)pend.idx * row_bytes;
    // slots past the last pair: the first pair's row with weight 0
    const unsigned row0 = __builtin_amdgcn_readfirstlane(row);
    wave_lds_sync();                    // the previous chunk has been read
    stage->geo[lane] = g;
    stage->row[lane] = live ? row : row0;
    if constexpr (Basis::kUsesAux) stage->aux[lane] = pend.aux;
    wave_lds_sync();
    pend = fetch_rest(m0 + kWave, next_idx);
    next_idx = fetch_index(m0 + 2 * kWave);
    const int steps = (cnt + 3) >> 2;
    for (int t = 0; t < steps; t += kFusedUnroll) {
      FVec<kCPL> f[kFusedUnroll];
      float w[kFusedUnroll][KT];
#pragma unroll
      for (int u = 0; u < kFusedUnroll; ++u) {
        const int n = 4 * (t + u) + quarter;
        const float4 gn = stage->geo[n];
        // one 32-bit lane offset on the wavefront's (scalar) base address
        const unsigned rn = stage->row[n];
#ifdef MCCNN_PROBE_NO_FEATURE_LOADS
        // measurement probe (wrong results): the B operands come from registers, so the run
        // time is that of the kernel with every feature row already on chip -- the bound of
        // any scheme that stages the rows in LDS
#pragma unroll
        for (int j = 0; j < kCPL; ++j) f[u].v[j] = gn.y + __uint_as_float(rn);
#else
#pragma unroll
        for (int j = 0; j < kCPL; ++j)
          f[u].v[j] = *reinterpret_cast<const float *>(feat_base + (size_t)(rn + lane_off) + j * 64);
#endif
        int aux = 0;
        if constexpr (Basis::kUsesAux) aux = stage->aux[n];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) w[u][kt] = basis(gn, kt, aux);
      }
#pragma unroll
      for (int u = 0; u < kFusedUnroll; ++u) {
        const int first = m0 + 4 * (t + u);           // pairs [first, first + 4) of the table
        const int mine = first + quarter;
        while (cur < nc && cur_end <= first + 4) {    // a centre ends inside this step
          if (cur_end > first && cur_end > cur_start) {
            const bool in = mine >= cur_start && mine < cur_end;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
              const float wm = in ? w[u][kt] : 0.0f;
#pragma unroll
              for (int j = 0; j < kCPL; ++j)
                acc[j][kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wm, f[u].v[j], acc[j][kt], 0, 0, 0);
            }
          }
          finish_centre();
        }
        if (cur < nc && cur_start < first + 4) {      // the rest of the step belongs to a centre that goes on
          const bool in = mine >= cur_start;
#pragma unroll
          for (int kt = 0; kt < KT; ++kt) {
            const float wm = in ? w[u][kt] : 0.0f;
#pragma unroll
            for (int j = 0; j < kCPL; ++j)
              acc[j][kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wm, f[u].v[j], acc[j][kt], 0, 0, 0);
          }
        }
      }
    }
  }
  while (cur < nc) finish_centre();     // a run without pairs, or trailing empty centres
}

template <int kCPL, int D, int kAct, int KT>
__global__ void __launch_bounds__(256) mc_conv_project16_kernel(
    int64_t n_out, int C, int chunks, const float *__restrict__ feat,
    const int2 *__restrict__ nbrs, const int *__restrict__ ranges, McParams<D> p,
    const int *__restrict__ out_rows, float *__restrict__ out) {
  __shared__ PairStage stages[kWavesPerBlock];
  const MlpBasis<D, kAct, KT> basis(p);
  project_run_body<kCPL, D, KT>(n_out, C, chunks, feat, nbrs, ranges, p, basis, out_rows, out,
                                &stages[threadIdx.x / kWave]);
}

// The same projection with the kernel-point correlation of KPConv as basis
// (KPConv.py:193-224: weights of up to 32 kernel points in one or two tiles of 16
// columns, zero padding beyond the last point).
template <int kCPL, int D, int kKind, int KT>
__global__ void __launch_bounds__(256) kp_conv_project16_kernel(
    int64_t n_out, int C, int chunks, const float *__restrict__ feat,
    const int2 *__restrict__ nbrs, const int *__restrict__ ranges, McParams<D> p,
    const float *__restrict__ kernel_points, int num_kp, float sigma,
    const int *__restrict__ out_rows, float *__restrict__ out) {
  __shared__ PairStage stages[kWavesPerBlock];
  const KpBasis<D, kKind, KT> basis(kernel_points, num_kp, sigma);
  project_run_body<kCPL, D, KT>(n_out, C, chunks, feat, nbrs, ranges, p, basis, out_rows, out,
                                &stages[threadIdx.x / kWave]);
}

// The projection of the deformable kernel-point convolution (KPConv.py:317-392): as
// above with every centre's kernel points shifted by its row of `offsets`
// [N_centres, num_kp, D].  Over the transposed pair table (`offsets_follow_points`)
// the shifts belong to the gathered side of a pair.
template <int kCPL, int D, int kKind>
__global__ void __launch_bounds__(256) kp_deform_project16_kernel(
    int64_t n_out, int C, int chunks, const float *__restrict__ feat,
    const int2 *__restrict__ nbrs, const int *__restrict__ ranges, McParams<D> p,
    const float *__restrict__ kernel_points, int num_kp, float sigma,
    const float *__restrict__ offsets, int offsets_follow_points,
    const int *__restrict__ out_rows, float *__restrict__ out) {
  __shared__ PairStage stages[kWavesPerBlock];
  const KpDeformBasis<D, kKind> basis(kernel_points, num_kp, sigma, offsets);
  project_run_body<kCPL, D, 1>(n_out, C, chunks, feat, nbrs, ranges, p, basis, out_rows, out,
                               &stages[threadIdx.x / kWave], offsets_follow_points != 0);
}

// Gradient of the deformable convolution with respect to the kernel-point offsets,
//   doff[i, k, :] = sum_{pairs m of centre i} dbasis[m, k] * w'(dist) * (-diff / dist),
//   dbasis[m, k] = sum_c G[i, c, k] * feat[nbr_m, c],   diff = delta_m - kp_k - off[i, k],
// without the [M, 16] basis gradient in memory: per centre the upstream tile G [C x 16]
// sits in registers as the A operand, a chunk of 64 pairs is parked in LDS, every tile
// of 16 pairs takes C/4 matrix steps for dbasis^T [k x pair], and each lane folds its
// four (pair, k) entries into running sums that are added over the 16 lanes of a
// quarter at the end of the centre: fixed order, no atomics.
template <int C, int D, int kKind>
__global__ void __launch_bounds__(256) kp_deform_offset_grads16_kernel(
    int64_t n_out, const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, McParams<D> p, const float *__restrict__ kernel_points,
    int num_kp, float sigma, const float *__restrict__ offsets,
    const float *__restrict__ in_grad, float *__restrict__ doffsets) {
  constexpr int K = kFusedK;
  constexpr int kQuarterC = C / 4;
  __shared__ PairStage stages[kWavesPerBlock];
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int quarter = lane >> 4, col = lane & 15;
  PairStage *stage = &stages[wave];
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = p.inv_radii[d];
  float kp[4][3];                     // kernel points 4 quarter + r of this lane's rows
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int d = 0; d < 3; ++d)
      kp[r][d] = (d < D && 4 * quarter + r < num_kp) ? kernel_points[(4 * quarter + r) * D + d]
                                                     : 0.0f;
  const char *feat_lane = reinterpret_cast<const char *>(feat + quarter * kQuarterC);
  const int64_t first = wave_slot() * kGradRun;
  const int64_t last = first + kGradRun < n_out ? first + kGradRun : n_out;
  for (int64_t centre = first; centre < last; ++centre) {
    const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
    float sum[4][3];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int d = 0; d < 3; ++d) sum[r][d] = 0.0f;
    if (b > a) {
      const float *gi = in_grad + centre * (int64_t)C * K;
      float gk[kQuarterC];
#pragma unroll
      for (int s = 0; s < kQuarterC; ++s) gk[s] = gi[(quarter * kQuarterC + s) * K + col];
      float ctr[D];
#pragma unroll
      for (int d = 0; d < D; ++d) ctr[d] = p.pout[centre * D + d];
      // this centre's shifted kernel points 4 quarter + r
      float kpo[4][3];
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int d = 0; d < 3; ++d)
          kpo[r][d] = kp[r][d] + ((d < D && 4 * quarter + r < num_kp)
                                      ? offsets[(centre * num_kp + 4 * quarter + r) * D + d]
                                      : 0.0f);
      for (int m0 = a; m0 < b; m0 += kWave) {
        const int cnt = b - m0 < kWave ? b - m0 : kWave;
        float4 g = {0.0f, 0.0f, 0.0f, 0.0f};
        unsigned row = 0;
        if (lane < cnt) {
          const int idx = nbrs[m0 + lane].x;
          float dl[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int d = 0; d < D; ++d) dl[d] = (p.pin[(int64_t)idx * D + d] - ctr[d]) * ir[d];
          g = make_float4(dl[0], dl[1], dl[2], 1.0f);
          row = (unsigned)idx * (unsigned)(C * 4);
        }
        const unsigned row0 = __builtin_amdgcn_readfirstlane(row);
        stage->geo[lane] = g;
        stage->row[lane] = lane < cnt ? row : row0;
        wave_lds_sync();
        const int tiles = (cnt + 15) >> 4;
        FVec<kQuarterC> f = load_vec<kQuarterC>(
            reinterpret_cast<const float *>(feat_lane + stage->row[col]), true);
        for (int t = 0; t < tiles; ++t) {
          FVec<kQuarterC> fn = f;
          if (t + 1 < tiles)
            fn = load_vec<kQuarterC>(
                reinterpret_cast<const float *>(feat_lane + stage->row[16 * (t + 1) + col]), true);
          const float4 geo = stage->geo[16 * t + col];
          v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int s = 0; s < kQuarterC; ++s)
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(gk[s], f.v[s], acc, 0, 0, 0);
          // acc[r] = dbasis[pair col][k = 4*quarter + r]; geo.w = 1 for a live pair, else 0
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float dx = geo.x - kpo[r][0], dy = geo.y - kpo[r][1], dz = geo.z - kpo[r][2];
            const float dist = sqrtf(dx * dx + dy * dy + dz * dz);
            float slope;
            if (kKind == 0) {
              slope = dist < sigma ? -1.0f / sigma : 0.0f;
            } else {
              const float sg = sigma / 3.0f, q = dist / sg;
              slope = -2.0f * q / sg * expf(-(q * q));
            }
            const float coef = dist > 0.0f ? -acc[r] * geo.w * slope / dist : 0.0f;
            sum[r][0] += coef * dx;
            sum[r][1] += coef * dy;
            if (D > 2) sum[r][2] += coef * dz;
          }
          f = fn;
        }
        wave_lds_sync();                      // the stage is free for the next chunk
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int d = 0; d < D; ++d)
#pragma unroll
          for (int off = 8; off > 0; off >>= 1) sum[r][d] += __shfl_xor(sum[r][d], off, kWave);
    }
    if (col == 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (4 * quarter + r < num_kp) {
#pragma unroll
          for (int d = 0; d < D; ++d)
            doffsets[(centre * num_kp + 4 * quarter + r) * D + d] = sum[r][d];
        }
    }
  }
}

// Feature gradient by scatter, for callers that do not use the transposed
// convolution: one wavefront per centre, per tile of 16 pairs the basis is
// recomputed in registers and dfeat [pair x channel] = basis [pair x k] * G [k x
// channel] comes from the matrix cores; it is added to the feature gradient with
// fp32 atomics or (pair_rows given) stored per pair for the atomic-free gather
// that follows.
template <int C, int D, int kAct>
__global__ void __launch_bounds__(256) mc_conv_feature_grads16_kernel(
    int64_t n_out, const int2 *__restrict__ nbrs, const int *__restrict__ ranges, McParams<D> p,
    const float *__restrict__ in_grad, float *__restrict__ dfeat,
    float *__restrict__ pair_rows) {
  constexpr int K = kFusedK;
  constexpr int kTiles = C / 16;
  __shared__ float wlds[K * (D + 1)];     // column j: D weights then the bias
  const int lane = lane_id();
  const int quarter = lane >> 4, col = lane & 15;
  if (threadIdx.x < K) {
    float w[D], bias;
    load_weight_column<D>(p, threadIdx.x, w, &bias);
#pragma unroll
    for (int d = 0; d < D; ++d) wlds[threadIdx.x * (D + 1) + d] = w[d];
    wlds[threadIdx.x * (D + 1) + D] = bias;
  }
  __syncthreads();
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = p.inv_radii[d];
  const int64_t total_waves = (int64_t)gridDim.x * kWavesPerBlock;
  for (int64_t centre = wave_slot(); centre < n_out; centre += total_waves) {
    const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
    if (b <= a) continue;
    const float *gi = in_grad + centre * (int64_t)C * K;
    float ctr[D];
#pragma unroll
    for (int d = 0; d < D; ++d) ctr[d] = p.pout[centre * D + d];

    for (int m0 = a; m0 < b; m0 += 16) {
      const int cnt = b - m0 < 16 ? b - m0 : 16;
      const bool valid = col < cnt;
      const int idx = nbrs[m0 + (valid ? col : 0)].x;
      const float inv_pdf = valid ? 1.0f / p.pdf[m0 + col] : 0.0f;
      float delta[D];
#pragma unroll
      for (int d = 0; d < D; ++d)
        delta[d] = valid ? (p.pin[(int64_t)idx * D + d] - ctr[d]) * ir[d] : 0.0f;
      // this lane's pair and its four basis columns 4*quarter .. +3
      float basis4[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float *wr = wlds + (4 * quarter + r) * (D + 1);
        float z = wr[D];
#pragma unroll
        for (int d = 0; d < D; ++d) z += delta[d] * wr[d];
        basis4[r] = valid ? act_fwd(kAct, z) * inv_pdf : 0.0f;
      }
#pragma unroll
      for (int t = 0; t < kTiles; ++t) {
        // B operand of channel tile t: G[c = 16 t + col][k = 4*quarter + s] (L1 resident)
        const FVec<4> gt = load_vec<4>(gi + (16 * t + col) * K + 4 * quarter, true);
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
        if (pair_rows) {
          // rows = channels, columns = pairs: this lane holds channels
          // 16 t + 4*quarter .. +3 of pair `col` -> one 16-byte store
#pragma unroll
          for (int s = 0; s < 4; ++s)
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(gt.v[s], basis4[s], acc, 0, 0, 0);
          if (valid)
            *reinterpret_cast<v4f *>(pair_rows + (int64_t)(m0 + col) * C + 16 * t +
                                     4 * quarter) = acc;
        } else {
          // rows = pairs, columns = channels: 64 consecutive bytes per row and atomic
#pragma unroll
          for (int s = 0; s < 4; ++s)
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(basis4[s], gt.v[s], acc, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int n = 4 * quarter + r;
            const int nidx = __shfl(idx, n, kWave);
            if (n < cnt) unsafeAtomicAdd(dfeat + (int64_t)nidx * C + 16 * t + col, acc[r]);
          }
        }
      }
    }
  }
}

// Kernel-MLP gradients alone (the layer obtains its feature gradient from the
// transposed convolution).  Per centre the upstream tile G [C x 16] sits in
// registers as the A operand; per chunk of 64 pairs lane n stages pair n in LDS
// (offset, 1/pdf, feature row), then every tile of 16 pairs takes 16*C/64 matrix
// steps for dbasis^T [k x pair] while the feature rows of the next tile are
// already in flight, and the result is folded in registers into
//   dW[d][k] += delta_d * dz,  db[k] += dz,  dz = dbasis * act'(z) / pdf.

static int64_t grad_blocks(int64_t num_samples) {
  const int64_t per_block = (int64_t)kWavesPerBlock * kGradRun;
  const int64_t b = (num_samples + per_block - 1) / per_block;
  return b < 1 ? 1 : b;
}

template <int C, int D, int kAct, int KT>
__global__ void __launch_bounds__(256) mc_conv_weight_grads16_kernel(
    int64_t n_out, const float *__restrict__ feat, const int2 *__restrict__ nbrs,
    const int *__restrict__ ranges, McParams<D> p, const float *__restrict__ in_grad,
    float *__restrict__ partials, float *__restrict__ pair_sums, int64_t pair_stride) {
  constexpr int K = kFusedK;               // a block works on basis columns k0 .. k0 + 15
  constexpr int num_basis = kFusedK * KT;  // of the KT * 16 the layer has
  constexpr int kQuarterC = C / 4;
  __shared__ float red[kWavesPerBlock][(D + 1) * K];
  __shared__ float4 wlds[K];               // column j: weights (z = 0 for D = 2), bias in w
  __shared__ PairStage stages[kWavesPerBlock];
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int quarter = lane >> 4, col = lane & 15;
  const int k0 = blockIdx.y * K;
  if (pair_sums) pair_sums += (int64_t)blockIdx.y * pair_stride;   // [K / 16][M]
  if (threadIdx.x < K) {
    float w[3] = {0.0f, 0.0f, 0.0f}, bias;
    load_weight_column<D>(p, k0 + threadIdx.x, w, &bias);
    wlds[threadIdx.x] = make_float4(w[0], w[1], w[2], bias);
  }
  __syncthreads();
  PairStage *stage = &stages[wave];
  float ir[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ir[d] = p.inv_radii[d];
  float dw[4][3], db[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    db[r] = 0.0f;
#pragma unroll
    for (int d = 0; d < 3; ++d) dw[r][d] = 0.0f;
  }
  const char *feat_lane = reinterpret_cast<const char *>(feat + quarter * kQuarterC);
  // A wavefront takes kGradRun consecutive centres and blocks are dispatched in
  // index order, so at any moment the device works on one compact window of the
  // (grid-ordered) centres and the feature rows of that window stay in L2.
  // (Giving each XCD its own contiguous eighth of the centres instead was measured
  // on the scene-scale case, for this kernel and the projection: 12 % slower; dealing
  // windows of consecutive blocks to the XCDs in turn leaves the time as it is and
  // cuts the re-fetched feature rows.)
  const int64_t first = wave_slot_xcd() * kGradRun;
  const int64_t last = first + kGradRun < n_out ? first + kGradRun : n_out;
  for (int64_t centre = first; centre < last; ++centre) {
    const int a = centre > 0 ? ranges[centre - 1] : 0, b = ranges[centre];
    if (b <= a) continue;
    const float *gi = in_grad + centre * (int64_t)C * num_basis + k0;
    float gk[kQuarterC];
#pragma unroll
    for (int s = 0; s < kQuarterC; ++s) gk[s] = gi[(quarter * kQuarterC + s) * num_basis + col];
    float ctr[D];
#pragma unroll
    for (int d = 0; d < D; ++d) ctr[d] = p.pout[centre * D + d];

    for (int m0 = a; m0 < b; m0 += kWave) {
      const int cnt = b - m0 < kWave ? b - m0 : kWave;
      float4 g = {0.0f, 0.0f, 0.0f, 0.0f};
      unsigned row = 0;
      if (lane < cnt) {
        const int idx = nbrs[m0 + lane].x;
        float dl[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int d = 0; d < D; ++d) dl[d] = (p.pin[(int64_t)idx * D + d] - ctr[d]) * ir[d];
        g = make_float4(dl[0], dl[1], dl[2], 1.0f / p.pdf[m0 + lane]);
        row = (unsigned)idx * (unsigned)(C * 4);
      }
      const unsigned row0 = __builtin_amdgcn_readfirstlane(row);
      stage->geo[lane] = g;
      stage->row[lane] = lane < cnt ? row : row0;
      wave_lds_sync();
      const int tiles = (cnt + 15) >> 4;
      FVec<kQuarterC> f = load_vec<kQuarterC>(
          reinterpret_cast<const float *>(feat_lane + stage->row[col]), true);
      for (int t = 0; t < tiles; ++t) {
        FVec<kQuarterC> fn = f;
        if (t + 1 < tiles)
          fn = load_vec<kQuarterC>(
              reinterpret_cast<const float *>(feat_lane + stage->row[16 * (t + 1) + col]), true);
        const float4 geo = stage->geo[16 * t + col];
        v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < kQuarterC; ++s)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(gk[s], f.v[s], acc, 0, 0, 0);
        // acc[r] = dbasis[pair col][k = 4*quarter + r]
        float along = 0.0f;                 // sum_k dbasis * act(z) over this lane's columns
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float4 wr = wlds[4 * quarter + r];
          const float z = wr.w + geo.x * wr.x + geo.y * wr.y + geo.z * wr.z;
          const float dz = acc[r] * act_bwd(kAct, z) * geo.w;
          db[r] += dz;
          dw[r][0] += geo.x * dz;
          dw[r][1] += geo.y * dz;
          if (D > 2) dw[r][2] += geo.z * dz;
          if (pair_sums) along += acc[r] * act_fwd(kAct, z);
        }
        if (pair_sums) {
          // the gradient with respect to the pair's scale 1/pdf, over the block's 16 columns
          along += __shfl_xor(along, 16, kWave);
          along += __shfl_xor(along, 32, kWave);
          if (quarter == 0 && 16 * t + col < cnt) pair_sums[m0 + 16 * t + col] = along;
        }
        f = fn;
      }
      wave_lds_sync();                      // the stage is free for the next chunk
    }
  }
  // reduce over the 16 pair-lanes of each quarter
#pragma unroll
  for (int r = 0; r < 4; ++r) {
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) {
      db[r] += __shfl_xor(db[r], off, kWave);
#pragma unroll
      for (int d = 0; d < D; ++d) dw[r][d] += __shfl_xor(dw[r][d], off, kWave);
    }
  }
  if (col == 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int k = 4 * quarter + r;
#pragma unroll
      for (int d = 0; d < D; ++d) red[wave][d * K + k] = dw[r][d];
      red[wave][D * K + k] = db[r];
    }
  }
  __syncthreads();
  if (threadIdx.x < (D + 1) * K) {
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) s += red[w][threadIdx.x];
    const int q = threadIdx.x / K, j = threadIdx.x - q * K;
    partials[(int64_t)blockIdx.x * (D + 1) * num_basis + q * num_basis + k0 + j] = s;
  }
}

// weight_grads [L, D, H], bias_grads [L*H] from partials [blocks][(D+1)][K]: one
// block per output, threads stride over the partials, fixed summation order.
__global__ void __launch_bounds__(256) mc_conv_reduce_kernel(int64_t blocks, int D, int K, int H,
                                                             const float *__restrict__ partials,
                                                             float *__restrict__ dweights,
                                                             float *__restrict__ dbiases) {
  __shared__ float red[256 / kWave];
  const int t = blockIdx.x;
  const int q = t / K, j = t - q * K;
  float s = 0.0f;
  for (int64_t b = threadIdx.x; b < blocks; b += 256) s += partials[b * (D + 1) * K + t];
  s = wave_sum(s);
  if (lane_id() == 0) red[threadIdx.x / kWave] = s;
  __syncthreads();
  if (threadIdx.x != 0) return;
  s = 0.0f;
#pragma unroll
  for (int w = 0; w < 256 / kWave; ++w) s += red[w];
  const int l = j / H, h = j - l * H;
  if (q < D) dweights[(l * D + q) * H + h] = s;
  else dbiases[j] = s;
}

// Weight-gradient kernel (one partial sum per block, reduced afterwards), then, if
// asked for, the feature-gradient half.
template <int C, int D, int ACT>
static int launch_fused_backward(hipStream_t s, int64_t num_samples, const float *features,
                                 const int2 *nb, const int *ranges, const McParams<D> &prm,
                                 int num_basis, const float *in_grads, float *feature_grads_out,
                                 float *pair_rows, float *workspace, bool want_dfeat,
                                 float *pair_sums, int64_t num_neighbors) {
  const dim3 grid((unsigned)grad_blocks(num_samples), (unsigned)(num_basis / kFusedK));
  switch (num_basis / kFusedK) {
    case 1:
      hipLaunchKernelGGL((mc_conv_weight_grads16_kernel<C, D, ACT, 1>), grid, dim3(256), 0, s,
                         num_samples, features, nb, ranges, prm, in_grads, workspace, pair_sums,
                         num_neighbors);
      break;
    case 2:
      hipLaunchKernelGGL((mc_conv_weight_grads16_kernel<C, D, ACT, 2>), grid, dim3(256), 0, s,
                         num_samples, features, nb, ranges, prm, in_grads, workspace, pair_sums,
                         num_neighbors);
      break;
    default:
      hipLaunchKernelGGL((mc_conv_weight_grads16_kernel<C, D, ACT, 4>), grid, dim3(256), 0, s,
                         num_samples, features, nb, ranges, prm, in_grads, workspace, pair_sums,
                         num_neighbors);
      break;
  }
  if (want_dfeat)        // the feature half keeps no running sums: one wavefront per centre
    hipLaunchKernelGGL((mc_conv_feature_grads16_kernel<C, D, ACT>),
                       dim3(wave_grid(num_samples)), dim3(256), 0, s, num_samples, nb, ranges, prm,
                       in_grads, feature_grads_out, pair_rows);
  return MCCNN_OK;
}

static bool fused_basis_count(int K) { return K == 16 || K == 32 || K == 64; }

// Shapes of the weight-gradient kernel (C is a template parameter); the
// feature-gradient half that goes with it exists for 16 basis columns only.
static bool fused_supported(int D, int C, int K, bool weights_only) {
  return (D == 2 || D == 3) && (weights_only ? fused_basis_count(K) : K == kFusedK) &&
         (C == 16 || C == 32 || C == 64 || C == 128);
}

// Shapes of the projection kernels: any multiple of 16 channels, in chunks of up
// to 128 channels per wavefront, 16 / 32 / 64 basis columns.
static bool project_supported(int D, int C, int K) {
  return (D == 2 || D == 3) && fused_basis_count(K) && C >= 16 && C <= 512 && C % 16 == 0;
}

static int check_fused_args(const char *op, bool project_only, bool weights_only, int num_dims,
                            int num_features, int num_basis, int num_mlps, int activation,
                            int64_t num_neighbors, int64_t num_samples) {
  MCCNN_REQUIRE(project_only ? project_supported(num_dims, num_features, num_basis)
                             : fused_supported(num_dims, num_features, num_basis, weights_only),
                "%s supports D in {2,3}, K in %s and C in %s (got D=%d, K=%d, C=%d); "
                "use mc_basis + basis_proj for other shapes", op,
                project_only || weights_only ? "{16,32,64}" : "{16}",
                project_only ? "{16, 32, ..., 512}" : "{16,32,64,128}", num_dims, num_basis,
                num_features);
  MCCNN_REQUIRE(num_mlps > 0 && num_basis % num_mlps == 0,
                "%s expects the number of basis functions to be divisible by the number of "
                "kernel MLPs", op);
  MCCNN_REQUIRE(activation >= 0 && activation <= 2, "%s expects a known activation", op);
  MCCNN_REQUIRE(num_neighbors >= 0 && num_neighbors < ((int64_t)1 << 31) && num_samples >= 0 &&
                    num_samples < ((int64_t)1 << 31),
                "%s expects sizes in [0, 2^31)", op);
  return MCCNN_OK;
}

}  // namespace mccnn

using namespace mccnn;

extern "C" int mccnn_mc_conv_supported(int num_dims, int num_features, int num_basis) {
  return fused_supported(num_dims, num_features, num_basis, false) ? 1 : 0;
}

extern "C" int mccnn_mc_conv_weight_grads_supported(int num_dims, int num_features,
                                                    int num_basis) {
  return fused_supported(num_dims, num_features, num_basis, true) ? 1 : 0;
}

extern "C" int mccnn_mc_conv_project_supported(int num_dims, int num_features, int num_basis) {
  return project_supported(num_dims, num_features, num_basis) ? 1 : 0;
}

extern "C" int mccnn_mc_conv_project(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                                     const float *points_in, int num_features,
                                     const float *features, int64_t num_samples,
                                     const float *points_out, int64_t num_neighbors,
                                     const int32_t *neighbors, const int32_t *ranges,
                                     const float *inv_radii, int num_basis, int num_mlps,
                                     int activation, const float *weights, const float *biases,
                                     const float *pdf, const int32_t *out_rows, float *out) {
  int rc = check_fused_args("mc_conv_project", true, false, num_dims, num_features, num_basis,
                            num_mlps, activation, num_neighbors, num_samples);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(num_pts >= 0 && num_pts * num_features < ((int64_t)1 << 30),
                "mc_conv_project expects a feature table of fewer than 2^30 elements");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && out && points_out && inv_radii && weights && biases &&
                    (num_neighbors == 0 || (points_in && features && neighbors && pdf)),
                "mc_conv_project received a null tensor");
  hipStream_t s = as_stream(stream);
  // channels per lane and pass: at most 8 accumulator tiles of 16 x 16 per wavefront
  const int kt = num_basis / kFusedK;
  int cpl = 1;
  for (int c = 8 / kt; c >= 1; c >>= 1)
    if (num_features % (16 * c) == 0) { cpl = c; break; }
  const int chunks = num_features / (16 * cpl);
  const dim3 grid(wave_grid((num_samples + kProjRun - 1) / kProjRun * chunks)), block(256);
  const int2 *nb = (const int2 *)neighbors;
#define MCCNN_FUSED_FWD(CPL_, D_, KT_)                                                         \
  {                                                                                            \
    McParams<D_> prm{points_in, points_out, inv_radii, weights, biases, pdf,                   \
                     num_basis / num_mlps, activation};                                        \
    MCCNN_ACT_SWITCH(activation,                                                               \
                     hipLaunchKernelGGL((mc_conv_project16_kernel<CPL_, D_, ACT, KT_>), grid,  \
                                        block, 0, s, num_samples, num_features, chunks,        \
                                        features, nb, ranges, prm, out_rows, out));            \
  }
#define MCCNN_FUSED_FWD_D(CPL_, KT_) \
  if (num_dims == 3) MCCNN_FUSED_FWD(CPL_, 3, KT_) else MCCNN_FUSED_FWD(CPL_, 2, KT_)
  switch (kt * 16 + cpl) {
    case 16 + 8: MCCNN_FUSED_FWD_D(8, 1); break;
    case 16 + 4: MCCNN_FUSED_FWD_D(4, 1); break;
    case 16 + 2: MCCNN_FUSED_FWD_D(2, 1); break;
    case 16 + 1: MCCNN_FUSED_FWD_D(1, 1); break;
    case 32 + 4: MCCNN_FUSED_FWD_D(4, 2); break;
    case 32 + 2: MCCNN_FUSED_FWD_D(2, 2); break;
    case 32 + 1: MCCNN_FUSED_FWD_D(1, 2); break;
    case 64 + 2: MCCNN_FUSED_FWD_D(2, 4); break;
    default: MCCNN_FUSED_FWD_D(1, 4); break;
  }
#undef MCCNN_FUSED_FWD_D
#undef MCCNN_FUSED_FWD
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" size_t mccnn_mc_conv_project_grads_workspace_bytes(int num_dims, int num_basis,
                                                              int64_t num_samples) {
  if (!valid_dims(num_dims) || num_basis <= 0 || num_samples < 0) return 0;
  return align256(sizeof(float) * (size_t)grad_blocks(num_samples) * (num_dims + 1) * num_basis);
}

static int project_grads(
    mccnn_stream_t stream, int num_dims, int64_t num_pts, const float *points_in,
    int num_features, const float *features, int64_t num_samples, const float *points_out,
    int64_t num_neighbors, const int32_t *neighbors, const int32_t *ranges,
    const float *inv_radii, int num_basis, int num_mlps, int activation, const float *weights,
    const float *biases, const float *pdf, const float *in_grads, void *workspace,
    size_t workspace_bytes, const int32_t *point_ranges, const int32_t *pair_order,
    float *pair_rows_workspace, float *feature_grads_out, float *weight_grads_out,
    float *bias_grads_out, float *pair_sums) {
  float *pair_rows = pair_rows_workspace;
  const bool gathered = pair_rows != nullptr;
  MCCNN_REQUIRE(!gathered || (point_ranges && pair_order),
                "mc_conv_project_grads needs the transposed pair lists with a pair-row "
                "workspace");
  int rc = check_fused_args("mc_conv_project_grads", false, feature_grads_out == nullptr,
                            num_dims, num_features, num_basis, num_mlps, activation,
                            num_neighbors, num_samples);
  if (rc != MCCNN_OK) return rc;
  MCCNN_REQUIRE(num_pts >= 0 && num_pts * num_features < ((int64_t)1 << 30),
                "mc_conv_project_grads expects a feature table of fewer than 2^30 elements");
  MCCNN_REQUIRE(workspace && weight_grads_out && bias_grads_out && weights && biases &&
                    inv_radii,
                "mc_conv_project_grads received a null tensor");
  MCCNN_REQUIRE(workspace_bytes >=
                    mccnn_mc_conv_project_grads_workspace_bytes(num_dims, num_basis, num_samples),
                "mc_conv_project_grads workspace too small");
  hipStream_t s = as_stream(stream);
  // A null feature_grads_out asks for the kernel-MLP gradients only.
  const bool want_dfeat = feature_grads_out != nullptr;
  MCCNN_REQUIRE(want_dfeat || !gathered,
                "mc_conv_project_grads received a pair-row workspace but no feature gradient");
  if (want_dfeat && num_pts > 0 && (!gathered || num_samples == 0 || num_neighbors == 0)) {
    rc = fill_zero(s, feature_grads_out, sizeof(float) * (size_t)num_pts * num_features);
    if (rc != MCCNN_OK) return rc;
  }
  MCCNN_REQUIRE(num_samples == 0 || num_neighbors == 0 ||
                    (points_in && points_out && features && neighbors && ranges && pdf &&
                     in_grads),
                "mc_conv_project_grads received a null tensor");
  const int2 *nb = (const int2 *)neighbors;
#define MCCNN_FUSED_BWD(C_, D_)                                                                \
  {                                                                                            \
    McParams<D_> prm{points_in, points_out, inv_radii, weights, biases, pdf,                   \
                     num_basis / num_mlps, activation};                                        \
    MCCNN_ACT_SWITCH(activation,                                                               \
                     rc = (launch_fused_backward<C_, D_, ACT>(                                 \
                         s, num_samples, features, nb, ranges, prm, num_basis, in_grads,       \
                         feature_grads_out, pair_rows, (float *)workspace, want_dfeat,         \
                         pair_sums, num_neighbors)));                                          \
  }
#define MCCNN_FUSED_BWD_D(C_) \
  if (num_dims == 3) MCCNN_FUSED_BWD(C_, 3) else MCCNN_FUSED_BWD(C_, 2)
  switch (num_features) {
    case 16: MCCNN_FUSED_BWD_D(16); break;
    case 32: MCCNN_FUSED_BWD_D(32); break;
    case 64: MCCNN_FUSED_BWD_D(64); break;
    default: MCCNN_FUSED_BWD_D(128); break;
  }
#undef MCCNN_FUSED_BWD_D
#undef MCCNN_FUSED_BWD
  if (rc != MCCNN_OK) return rc;
  MCCNN_LAUNCH_CHECK();
  const int outs = (num_dims + 1) * num_basis;
  hipLaunchKernelGGL(mc_conv_reduce_kernel, dim3(outs), dim3(256), 0, s,
                     grad_blocks(num_samples), num_dims, num_basis, num_basis / num_mlps, (const float *)workspace,
                     weight_grads_out, bias_grads_out);
  MCCNN_LAUNCH_CHECK();
  if (gathered && num_samples > 0 && num_neighbors > 0)
    return launch_dfeat_gather(s, num_pts, num_features, point_ranges, pair_order, pair_rows,
                               feature_grads_out);
  return MCCNN_OK;
}

extern "C" int mccnn_mc_conv_project_grads(
    mccnn_stream_t stream, int num_dims, int64_t num_pts, const float *points_in,
    int num_features, const float *features, int64_t num_samples, const float *points_out,
    int64_t num_neighbors, const int32_t *neighbors, const int32_t *ranges,
    const float *inv_radii, int num_basis, int num_mlps, int activation, const float *weights,
    const float *biases, const float *pdf, const float *in_grads, void *workspace,
    size_t workspace_bytes, const int32_t *point_ranges, const int32_t *pair_order,
    float *pair_rows_workspace, float *feature_grads_out, float *weight_grads_out,
    float *bias_grads_out) {
  return project_grads(stream, num_dims, num_pts, points_in, num_features, features, num_samples,
                       points_out, num_neighbors, neighbors, ranges, inv_radii, num_basis,
                       num_mlps, activation, weights, biases, pdf, in_grads, workspace,
                       workspace_bytes, point_ranges, pair_order, pair_rows_workspace,
                       feature_grads_out, weight_grads_out, bias_grads_out, nullptr);
}

extern "C" int mccnn_mc_conv_weight_and_scale_grads(
    mccnn_stream_t stream, int num_dims, int64_t num_pts, const float *points_in,
    int num_features, const float *features, int64_t num_samples, const float *points_out,
    int64_t num_neighbors, const int32_t *neighbors, const int32_t *ranges,
    const float *inv_radii, int num_basis, int num_mlps, int activation, const float *weights,
    const float *biases, const float *pdf, const float *in_grads, void *workspace,
    size_t workspace_bytes, float *weight_grads_out, float *bias_grads_out,
    float *pair_scale_grads_out) {
  MCCNN_REQUIRE(pair_scale_grads_out || num_neighbors == 0,
                "mc_conv_weight_and_scale_grads received a null output");
  return project_grads(stream, num_dims, num_pts, points_in, num_features, features, num_samples,
                       points_out, num_neighbors, neighbors, ranges, inv_radii, num_basis,
                       num_mlps, activation, weights, biases, pdf, in_grads, workspace,
                       workspace_bytes, nullptr, nullptr, nullptr, nullptr, weight_grads_out,
                       bias_grads_out, pair_scale_grads_out);
}

extern "C" int mccnn_kp_conv_project(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                                     const float *points_in, int num_features,
                                     const float *features, int64_t num_samples,
                                     const float *points_out, int64_t num_neighbors,
                                     const int32_t *neighbors, const int32_t *ranges,
                                     const float *inv_radii, int num_kernel_points,
                                     const float *kernel_points, int kind, float sigma,
                                     const int32_t *out_rows, float *out) {
  MCCNN_REQUIRE(project_supported(num_dims, num_features, kFusedK),
                "kp_conv_project supports D in {2,3} and C in {16, 32, ..., 512} (got D=%d, C=%d); "
                "use kp_basis + basis_proj for other shapes", num_dims, num_features);
  MCCNN_REQUIRE(num_kernel_points > 0 && num_kernel_points <= 2 * kFusedK,
                "kp_conv_project supports 1 to 32 kernel points (got %d)", num_kernel_points);
  MCCNN_REQUIRE(kind == 0 || kind == 1, "kp_conv_project expects kind 0 (linear) or 1 (gaussian)");
  MCCNN_REQUIRE(sigma > 0.0f, "kp_conv_project expects a positive sigma");
  MCCNN_REQUIRE(num_neighbors >= 0 && num_neighbors < ((int64_t)1 << 31) && num_samples >= 0 &&
                    num_samples < ((int64_t)1 << 31),
                "kp_conv_project expects sizes in [0, 2^31)");
  MCCNN_REQUIRE(num_pts >= 0 && num_pts * num_features < ((int64_t)1 << 30),
                "kp_conv_project expects a feature table of fewer than 2^30 elements");
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && out && points_out && inv_radii && kernel_points &&
                    (num_neighbors == 0 || (points_in && features && neighbors)),
                "kp_conv_project received a null tensor");
  hipStream_t s = as_stream(stream);
  // out is [N_out, C, 16] for up to 16 kernel points and [N_out, C, 32] beyond
  const int kt = num_kernel_points > kFusedK ? 2 : 1;
  int cpl = 1;
  for (int c = 8 / kt; c >= 1; c >>= 1)
    if (num_features % (16 * c) == 0) { cpl = c; break; }
  const int chunks = num_features / (16 * cpl);
  const dim3 grid(wave_grid((num_samples + kProjRun - 1) / kProjRun * chunks)), block(256);
  const int2 *nb = (const int2 *)neighbors;
#define MCCNN_KP_FWD(CPL_, D_, KIND_, KT_)                                                     \
  {                                                                                            \
    McParams<D_> prm{points_in, points_out, inv_radii, nullptr, nullptr, nullptr, 1, 0};       \
    hipLaunchKernelGGL((kp_conv_project16_kernel<CPL_, D_, KIND_, KT_>), grid, block, 0, s,    \
                       num_samples, num_features, chunks, features, nb, ranges, prm,           \
                       kernel_points, num_kernel_points, sigma, out_rows, out);                \
  }
#define MCCNN_KP_FWD_D(CPL_, KT_)                                                  \
  if (num_dims == 3) {                                                             \
    if (kind == 0) MCCNN_KP_FWD(CPL_, 3, 0, KT_) else MCCNN_KP_FWD(CPL_, 3, 1, KT_) \
  } else {                                                                         \
    if (kind == 0) MCCNN_KP_FWD(CPL_, 2, 0, KT_) else MCCNN_KP_FWD(CPL_, 2, 1, KT_) \
  }
  switch (kt * 16 + cpl) {
    case 16 + 8: MCCNN_KP_FWD_D(8, 1); break;
    case 16 + 4: MCCNN_KP_FWD_D(4, 1); break;
    case 16 + 2: MCCNN_KP_FWD_D(2, 1); break;
    case 16 + 1: MCCNN_KP_FWD_D(1, 1); break;
    case 32 + 4: MCCNN_KP_FWD_D(4, 2); break;
    case 32 + 2: MCCNN_KP_FWD_D(2, 2); break;
    default: MCCNN_KP_FWD_D(1, 2); break;
  }
#undef MCCNN_KP_FWD_D
#undef MCCNN_KP_FWD
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

static int check_deform_args(const char *op, int num_dims, int num_features, int num_kernel_points,
                             int kind, float sigma, int64_t num_pts, int64_t num_neighbors,
                             int64_t num_samples) {
  MCCNN_REQUIRE(num_kernel_points > 0 && num_kernel_points <= kFusedK,
                "%s supports 1 to 16 kernel points (got %d)", op, num_kernel_points);
  MCCNN_REQUIRE(kind == 0 || kind == 1, "%s expects kind 0 (linear) or 1 (gaussian)", op);
  MCCNN_REQUIRE(sigma > 0.0f, "%s expects a positive sigma", op);
  MCCNN_REQUIRE(num_neighbors >= 0 && num_neighbors < ((int64_t)1 << 31) && num_samples >= 0 &&
                    num_samples < ((int64_t)1 << 31),
                "%s expects sizes in [0, 2^31)", op);
  MCCNN_REQUIRE(num_pts >= 0 && num_pts * num_features < ((int64_t)1 << 30),
                "%s expects a feature table of fewer than 2^30 elements", op);
  return MCCNN_OK;
}

extern "C" int mccnn_kp_deform_project(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                                       const float *points_in, int num_features,
                                       const float *features, int64_t num_samples,
                                       const float *points_out, int64_t num_neighbors,
                                       const int32_t *neighbors, const int32_t *ranges,
                                       const float *inv_radii, int num_kernel_points,
                                       const float *kernel_points, int kind, float sigma,
                                       const float *offsets, int offsets_follow_points,
                                       const int32_t *out_rows, float *out) {
  MCCNN_REQUIRE(project_supported(num_dims, num_features, kFusedK),
                "kp_deform_project supports D in {2,3} and C in {16, 32, ..., 512} (got D=%d, "
                "C=%d)", num_dims, num_features);
  int rc = check_deform_args("kp_deform_project", num_dims, num_features, num_kernel_points,
                             kind, sigma, num_pts, num_neighbors, num_samples);
  if (rc != MCCNN_OK) return rc;
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && out && points_out && inv_radii && kernel_points &&
                    (num_neighbors == 0 || (points_in && features && neighbors && offsets)),
                "kp_deform_project received a null tensor");
  hipStream_t s = as_stream(stream);
  int cpl = 1;
  for (int c = 8; c >= 1; c >>= 1)
    if (num_features % (16 * c) == 0) { cpl = c; break; }
  const int chunks = num_features / (16 * cpl);
  const dim3 grid(wave_grid((num_samples + kProjRun - 1) / kProjRun * chunks)), block(256);
  const int2 *nb = (const int2 *)neighbors;
#define MCCNN_KPD(CPL_, D_, KIND_)                                                             \
  {                                                                                            \
    McParams<D_> prm{points_in, points_out, inv_radii, nullptr, nullptr, nullptr, 1, 0};       \
    hipLaunchKernelGGL((kp_deform_project16_kernel<CPL_, D_, KIND_>), grid, block, 0, s,       \
                       num_samples, num_features, chunks, features, nb, ranges, prm,           \
                       kernel_points, num_kernel_points, sigma, offsets, offsets_follow_points, \
                       out_rows, out);                                                         \
  }
#define MCCNN_KPD_D(CPL_)                                                  \
  if (num_dims == 3) {                                                     \
    if (kind == 0) MCCNN_KPD(CPL_, 3, 0) else MCCNN_KPD(CPL_, 3, 1)        \
  } else {                                                                 \
    if (kind == 0) MCCNN_KPD(CPL_, 2, 0) else MCCNN_KPD(CPL_, 2, 1)        \
  }
  switch (cpl) {
    case 8: MCCNN_KPD_D(8); break;
    case 4: MCCNN_KPD_D(4); break;
    case 2: MCCNN_KPD_D(2); break;
    default: MCCNN_KPD_D(1); break;
  }
#undef MCCNN_KPD_D
#undef MCCNN_KPD
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}

extern "C" int mccnn_kp_deform_offset_grads_supported(int num_dims, int num_features) {
  return fused_supported(num_dims, num_features, kFusedK, true) ? 1 : 0;
}

extern "C" int mccnn_kp_deform_offset_grads(mccnn_stream_t stream, int num_dims, int64_t num_pts,
                                            const float *points_in, int num_features,
                                            const float *features, int64_t num_samples,
                                            const float *points_out, int64_t num_neighbors,
                                            const int32_t *neighbors, const int32_t *ranges,
                                            const float *inv_radii, int num_kernel_points,
                                            const float *kernel_points, int kind, float sigma,
                                            const float *offsets, const float *in_grads,
                                            float *offset_grads_out) {
  MCCNN_REQUIRE(fused_supported(num_dims, num_features, kFusedK, true),
                "kp_deform_offset_grads supports D in {2,3} and C in {16,32,64,128} (got D=%d, "
                "C=%d)", num_dims, num_features);
  int rc = check_deform_args("kp_deform_offset_grads", num_dims, num_features,
                             num_kernel_points, kind, sigma, num_pts, num_neighbors, num_samples);
  if (rc != MCCNN_OK) return rc;
  if (num_samples == 0) return MCCNN_OK;
  MCCNN_REQUIRE(ranges && offset_grads_out && points_out && inv_radii && kernel_points &&
                    offsets && in_grads && (num_neighbors == 0 || (points_in && features &&
                                                                   neighbors)),
                "kp_deform_offset_grads received a null tensor");
  hipStream_t s = as_stream(stream);
  const dim3 grid((unsigned)grad_blocks(num_samples)), block(256);
  const int2 *nb = (const int2 *)neighbors;
#define MCCNN_KPG(C_, D_, KIND_)                                                               \
  {                                                                                            \
    McParams<D_> prm{points_in, points_out, inv_radii, nullptr, nullptr, nullptr, 1, 0};       \
    hipLaunchKernelGGL((kp_deform_offset_grads16_kernel<C_, D_, KIND_>), grid, block, 0, s,    \
                       num_samples, features, nb, ranges, prm, kernel_points,                  \
                       num_kernel_points, sigma, offsets, in_grads, offset_grads_out);         \
  }
#define MCCNN_KPG_D(C_)                                                  \
  if (num_dims == 3) {                                                   \
    if (kind == 0) MCCNN_KPG(C_, 3, 0) else MCCNN_KPG(C_, 3, 1)          \
  } else {                                                               \
    if (kind == 0) MCCNN_KPG(C_, 2, 0) else MCCNN_KPG(C_, 2, 1)          \
  }
  switch (num_features) {
    case 16: MCCNN_KPG_D(16); break;
    case 32: MCCNN_KPG_D(32); break;
    case 64: MCCNN_KPG_D(64); break;
    default: MCCNN_KPG_D(128); break;
  }
#undef MCCNN_KPG_D
#undef MCCNN_KPG
  MCCNN_LAUNCH_CHECK();
  return MCCNN_OK;
}
