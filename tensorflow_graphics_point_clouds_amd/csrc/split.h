// float32 products on the bf16 matrix pipe.
//
// A float32 value x is split into three bfloat16 parts x = x1 + x2 + x3 (x1 = bf16(x),
// x2 = bf16(x - x1), x3 = bf16(x - x1 - x2); the differences are exact and the three parts
// carry the 24 bits of x).  A product x * w is then the sum of the nine part products, each
// exact in float32; the six of them with i + j <= 4,
//     x1 w1 + (x1 w2 + x2 w1) + (x1 w3 + x2 w2 + x3 w1),
// leave out terms below 2^-24 |x w| -- what one float32 rounding of the product would lose.
// v_mfma_f32_32x32x16_bf16 multiplies 16 pairs per lane and instruction with float32
// accumulation at sixteen times the rate of v_mfma_f32_16x16x4_f32, so the six instructions
// that stand for one float32 matrix step still take 2.7 times less of the matrix pipe.
// Measured error of a 1024-term sum against float64: 1.7e-7 of the sum of the absolute
// values of its terms, the same as a serial float32 sum of the same terms.
#pragma once
#include "common.h"
#include "mfma.h"

namespace mccnn {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

struct Split8 {
  v8bf p[3];
};

// Two values at a time: one packed conversion per part (v_cvt_pk_bf16_f32, round to nearest
// even) and the float value of each half of the packed word from a shift or a mask --
// 5.5 vector instructions per value, against 7.5 when every value is converted on its own.
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

__device__ __forceinline__ v2f widen2(v2bf packed) {
  const unsigned u = __builtin_bit_cast(unsigned, packed);
  return v2f{__uint_as_float(u << 16), __uint_as_float(u & 0xffff0000u)};
}

__device__ __forceinline__ Split8 split8(const v4f &lo, const v4f &hi) {
  Split8 s;
  unsigned w[3][4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const v2f x = e < 2 ? v2f{lo[2 * e], lo[2 * e + 1]} : v2f{hi[2 * e - 4], hi[2 * e - 3]};
    const v2bf a = __builtin_convertvector(x, v2bf);
    const v2f r1 = x - widen2(a);
    const v2bf b = __builtin_convertvector(r1, v2bf);
    const v2f r2 = r1 - widen2(b);
    const v2bf c = __builtin_convertvector(r2, v2bf);
    w[0][e] = __builtin_bit_cast(unsigned, a);
    w[1][e] = __builtin_bit_cast(unsigned, b);
    w[2][e] = __builtin_bit_cast(unsigned, c);
  }
#pragma unroll
  for (int q = 0; q < 3; ++q) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const v4u packed = {w[q][0], w[q][1], w[q][2], w[q][3]};
    s.p[q] = __builtin_bit_cast(v8bf, packed);
  }
  return s;
}

// acc += a * b for one 32 x 32 x 16 step, smallest terms first.
__device__ __forceinline__ v16f mma_split(const Split8 &a, const Split8 &b, v16f acc) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p[2], b.p[0], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p[0], b.p[2], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p[1], b.p[1], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p[1], b.p[0], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p[0], b.p[1], acc, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p[0], b.p[0], acc, 0, 0, 0);
}

// Whether the dense products of the layers run on the bf16 pipe (default) or keep the
// float32 matrix instructions (mccnn_set_split_products(0), or MCCNN_DENSE_FP32=1 in the
// environment of the process).
bool split_products_enabled();

// out[n, r] = sum_f x[n, f] * w[r, f] (defined in split_dense.hip).
bool nt_split_supported(int F, int R);
int launch_nt_split(hipStream_t s, int64_t n, int F, const float *x, int R, const float *w,
                    float *out);


// out = x * w for x [N, R] and wt = w^T [F, R] as a tiled product (defined in split_dense.hip);
// same shapes as the float32 tiled product of dense.hip.
int launch_tile_split(hipStream_t s, int64_t n, int R, const float *x, int F, const float *wt,
                      const int *out_rows, float *out);

// Partial sums of out[c, r] = sum_n x[n, c] * y[n, r] per slice of the points (defined in
// split_dense.hip): partials [slices, C, R], to be added up in slice order.
bool tn_split_supported(int C, int R);
int tn_split_slices(int C, int R);
int launch_tn_split(hipStream_t s, int64_t n, int C, const float *x, int R, const float *y,
                    int slices, float *partials);

}  // namespace mccnn
