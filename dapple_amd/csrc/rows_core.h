// Row kernels of the fp32 residual stream as device functions (one wave per row), shared by the kernels of their own in
// elementwise.hip and the grouped launches of group.hip.
#pragma once
#include "common.h"

namespace dsrows {

__device__ __forceinline__ void ln_load8(const float* p, float (&v)[8]) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
  for (int e = 0; e < 4; ++e) { v[e] = a[e]; v[4 + e] = b[e]; }
}
__device__ __forceinline__ void ln_store8(float* p, const float (&v)[8]) {
  const f32x4 a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
  *reinterpret_cast<f32x4*>(p) = a;
  *reinterpret_cast<f32x4*>(p + 4) = b;
}
__device__ __forceinline__ void ln_store8(bf16* p, const float (&v)[8]) {
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (bf16)v[e];
  *reinterpret_cast<bf16x8*>(p) = o;
}

// y = LayerNorm(x): x fp32, y16 bf16, y32 (nullable) fp32.  One wave per row, NG groups of 8 columns per lane.
template <int NG>
__device__ __forceinline__ void layernorm_fwd_mixed_row(int row, int lane, int rows, int cols, const float* __restrict__ x,
                                                                 const float* __restrict__ gamma, const float* __restrict__ beta,
                                                                 float eps, bf16* __restrict__ y16, float* __restrict__ y32,
                                                                 float* __restrict__ stats) {
  if (row >= rows) return;
  const float* xr = x + (int64_t)row * cols;
  float v[NG][8], gm[NG][8], bt[NG][8];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int c = (lane + i * 64) * 8;
    if (c < cols) {
      ln_load8(xr + c, v[i]);
      ln_load8(gamma + c, gm[i]);  // with x: read where they are used they would cost a second trip to memory
      ln_load8(beta + c, bt[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) sum += v[i][e];
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[i][e] = 0.f;
    }
  }
  const float mean = wave_sum(sum) / cols;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < NG; ++i)
    if ((lane + i * 64) * 8 < cols) {
#pragma unroll
      for (int e = 0; e < 8; ++e) { const float d = v[i][e] - mean; sq += d * d; }
    }
  const float rstd = rsqrtf(wave_sum(sq) / cols + eps);
  if (lane == 0 && stats) { stats[2 * row] = mean; stats[2 * row + 1] = rstd; }
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int c = (lane + i * 64) * 8;
    if (c < cols) {
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (v[i][e] - mean) * rstd * gm[i][e] + bt[i][e];
      ln_store8(y16 + (int64_t)row * cols + c, o);
      if (y32) ln_store8(y32 + (int64_t)row * cols + c, o);
    }
  }
}

// The same backward pass without the parameter gradients: one wave per row, no LDS, no atomics - the form for a chain
// of dependent kernels.  dy16 (nullable) receives a bf16 copy of dy: with x and stats (kept by the caller) and dx16 it is
// all layernorm_param_grad_mixed_kernel needs to produce d_gamma, d_beta and the column sums of dx later, elsewhere.
// dy32 / rowsums (nullable) are the same hand-over without rounding: an fp32 copy of dy and, per row, the two means
// (of dy gamma and of dy gamma x_hat) from which layernorm_param_grad_exact_kernel rebuilds the fp32 dx.
template <int NG>
__device__ __forceinline__ void layernorm_bwd_mixed_rows_row(int row, int lane, int rows, int cols, const float* __restrict__ dy,
                                                                      const float* __restrict__ x, const float* __restrict__ gamma,
                                                                      const float* __restrict__ stats, bf16* __restrict__ dx16,
                                                                      float* __restrict__ dx32, bf16* __restrict__ dy16,
                                                                      float* __restrict__ dy32 = nullptr, float* __restrict__ rowsums = nullptr) {
  if (row >= rows) return;
  const int64_t ro = (int64_t)row * cols;
  float a[NG][8], b[NG][8], g[NG][8];
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int c = (lane + i * 64) * 8;
    if (c < cols) {
      ln_load8(dy + ro + c, a[i]);
      ln_load8(x + ro + c, b[i]);
      ln_load8(gamma + c, g[i]);
    }
  }
  const float mean = stats[2 * row], rstd = stats[2 * row + 1];
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int c = (lane + i * 64) * 8;
    if (c < cols) {
      if (dy16) ln_store8(dy16 + ro + c, a[i]);
      if (dy32) ln_store8(dy32 + ro + c, a[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        b[i][e] = (b[i][e] - mean) * rstd;
        a[i][e] *= g[i][e];
        s1 += a[i][e];
        s2 += a[i][e] * b[i][e];
      }
    }
  }
  s1 = wave_sum(s1) / cols;
  s2 = wave_sum(s2) / cols;
  if (rowsums && lane == 0) { rowsums[2 * row] = s1; rowsums[2 * row + 1] = s2; }
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int c = (lane + i * 64) * 8;
    if (c < cols) {
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = rstd * (a[i][e] - s1 - b[i][e] * s2);
      ln_store8(dx16 + ro + c, o);
      if (dx32) ln_store8(dx32 + ro + c, o);
    }
  }
}

}  // namespace dsrows
