// HBM-bound kernels: gradient accumulation, casts, LayerNorm, softmax, column sums.
// All move data as 16-byte vectors per lane with grid-stride or one-wave-per-row mappings.
#include <stdlib.h>
#include <string.h>

#include "common.h"
#include "rows_core.h"

namespace {

// ------------------------------------------------------------------ accumulate / cast
// acc[i] += g[i]; 12 B/element (fp32 g) or 10 B/element (bf16 g) of HBM traffic.
template <typename G>
__global__ __launch_bounds__(256) void accumulate_kernel(float* __restrict__ acc, const G* __restrict__ g, size_t n) {
  constexpr int VEC = Vec16<G>::N;
  typedef typename Vec16<G>::type GV;
  const size_t nvec = n / VEC;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += stride) {
    const GV gv = reinterpret_cast<const GV*>(g)[v];
    f32x4* ap = reinterpret_cast<f32x4*>(acc) + v * (VEC / 4);
#pragma unroll
    for (int q = 0; q < VEC / 4; ++q) {
      f32x4 a = ap[q];
#pragma unroll
      for (int e = 0; e < 4; ++e) a[e] += to_f32(gv[q * 4 + e]);
      ap[q] = a;
    }
  }
  // tail (n not a multiple of the vector width)
  const size_t tail0 = nvec * VEC;
  const size_t t = tail0 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) acc[t] += to_f32(g[t]);
}

template <typename D, typename S>
__global__ __launch_bounds__(256) void cast_kernel(D* __restrict__ dst, const S* __restrict__ src, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x * 4;
  for (size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < n; i += stride) {
    if (i + 4 <= n) {
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[i + e] = from_f32<D>(to_f32(src[i + e]));
    } else {
      for (size_t e = i; e < n; ++e) dst[e] = from_f32<D>(to_f32(src[e]));
    }
  }
}

inline int grid_for(size_t work_items, int per_block) {
  size_t b = (work_items + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > 256 * 16) b = 256 * 16;
  return (int)b;
}

// ------------------------------------------------------------------ LayerNorm
// One wave per row; a lane keeps NV 16-byte vectors of the row in registers.
template <typename T, int NV>
__global__ __launch_bounds__(256) void layernorm_fwd_kernel(int rows, int cols, const T* __restrict__ x,
                                                           const float* __restrict__ gamma,
                                                           const float* __restrict__ beta, float eps,
                                                           T* __restrict__ y, float* __restrict__ stats) {
  constexpr int VEC = Vec16<T>::N;
  typedef typename Vec16<T>::type V;
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + (int64_t)row * cols;
  float v[NV][VEC], gm[NV][VEC], bt[NV][VEC];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * VEC;
    if (c < cols) {
      const V t = *reinterpret_cast<const V*>(xr + c);
      // gamma and beta are fetched here, with x: read where they are used they would cost a second trip to memory
      // behind the two reductions
#pragma unroll
      for (int e = 0; e < VEC; e += 4) {
        const f32x4 g4 = *reinterpret_cast<const f32x4*>(gamma + c + e), b4 = *reinterpret_cast<const f32x4*>(beta + c + e);
#pragma unroll
        for (int q = 0; q < 4; ++q) { gm[i][e + q] = g4[q]; bt[i][e + q] = b4[q]; }
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) { v[i][e] = to_f32(t[e]); sum += v[i][e]; }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[i][e] = 0.f;
    }
  }
  const float mean = wave_sum(sum) / cols;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * VEC;
    if (c < cols) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) { const float d = v[i][e] - mean; sq += d * d; }
    }
  }
  const float rstd = rsqrtf(wave_sum(sq) / cols + eps);
  if (lane == 0 && stats) { stats[2 * row] = mean; stats[2 * row + 1] = rstd; }
  T* yr = y + (int64_t)row * cols;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * VEC;
    if (c < cols) {
      V o;
#pragma unroll
      for (int e = 0; e < VEC; ++e) o[e] = from_f32<T>((v[i][e] - mean) * rstd * gm[i][e] + bt[i][e]);
      *reinterpret_cast<V*>(yr + c) = o;
    }
  }
}

// Backward: each wave walks ROWS_PER_WAVE rows and keeps the column partial sums of
// d_gamma, d_beta and dx in registers; the 4 waves of a block combine through LDS and
// issue one atomicAdd per column and quantity.
template <typename T, int NV>
__global__ __launch_bounds__(256) void layernorm_bwd_kernel(int rows, int cols, int rows_per_wave,
                                                           const T* __restrict__ dy, const T* __restrict__ x,
                                                           const float* __restrict__ gamma,
                                                           const float* __restrict__ stats,
                                                           const T* __restrict__ dx_add, T* __restrict__ dx,
                                                           float* __restrict__ d_gamma, float* __restrict__ d_beta,
                                                           float* __restrict__ d_colsum) {
  constexpr int VEC = Vec16<T>::N;
  typedef typename Vec16<T>::type V;
  extern __shared__ __attribute__((aligned(16))) float red[];  // [3][cols]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float g[NV][VEC], pg[NV][VEC], pb[NV][VEC], ps[NV][VEC];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * VEC;
#pragma unroll
    for (int e = 0; e < VEC; e += 4) {  // whole 16-byte vectors: a predicate per element keeps the loads scalar
      f32x4 gv = {0.f, 0.f, 0.f, 0.f};
      if (c < cols) gv = *reinterpret_cast<const f32x4*>(gamma + c + e);
      g[i][e] = gv[0]; g[i][e + 1] = gv[1]; g[i][e + 2] = gv[2]; g[i][e + 3] = gv[3];
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) pg[i][e] = pb[i][e] = ps[i][e] = 0.f;
  }
  const int row0 = (blockIdx.x * 4 + wave) * rows_per_wave;
  // the next row's dy, x and statistics are fetched before this row is reduced and written: one trip to memory per
  // wave, not one per row
  V na[NV], nb[NV];
  float nmean = 0.f, nrstd = 0.f;
  auto fetch = [&](int row) {
    if (row >= rows) return;
    nmean = stats[2 * row]; nrstd = stats[2 * row + 1];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = (lane + i * 64) * VEC;
      if (c < cols) {
        na[i] = *reinterpret_cast<const V*>(dy + (int64_t)row * cols + c);
        nb[i] = *reinterpret_cast<const V*>(x + (int64_t)row * cols + c);
      }
    }
  };
  fetch(row0);
  for (int r = 0; r < rows_per_wave; ++r) {
    const int row = row0 + r;
    if (row >= rows) break;
    const float mean = nmean, rstd = nrstd;
    V ca[NV], cb[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) { ca[i] = na[i]; cb[i] = nb[i]; }
    if (r + 1 < rows_per_wave) fetch(row + 1);
    float dyv[NV][VEC], xh[NV][VEC];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = (lane + i * 64) * VEC;
      if (c < cols) {
        const V a = ca[i];
        const V b = cb[i];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          dyv[i][e] = to_f32(a[e]);
          xh[i][e] = (to_f32(b[e]) - mean) * rstd;
          const float dxh = dyv[i][e] * g[i][e];
          s1 += dxh;
          s2 += dxh * xh[i][e];
          pg[i][e] += dyv[i][e] * xh[i][e];
          pb[i][e] += dyv[i][e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) { dyv[i][e] = 0.f; xh[i][e] = 0.f; }
      }
    }
    s1 = wave_sum(s1) / cols;
    s2 = wave_sum(s2) / cols;
    T* dxr = dx + (int64_t)row * cols;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = (lane + i * 64) * VEC;
      if (c < cols) {
        V o;
        V add = {};
        if (dx_add) add = *reinterpret_cast<const V*>(dx_add + (int64_t)row * cols + c);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float d = rstd * (dyv[i][e] * g[i][e] - s1 - xh[i][e] * s2);
          ps[i][e] += d;
          o[e] = from_f32<T>(d + (dx_add ? to_f32(add[e]) : 0.f));
        }
        *reinterpret_cast<V*>(dxr + c) = o;
      }
    }
  }
  // combine the 4 waves' column partials in LDS, one wave at a time (plain vector stores / read-modify-writes:
  // LDS float atomics on 32-byte-strided addresses serialise 16 ways; parking all four sets and summing them in
  // one step needs 4x the LDS, which costs more in co-residency with other kernels than the barriers it saves)
  for (int wv = 0; wv < 4; ++wv) {
    if (wave == wv) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int c = (lane + i * 64) * VEC;
        if (c < cols) {
#pragma unroll
          for (int e = 0; e < VEC; e += 4) {
            f32x4* r0 = reinterpret_cast<f32x4*>(&red[c + e]);
            f32x4* r1 = reinterpret_cast<f32x4*>(&red[cols + c + e]);
            f32x4* r2 = reinterpret_cast<f32x4*>(&red[2 * cols + c + e]);
            f32x4 a0 = {pg[i][e], pg[i][e + 1], pg[i][e + 2], pg[i][e + 3]};
            f32x4 a1 = {pb[i][e], pb[i][e + 1], pb[i][e + 2], pb[i][e + 3]};
            f32x4 a2 = {ps[i][e], ps[i][e + 1], ps[i][e + 2], ps[i][e + 3]};
            if (wv > 0) { a0 += *r0; a1 += *r1; a2 += *r2; }
            *r0 = a0; *r1 = a1; *r2 = a2;
          }
        }
      }
    }
    __syncthreads();
  }
  for (int c = threadIdx.x; c < cols; c += 256) {
    atomicAdd(d_gamma + c, red[c]);
    atomicAdd(d_beta + c, red[cols + c]);
    if (d_colsum) atomicAdd(d_colsum + c, red[2 * cols + c]);
  }
}

// ------------------------------------------------------------------ LayerNorm on an fp32 residual stream
// A bf16 stage that keeps its residual stream (the sums in front of every LayerNorm and the LayerNorm outputs that
// feed the next sum) in fp32 rounds to bf16 only where a tensor becomes a GEMM operand.  These kernels read fp32 and
// write the bf16 operand copy and, optionally, the fp32 carrier; a lane owns groups of 8 consecutive columns.
using dsrows::ln_load8;
using dsrows::ln_store8;

// y = LayerNorm(x): x fp32, y16 bf16, y32 (nullable) fp32.  One wave per row, NG groups of 8 columns per lane.
template <int NG>
__global__ __launch_bounds__(256) void layernorm_fwd_mixed_kernel(int rows, int cols, const float* __restrict__ x,
                                                                 const float* __restrict__ gamma, const float* __restrict__ beta,
                                                                 float eps, bf16* __restrict__ y16, float* __restrict__ y32,
                                                                 float* __restrict__ stats, int prio) {
  ds_wave_prio(prio);
  dsrows::layernorm_fwd_mixed_row<NG>(blockIdx.x * 4 + (threadIdx.x >> 6), threadIdx.x & 63, rows, cols, x, gamma, beta, eps, y16, y32, stats);
}

// Backward of the same: dy, x fp32 in; dx16 bf16 and dx32 (nullable) fp32 out; the parameter gradients and the column
// sums of dx as in layernorm_bwd_kernel (column partials per wave, combined through LDS, one atomic per column and block).
template <int NG>
__global__ __launch_bounds__(256) void layernorm_bwd_mixed_kernel(int rows, int cols, int rows_per_wave, const float* __restrict__ dy,
                                                                 const float* __restrict__ x, const float* __restrict__ gamma,
                                                                 const float* __restrict__ stats, bf16* __restrict__ dx16,
                                                                 float* __restrict__ dx32, float* __restrict__ d_gamma,
                                                                 float* __restrict__ d_beta, float* __restrict__ d_colsum) {
  extern __shared__ __attribute__((aligned(16))) float red[];  // [3][cols]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float g[NG][8], pg[NG][8], pb[NG][8], ps[NG][8];
#pragma unroll
  for (int i = 0; i < NG; ++i) {
    const int c = (lane + i * 64) * 8;
    if (c < cols) ln_load8(gamma + c, g[i]);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (c >= cols) g[i][e] = 0.f;
      pg[i][e] = pb[i][e] = ps[i][e] = 0.f;
    }
  }
  const int row0 = (blockIdx.x * 4 + wave) * rows_per_wave;
  // the next row's operands are in flight while this row is reduced and written
  float na[NG][8], nb[NG][8];
  float nmean = 0.f, nrstd = 0.f;
  auto fetch = [&](int row) {
    if (row >= rows) return;
    nmean = stats[2 * row]; nrstd = stats[2 * row + 1];
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int c = (lane + i * 64) * 8;
      if (c < cols) {
        ln_load8(dy + (int64_t)row * cols + c, na[i]);
        ln_load8(x + (int64_t)row * cols + c, nb[i]);
      }
    }
  };
  fetch(row0);
  for (int r = 0; r < rows_per_wave; ++r) {
    const int row = row0 + r;
    if (row >= rows) break;
    const float mean = nmean, rstd = nrstd;
    float dyv[NG][8], xh[NG][8];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const bool in = (lane + i * 64) * 8 < cols;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        dyv[i][e] = in ? na[i][e] : 0.f;
        xh[i][e] = in ? (nb[i][e] - mean) * rstd : 0.f;
        const float dxh = dyv[i][e] * g[i][e];
        s1 += dxh;
        s2 += dxh * xh[i][e];
        pg[i][e] += dyv[i][e] * xh[i][e];
        pb[i][e] += dyv[i][e];
      }
    }
    if (r + 1 < rows_per_wave) fetch(row + 1);
    s1 = wave_sum(s1) / cols;
    s2 = wave_sum(s2) / cols;
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int c = (lane + i * 64) * 8;
      if (c < cols) {
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          o[e] = rstd * (dyv[i][e] * g[i][e] - s1 - xh[i][e] * s2);
          ps[i][e] += o[e];
        }
        ln_store8(dx16 + (int64_t)row * cols + c, o);
        if (dx32) ln_store8(dx32 + (int64_t)row * cols + c, o);
      }
    }
  }
  for (int wv = 0; wv < 4; ++wv) {
    if (wave == wv) {
#pragma unroll
      for (int i = 0; i < NG; ++i) {
        const int c = (lane + i * 64) * 8;
        if (c < cols) {
#pragma unroll
          for (int e = 0; e < 8; e += 4) {
            f32x4* r0 = reinterpret_cast<f32x4*>(&red[c + e]);
            f32x4* r1 = reinterpret_cast<f32x4*>(&red[cols + c + e]);
            f32x4* r2 = reinterpret_cast<f32x4*>(&red[2 * cols + c + e]);
            f32x4 a0 = {pg[i][e], pg[i][e + 1], pg[i][e + 2], pg[i][e + 3]};
            f32x4 a1 = {pb[i][e], pb[i][e + 1], pb[i][e + 2], pb[i][e + 3]};
            f32x4 a2 = {ps[i][e], ps[i][e + 1], ps[i][e + 2], ps[i][e + 3]};
            if (wv > 0) { a0 += *r0; a1 += *r1; a2 += *r2; }
            *r0 = a0; *r1 = a1; *r2 = a2;
          }
        }
      }
    }
    __syncthreads();
  }
  for (int c = threadIdx.x; c < cols; c += 256) {
    atomicAdd(d_gamma + c, red[c]);
    atomicAdd(d_beta + c, red[cols + c]);
    if (d_colsum) atomicAdd(d_colsum + c, red[2 * cols + c]);
  }
}

// The backward pass without the parameter gradients: one wave per row, no LDS, no atomics - the form for a chain of
// dependent kernels (dsrows::layernorm_bwd_mixed_rows_row).
template <int NG>
__global__ __launch_bounds__(256) void layernorm_bwd_mixed_rows_kernel(int rows, int cols, const float* __restrict__ dy,
                                                                      const float* __restrict__ x, const float* __restrict__ gamma,
                                                                      const float* __restrict__ stats, bf16* __restrict__ dx16,
                                                                      float* __restrict__ dx32, bf16* __restrict__ dy16, float* __restrict__ dy32,
                                                                      float* __restrict__ rowsums, int prio) {
  ds_wave_prio(prio);
  dsrows::layernorm_bwd_mixed_rows_row<NG>(blockIdx.x * 4 + (threadIdx.x >> 6), threadIdx.x & 63, rows, cols, dy, x, gamma, stats, dx16, dx32, dy16,
                                           dy32, rowsums);
}

// d_gamma[c] += sum_rows dy x_hat, d_beta[c] += sum_rows dy, d_colsum[c] += sum_rows dx (dx, d_colsum nullable) from the
// bf16 copies layernorm_bwd_mixed_rows_kernel left and the fp32 x.  A block owns a strip of 64 x 8 columns and a chunk
// of rows; its 4 waves take every 4th row and meet in LDS; one atomic per column and block.
__global__ __launch_bounds__(256) void layernorm_param_grad_mixed_kernel(int rows, int cols, int rows_per_block,
                                                                        const bf16* __restrict__ dy, const float* __restrict__ x,
                                                                        const float* __restrict__ stats, const bf16* __restrict__ dx,
                                                                        float* __restrict__ d_gamma, float* __restrict__ d_beta,
                                                                        float* __restrict__ d_colsum) {
  __shared__ float red[3][4][64 * 8];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int c = (blockIdx.x * 64 + lane) * 8;
  const int r0 = blockIdx.y * rows_per_block;
  int r1 = r0 + rows_per_block;
  if (r1 > rows) r1 = rows;
  float pg[8], pb[8], ps[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) pg[e] = pb[e] = ps[e] = 0.f;
  if (c < cols) {
    // two rows in flight per wave
    for (int r = r0 + g; r < r1; r += 8) {
      const int rb = r + 4;
      const bool two = rb < r1;
      const bf16x8 a0 = *reinterpret_cast<const bf16x8*>(dy + (int64_t)r * cols + c);
      float b0[8], b1[8];
      ln_load8(x + (int64_t)r * cols + c, b0);
      const float mean0 = stats[2 * r], rstd0 = stats[2 * r + 1];
      bf16x8 a1 = {}, v0 = {}, v1 = {};
      float mean1 = 0.f, rstd1 = 0.f;
      if (dx) v0 = *reinterpret_cast<const bf16x8*>(dx + (int64_t)r * cols + c);
      if (two) {
        a1 = *reinterpret_cast<const bf16x8*>(dy + (int64_t)rb * cols + c);
        ln_load8(x + (int64_t)rb * cols + c, b1);
        mean1 = stats[2 * rb]; rstd1 = stats[2 * rb + 1];
        if (dx) v1 = *reinterpret_cast<const bf16x8*>(dx + (int64_t)rb * cols + c);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = to_f32(a0[e]);
        pg[e] += d * (b0[e] - mean0) * rstd0;
        pb[e] += d;
        ps[e] += to_f32(v0[e]);
      }
      if (two) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float d = to_f32(a1[e]);
          pg[e] += d * (b1[e] - mean1) * rstd1;
          pb[e] += d;
          ps[e] += to_f32(v1[e]);
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    red[0][g][lane * 8 + e] = pg[e];
    red[1][g][lane * 8 + e] = pb[e];
    red[2][g][lane * 8 + e] = ps[e];
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * 8; i += 256) {
    const int p = blockIdx.x * 64 * 8 + i;
    if (p < cols) {
      atomicAdd(d_gamma + p, red[0][0][i] + red[0][1][i] + red[0][2][i] + red[0][3][i]);
      atomicAdd(d_beta + p, red[1][0][i] + red[1][1][i] + red[1][2][i] + red[1][3][i]);
      if (d_colsum) atomicAdd(d_colsum + p, red[2][0][i] + red[2][1][i] + red[2][2][i] + red[2][3][i]);
    }
  }
}

// The same sums without rounding: dy comes as the fp32 copy, and dx is rebuilt in fp32 from the two per-row means the
// row kernel left (dx = rstd (dy gamma - s1 - x_hat s2)), so the results equal those of layernorm_bwd_mixed_kernel up
// to the order of the fp32 additions.  Same block shape as layernorm_param_grad_mixed_kernel.
// x and stats may come in segments of seg_rows rows whose starts are x_seg / st_seg elements apart (activations of several
// micro-batches in different stash slots); dy and rowsums are always one run of rows.
__global__ __launch_bounds__(256) void layernorm_param_grad_exact_kernel(int rows, int cols, int rows_per_block, const float* __restrict__ dy,
                                                                        const float* __restrict__ x, const float* __restrict__ gamma,
                                                                        const float* __restrict__ stats, const float* __restrict__ rowsums,
                                                                        float* __restrict__ d_gamma, float* __restrict__ d_beta,
                                                                        float* __restrict__ d_colsum, int seg_rows, int64_t x_seg, int64_t st_seg) {
  __shared__ float red[3][4][64 * 8];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int c = (blockIdx.x * 64 + lane) * 8;
  const int r0 = blockIdx.y * rows_per_block;
  int r1 = r0 + rows_per_block;
  if (r1 > rows) r1 = rows;
  float pg[8], pb[8], ps[8], gm[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) pg[e] = pb[e] = ps[e] = gm[e] = 0.f;
  if (c < cols) {
    ln_load8(gamma + c, gm);
    // two rows in flight per wave
    for (int r = r0 + g; r < r1; r += 8) {
      const int rb = r + 4;
      const bool two = rb < r1;
      float a0[8], b0[8], a1[8], b1[8];
      const int sg0 = r / seg_rows, w0 = r - sg0 * seg_rows;
      const float* st0 = stats + sg0 * st_seg + 2 * w0;
      ln_load8(dy + (int64_t)r * cols + c, a0);
      ln_load8(x + sg0 * x_seg + (int64_t)w0 * cols + c, b0);
      const float mean0 = st0[0], rstd0 = st0[1], s10 = rowsums[2 * r], s20 = rowsums[2 * r + 1];
      float mean1 = 0.f, rstd1 = 0.f, s11 = 0.f, s21 = 0.f;
      if (two) {
        const int sg1 = rb / seg_rows, w1 = rb - sg1 * seg_rows;
        const float* st1 = stats + sg1 * st_seg + 2 * w1;
        ln_load8(dy + (int64_t)rb * cols + c, a1);
        ln_load8(x + sg1 * x_seg + (int64_t)w1 * cols + c, b1);
        mean1 = st1[0]; rstd1 = st1[1]; s11 = rowsums[2 * rb]; s21 = rowsums[2 * rb + 1];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xh = (b0[e] - mean0) * rstd0;
        pg[e] += a0[e] * xh;
        pb[e] += a0[e];
        ps[e] += rstd0 * (a0[e] * gm[e] - s10 - xh * s20);
      }
      if (two) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float xh = (b1[e] - mean1) * rstd1;
          pg[e] += a1[e] * xh;
          pb[e] += a1[e];
          ps[e] += rstd1 * (a1[e] * gm[e] - s11 - xh * s21);
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    red[0][g][lane * 8 + e] = pg[e];
    red[1][g][lane * 8 + e] = pb[e];
    red[2][g][lane * 8 + e] = ps[e];
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * 8; i += 256) {
    const int p = blockIdx.x * 64 * 8 + i;
    if (p < cols) {
      atomicAdd(d_gamma + p, red[0][0][i] + red[0][1][i] + red[0][2][i] + red[0][3][i]);
      atomicAdd(d_beta + p, red[1][0][i] + red[1][1][i] + red[1][2][i] + red[1][3][i]);
      if (d_colsum) atomicAdd(d_colsum + p, red[2][0][i] + red[2][1][i] + red[2][2][i] + red[2][3][i]);
    }
  }
}

// Backward without the parameter gradients: one wave per row, dx only.  For callers that take d_gamma / d_beta (and the
// column sums of dx) from layernorm_param_grad_kernel on another stream, off the chain of dependent kernels.
template <typename T, int NV>
__global__ __launch_bounds__(256) void layernorm_bwd_rows_kernel(int rows, int cols, const T* __restrict__ dy, const T* __restrict__ x,
                                                                const float* __restrict__ gamma, const float* __restrict__ stats,
                                                                const T* __restrict__ dx_add, T* __restrict__ dx) {
  constexpr int VEC = Vec16<T>::N;
  typedef typename Vec16<T>::type V;
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float mean = stats[2 * row], rstd = stats[2 * row + 1];
  const T* dyr = dy + (int64_t)row * cols;
  const T* xr = x + (int64_t)row * cols;
  float dg[NV][VEC], xh[NV][VEC];
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * VEC;
    if (c < cols) {
      const V a = *reinterpret_cast<const V*>(dyr + c);
      const V b = *reinterpret_cast<const V*>(xr + c);
#pragma unroll
      for (int e = 0; e < VEC; e += 4) {
        const f32x4 gv = *reinterpret_cast<const f32x4*>(gamma + c + e);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          xh[i][e + k] = (to_f32(b[e + k]) - mean) * rstd;
          dg[i][e + k] = to_f32(a[e + k]) * gv[k];
          s1 += dg[i][e + k];
          s2 += dg[i][e + k] * xh[i][e + k];
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) { dg[i][e] = 0.f; xh[i][e] = 0.f; }
    }
  }
  s1 = wave_sum(s1) / cols;
  s2 = wave_sum(s2) / cols;
  T* dxr = dx + (int64_t)row * cols;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * VEC;
    if (c < cols) {
      V o;
      V add = {};
      if (dx_add) add = *reinterpret_cast<const V*>(dx_add + (int64_t)row * cols + c);
#pragma unroll
      for (int e = 0; e < VEC; ++e) o[e] = from_f32<T>(rstd * (dg[i][e] - s1 - xh[i][e] * s2) + (dx_add ? to_f32(add[e]) : 0.f));
      *reinterpret_cast<V*>(dxr + c) = o;
    }
  }
}

// d_gamma[c] += sum_rows dy x_hat, d_beta[c] += sum_rows dy, d_colsum[c] += sum_rows dx (dx nullable).  A block owns a
// strip of 64 16-byte vectors and a chunk of rows; its 4 waves take every 4th row and meet in LDS.
template <typename T>
__global__ __launch_bounds__(256) void layernorm_param_grad_kernel(int rows, int cols, int rows_per_block, const T* __restrict__ dy,
                                                                  const T* __restrict__ x, const float* __restrict__ stats,
                                                                  const T* __restrict__ dx, float* __restrict__ d_gamma,
                                                                  float* __restrict__ d_beta, float* __restrict__ d_colsum) {
  constexpr int VEC = Vec16<T>::N;
  typedef typename Vec16<T>::type V;
  __shared__ float red[3][4][64 * VEC];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int c = (blockIdx.x * 64 + lane) * VEC;
  const int r0 = blockIdx.y * rows_per_block;
  int r1 = r0 + rows_per_block;
  if (r1 > rows) r1 = rows;
  float pg[VEC], pb[VEC], ps[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) pg[e] = pb[e] = ps[e] = 0.f;
  if (c < cols)
    for (int r = r0 + g; r < r1; r += 4) {
      const float mean = stats[2 * r], rstd = stats[2 * r + 1];
      const V a = *reinterpret_cast<const V*>(dy + (int64_t)r * cols + c);
      const V b = *reinterpret_cast<const V*>(x + (int64_t)r * cols + c);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float d = to_f32(a[e]);
        pg[e] += d * (to_f32(b[e]) - mean) * rstd;
        pb[e] += d;
      }
      if (dx) {
        const V v = *reinterpret_cast<const V*>(dx + (int64_t)r * cols + c);
#pragma unroll
        for (int e = 0; e < VEC; ++e) ps[e] += to_f32(v[e]);
      }
    }
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    red[0][g][lane * VEC + e] = pg[e];
    red[1][g][lane * VEC + e] = pb[e];
    red[2][g][lane * VEC + e] = ps[e];
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * VEC; i += 256) {
    const int p = blockIdx.x * 64 * VEC + i;
    if (p < cols) {
      atomicAdd(d_gamma + p, red[0][0][i] + red[0][1][i] + red[0][2][i] + red[0][3][i]);
      atomicAdd(d_beta + p, red[1][0][i] + red[1][1][i] + red[1][2][i] + red[1][3][i]);
      if (d_colsum) atomicAdd(d_colsum + p, red[2][0][i] + red[2][1][i] + red[2][2][i] + red[2][3][i]);
    }
  }
}

// ------------------------------------------------------------------ softmax
// One wave per row of fp32 scores; NV 16-byte vectors (4 floats) per lane.
template <typename T, int NV>
__global__ __launch_bounds__(256) void softmax_fwd_kernel(int64_t rows, int k, int rows_per_batch,
                                                         const float* __restrict__ scores, float scale,
                                                         const float* __restrict__ key_mask, float mask_value,
                                                         T* __restrict__ p) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* sr = scores + row * k;
  const float* mk = key_mask ? key_mask + (row / rows_per_batch) * k : nullptr;
  float v[NV][4];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * 4;
    if (c < k) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(sr + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float s = t[e] * scale;
        if (mk) s += (1.0f - mk[c + e]) * mask_value;
        v[i][e] = s;
        mx = fmaxf(mx, s);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[i][e] = -INFINITY;
    }
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) { v[i][e] = expf(v[i][e] - mx); sum += v[i][e]; }
  const float inv = 1.0f / wave_sum(sum);
  T* pr = p + row * k;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * 4;
    if (c < k) {
#pragma unroll
      for (int e = 0; e < 4; ++e) pr[c + e] = from_f32<T>(v[i][e] * inv);
    }
  }
}

template <typename T, int NV>
__global__ __launch_bounds__(256) void softmax_bwd_kernel(int64_t rows, int k, const T* __restrict__ p,
                                                         const float* __restrict__ dp, float scale,
                                                         T* __restrict__ ds) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* pr = p + row * k;
  const float* dr = dp + row * k;
  float pv[NV][4], dv[NV][4];
  float dot = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (c < k) { pv[i][e] = to_f32(pr[c + e]); dv[i][e] = dr[c + e]; } else { pv[i][e] = 0.f; dv[i][e] = 0.f; }
      dot += pv[i][e] * dv[i][e];
    }
  }
  dot = wave_sum(dot);
  T* out = ds + row * k;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = (lane + i * 64) * 4;
    if (c < k) {
#pragma unroll
      for (int e = 0; e < 4; ++e) out[c + e] = from_f32<T>(scale * pv[i][e] * (dv[i][e] - dot));
    }
  }
}

// ------------------------------------------------------------------ column sums
// Block = 4 row groups x 64 lanes; a lane owns one 16-byte vector of columns and strides down the
// rows of its group; groups combine through LDS, then one atomicAdd per column.  A matrix narrower than the 64
// vectors of a wave is read `fold` rows at a time (contiguous rows form one super row of cols * fold elements), so
// that all lanes have work; the fold copies of a column meet in the final atomic adds.
struct ColsumBatch { const void* x[4]; float* out[4]; };  // matrices of one shape summed by one launch (blockIdx.z)

template <typename T>
__global__ __launch_bounds__(256) void colsum_kernel(int rows, int cols, ColsumBatch cb, int64_t ldx,
                                                    int rows_per_block, int fold) {
  constexpr int VEC = Vec16<T>::N;
  typedef typename Vec16<T>::type V;
  __shared__ float red[4][64 * VEC];
  const T* __restrict__ x = reinterpret_cast<const T*>(cb.x[blockIdx.z]);
  float* __restrict__ out = cb.out[blockIdx.z];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int c = (blockIdx.x * 64 + lane) * VEC;  // position inside the super row
  const int sub = c / cols, cc = c - sub * cols;
  const int r0 = blockIdx.y * rows_per_block;
  const int nsr = (rows + fold - 1) / fold;
  int r1 = r0 + rows_per_block;
  if (r1 > nsr) r1 = nsr;
  float s[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) s[e] = 0.f;
  if (sub < fold)
    for (int r = r0 + g; r < r1; r += 4) {
      const int64_t row = (int64_t)r * fold + sub;
      if (row >= rows) break;
      const V v = *reinterpret_cast<const V*>(x + row * ldx + cc);
#pragma unroll
      for (int e = 0; e < VEC; ++e) s[e] += to_f32(v[e]);
    }
#pragma unroll
  for (int e = 0; e < VEC; ++e) red[g][lane * VEC + e] = s[e];
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * VEC; i += 256) {
    const int p = blockIdx.x * 64 * VEC + i;
    if (p < cols * fold) atomicAdd(out + p % cols, red[0][i] + red[1][i] + red[2][i] + red[3][i]);
  }
}

}  // namespace

// =================================================================== C ABI
extern "C" int ds_grad_accumulate(void* acc, const void* g, size_t n, int g_dtype, void* stream) {
  DS_CHECK_ARG(g_dtype == DS_F32 || g_dtype == DS_BF16, "ds_grad_accumulate: g_dtype %d", g_dtype);
  if (n == 0) return DS_OK;  // an empty tensor has no storage to point at
  DS_CHECK_ARG(acc && g, "ds_grad_accumulate: null pointer");
  DS_CHECK_ARG(ds_aligned16(acc) && ds_aligned16(g), "ds_grad_accumulate: pointers must be 16-byte aligned");
  if (n == 0) return DS_OK;
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, g_dtype == DS_F32 ? "accumulate_kernel<float>" : "accumulate_kernel<bf16>",
                     (double)n * (g_dtype == DS_F32 ? 12 : 10), "B");
  if (g_dtype == DS_F32) {
    const int grid = grid_for((n + 3) / 4, 256 * 4);
    hipLaunchKernelGGL(accumulate_kernel<float>, dim3(grid), dim3(256), 0, s, (float*)acc, (const float*)g, n);
  } else {
    const int grid = grid_for((n + 7) / 8, 256 * 4);
    hipLaunchKernelGGL(accumulate_kernel<bf16>, dim3(grid), dim3(256), 0, s, (float*)acc, (const bf16*)g, n);
  }
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_cast_f32_to_bf16(void* dst, const void* src, size_t n, void* stream) {
  DS_CHECK_ARG(dst && src, "ds_cast_f32_to_bf16: null pointer");
  if (n == 0) return DS_OK;
  ds_prof_scope prof((hipStream_t)stream, "cast_kernel<bf16,float>", (double)n * 6, "B");
  hipLaunchKernelGGL((cast_kernel<bf16, float>), dim3(grid_for((n + 3) / 4, 256)), dim3(256), 0, (hipStream_t)stream,
                     (bf16*)dst, (const float*)src, n);
  DS_CHECK_LAUNCH();
  return DS_OK;
}
extern "C" int ds_cast_bf16_to_f32(void* dst, const void* src, size_t n, void* stream) {
  DS_CHECK_ARG(dst && src, "ds_cast_bf16_to_f32: null pointer");
  if (n == 0) return DS_OK;
  ds_prof_scope prof((hipStream_t)stream, "cast_kernel<float,bf16>", (double)n * 6, "B");
  hipLaunchKernelGGL((cast_kernel<float, bf16>), dim3(grid_for((n + 3) / 4, 256)), dim3(256), 0, (hipStream_t)stream,
                     (float*)dst, (const bf16*)src, n);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

template <typename T> static int max_cols_rowkernel(int nv) { return 64 * Vec16<T>::N * nv; }

#define DISPATCH_NV(T, need, CALL)                                   \
  do {                                                               \
    if ((need) <= 1) { constexpr int NV = 1; CALL; }                 \
    else if ((need) <= 2) { constexpr int NV = 2; CALL; }            \
    else if ((need) <= 4) { constexpr int NV = 4; CALL; }            \
    else { constexpr int NV = 8; CALL; }                             \
  } while (0)

template <typename T>
static int layernorm_fwd_t(int rows, int cols, const void* x, const float* gamma, const float* beta, float eps, void* y,
                           float* stats, hipStream_t s) {
  const int vec = Vec16<T>::N;
  const int need = (cols / vec + 63) / 64;
  dim3 grid((rows + 3) / 4);
  ds_prof_scope prof(s, sizeof(T) == 2 ? "layernorm_fwd_kernel<bf16>" : "layernorm_fwd_kernel<float>",
                     (double)rows * cols * sizeof(T) * 2, "B");
  DISPATCH_NV(T, need, hipLaunchKernelGGL((layernorm_fwd_kernel<T, NV>), grid, dim3(256), 0, s, rows, cols, (const T*)x,
                                          gamma, beta, eps, (T*)y, stats));
  DS_CHECK_LAUNCH();
  return DS_OK;
}

static int check_rows(const char* who, int dtype, int rows, int cols) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "%s: dtype %d", who, dtype);
  const int vec = dtype == DS_BF16 ? 8 : 4;
  DS_CHECK_ARG(rows > 0 && cols > 0, "%s: rows/cols must be positive", who);
  DS_CHECK_ARG(cols % vec == 0, "%s: cols=%d must be a multiple of %d", who, cols, vec);
  DS_CHECK_ARG(cols <= 64 * vec * 8, "%s: cols=%d exceeds the %d this kernel keeps in registers", who, cols, 64 * vec * 8);
  return DS_OK;
}

extern "C" int ds_layernorm_fwd(int dtype, int rows, int cols, const void* x, const float* gamma, const float* beta,
                                float eps, void* y, float* stats, void* stream) {
  DS_PROPAGATE(check_rows("ds_layernorm_fwd", dtype, rows, cols));
  DS_CHECK_ARG(x && gamma && beta && y, "ds_layernorm_fwd: null pointer");
  DS_CHECK_ARG(ds_aligned16(x) && ds_aligned16(y) && ds_aligned16(gamma) && ds_aligned16(beta),
               "ds_layernorm_fwd: x, y, gamma and beta must be 16-byte aligned");
  if (dtype == DS_BF16) return layernorm_fwd_t<bf16>(rows, cols, x, gamma, beta, eps, y, stats, (hipStream_t)stream);
  return layernorm_fwd_t<float>(rows, cols, x, gamma, beta, eps, y, stats, (hipStream_t)stream);
}

template <typename T>
static int layernorm_bwd_t(int rows, int cols, const void* dy, const void* x, const float* gamma, const float* stats,
                           const void* dx_add, void* dx, float* dg, float* db, float* dcs, hipStream_t s) {
  const int vec = Vec16<T>::N;
  const int need = (cols / vec + 63) / 64;
  // aim for ~64 blocks of 4 waves (the column atomics at the end cost more than the row work)
  int rpw = rows / (128 * 4);
  if (rpw < 1) rpw = 1;
  if (rpw > 16) rpw = 16;
  dim3 grid((rows + 4 * rpw - 1) / (4 * rpw));
  const size_t lds = 3 * (size_t)cols * sizeof(float);
  ds_prof_scope prof(s, sizeof(T) == 2 ? "layernorm_bwd_kernel<bf16>" : "layernorm_bwd_kernel<float>",
                     (double)rows * cols * sizeof(T) * (dx_add ? 4 : 3), "B");
  DISPATCH_NV(T, need, hipLaunchKernelGGL((layernorm_bwd_kernel<T, NV>), grid, dim3(256), lds, s, rows, cols, rpw,
                                          (const T*)dy, (const T*)x, gamma, stats, (const T*)dx_add, (T*)dx, dg, db, dcs));
  DS_CHECK_LAUNCH();
  return DS_OK;
}

template <typename T>
static int layernorm_bwd_rows_t(int rows, int cols, const void* dy, const void* x, const float* gamma, const float* stats,
                                const void* dx_add, void* dx, hipStream_t s) {
  const int need = (cols / Vec16<T>::N + 63) / 64;
  dim3 grid((rows + 3) / 4);
  ds_prof_scope prof(s, sizeof(T) == 2 ? "layernorm_bwd_rows_kernel<bf16>" : "layernorm_bwd_rows_kernel<float>",
                     (double)rows * cols * sizeof(T) * (dx_add ? 4 : 3), "B");
  DISPATCH_NV(T, need, hipLaunchKernelGGL((layernorm_bwd_rows_kernel<T, NV>), grid, dim3(256), 0, s, rows, cols, (const T*)dy,
                                          (const T*)x, gamma, stats, (const T*)dx_add, (T*)dx));
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_layernorm_param_grads(int dtype, int rows, int cols, const void* dy, const void* x, const float* stats,
                                        const void* dx, float* d_gamma, float* d_beta, float* d_colsum, void* stream) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "ds_layernorm_param_grads: dtype %d", dtype);
  const int vec = dtype == DS_BF16 ? 8 : 4;
  DS_CHECK_ARG(rows > 0 && cols > 0 && cols % vec == 0, "ds_layernorm_param_grads: rows %d, cols %d (multiple of %d)", rows, cols, vec);
  DS_CHECK_ARG(dy && x && stats && d_gamma && d_beta && (!d_colsum || dx), "ds_layernorm_param_grads: null pointer (d_colsum needs dx)");
  DS_CHECK_ARG(ds_aligned16(dy) && ds_aligned16(x) && ds_aligned16(dx), "ds_layernorm_param_grads: tensors must be 16-byte aligned");
  const int strips = (cols + 64 * vec - 1) / (64 * vec);
  int rpb = 8;  // every block ends in one atomic add per column and quantity: keep the row chunks in the hundreds
  while ((int64_t)strips * ((rows + rpb - 1) / rpb) > 512) rpb *= 2;
  dim3 grid(strips, (rows + rpb - 1) / rpb);
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, dtype == DS_BF16 ? "layernorm_param_grad_kernel<bf16>" : "layernorm_param_grad_kernel<float>",
                     (double)rows * cols * (dtype == DS_BF16 ? 2 : 4) * (d_colsum ? 3 : 2), "B");
  if (dtype == DS_BF16)
    hipLaunchKernelGGL(layernorm_param_grad_kernel<bf16>, grid, dim3(256), 0, s, rows, cols, rpb, (const bf16*)dy, (const bf16*)x, stats,
                       d_colsum ? (const bf16*)dx : nullptr, d_gamma, d_beta, d_colsum);
  else
    hipLaunchKernelGGL(layernorm_param_grad_kernel<float>, grid, dim3(256), 0, s, rows, cols, rpb, (const float*)dy, (const float*)x, stats,
                       d_colsum ? (const float*)dx : nullptr, d_gamma, d_beta, d_colsum);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_layernorm_bwd(int dtype, int rows, int cols, const void* dy, const void* x, const float* gamma,
                                const float* stats, const void* dx_add, void* dx, float* d_gamma, float* d_beta,
                                float* d_colsum, void* stream) {
  DS_PROPAGATE(check_rows("ds_layernorm_bwd", dtype, rows, cols));
  DS_CHECK_ARG(ds_aligned16(dy) && ds_aligned16(x) && ds_aligned16(dx) && ds_aligned16(dx_add) && ds_aligned16(gamma),
               "ds_layernorm_bwd: tensors must be 16-byte aligned");
  if (!d_gamma && !d_beta) {  // dx only: the parameter gradients come from ds_layernorm_param_grads
    DS_CHECK_ARG(dy && x && gamma && stats && dx && !d_colsum, "ds_layernorm_bwd: null pointer (or d_colsum without d_gamma / d_beta)");
    if (dtype == DS_BF16) return layernorm_bwd_rows_t<bf16>(rows, cols, dy, x, gamma, stats, dx_add, dx, (hipStream_t)stream);
    return layernorm_bwd_rows_t<float>(rows, cols, dy, x, gamma, stats, dx_add, dx, (hipStream_t)stream);
  }
  DS_CHECK_ARG(dy && x && gamma && stats && dx && d_gamma && d_beta, "ds_layernorm_bwd: null pointer");
  if (dtype == DS_BF16)
    return layernorm_bwd_t<bf16>(rows, cols, dy, x, gamma, stats, dx_add, dx, d_gamma, d_beta, d_colsum, (hipStream_t)stream);
  return layernorm_bwd_t<float>(rows, cols, dy, x, gamma, stats, dx_add, dx, d_gamma, d_beta, d_colsum, (hipStream_t)stream);
}

static int check_mixed(const char* who, int rows, int cols) {
  DS_CHECK_ARG(rows > 0 && cols > 0 && cols % 8 == 0 && cols <= 64 * 8 * 4, "%s: rows %d, cols %d (a multiple of 8, at most 2048)", who, rows, cols);
  return DS_OK;
}
#define DISPATCH_NG(need, CALL)                      \
  do {                                               \
    if ((need) <= 1) { constexpr int NG = 1; CALL; } \
    else if ((need) <= 2) { constexpr int NG = 2; CALL; } \
    else { constexpr int NG = 4; CALL; }             \
  } while (0)

extern "C" int ds_layernorm_fwd_mixed(int rows, int cols, const float* x, const float* gamma, const float* beta, float eps,
                                      void* y_bf16, float* y_f32, float* stats, void* stream) {
  DS_PROPAGATE(check_mixed("ds_layernorm_fwd_mixed", rows, cols));
  DS_CHECK_ARG(x && gamma && beta && y_bf16, "ds_layernorm_fwd_mixed: null pointer");
  DS_CHECK_ARG(ds_aligned16(x) && ds_aligned16(y_bf16) && ds_aligned16(y_f32) && ds_aligned16(gamma) && ds_aligned16(beta),
               "ds_layernorm_fwd_mixed: tensors must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int need = (cols / 8 + 63) / 64;
  ds_prof_scope prof(s, "layernorm_fwd_mixed_kernel", (double)rows * cols * (4 + 2 + (y_f32 ? 4 : 0)), "B");
  DISPATCH_NG(need, hipLaunchKernelGGL((layernorm_fwd_mixed_kernel<NG>), dim3((rows + 3) / 4), dim3(256), 0, s, rows, cols, x, gamma, beta,
                                       eps, (bf16*)y_bf16, y_f32, stats, ds_launch_prio));
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_layernorm_bwd_mixed(int rows, int cols, const float* dy, const float* x, const float* gamma, const float* stats,
                                      void* dx_bf16, float* dx_f32, void* dy_bf16, float* d_gamma, float* d_beta, float* d_colsum,
                                      void* stream) {
  DS_PROPAGATE(check_mixed("ds_layernorm_bwd_mixed", rows, cols));
  DS_CHECK_ARG(dy && x && gamma && stats && dx_bf16, "ds_layernorm_bwd_mixed: null pointer");
  DS_CHECK_ARG(ds_aligned16(dy) && ds_aligned16(x) && ds_aligned16(dx_bf16) && ds_aligned16(dx_f32) && ds_aligned16(gamma) &&
               ds_aligned16(dy_bf16), "ds_layernorm_bwd_mixed: tensors must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int need = (cols / 8 + 63) / 64;
  if (!d_gamma && !d_beta) {  // dx only: the parameter gradients come from ds_layernorm_param_grads_mixed
    DS_CHECK_ARG(!d_colsum, "ds_layernorm_bwd_mixed: d_colsum without d_gamma / d_beta");
    ds_prof_scope prof(s, "layernorm_bwd_mixed_rows_kernel",
                       (double)rows * cols * (4 + 4 + 2 + (dx_f32 ? 4 : 0) + (dy_bf16 ? 2 : 0)), "B");
    DISPATCH_NG(need, hipLaunchKernelGGL((layernorm_bwd_mixed_rows_kernel<NG>), dim3((rows + 3) / 4), dim3(256), 0, s, rows, cols, dy, x,
                                         gamma, stats, (bf16*)dx_bf16, dx_f32, (bf16*)dy_bf16, nullptr, nullptr, ds_launch_prio));
    DS_CHECK_LAUNCH();
    return DS_OK;
  }
  DS_CHECK_ARG(d_gamma && d_beta && !dy_bf16, "ds_layernorm_bwd_mixed: d_gamma and d_beta come together, and without dy_bf16");
  int rpw = rows / (128 * 4);
  if (rpw < 1) rpw = 1;
  if (rpw > 16) rpw = 16;
  dim3 grid((rows + 4 * rpw - 1) / (4 * rpw));
  const size_t lds = 3 * (size_t)cols * sizeof(float);
  ds_prof_scope prof(s, "layernorm_bwd_mixed_kernel", (double)rows * cols * (4 + 4 + 2 + (dx_f32 ? 4 : 0)), "B");
  DISPATCH_NG(need, hipLaunchKernelGGL((layernorm_bwd_mixed_kernel<NG>), grid, dim3(256), lds, s, rows, cols, rpw, dy, x, gamma, stats,
                                       (bf16*)dx_bf16, dx_f32, d_gamma, d_beta, d_colsum));
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_layernorm_param_grads_mixed(int rows, int cols, const void* dy_bf16, const float* x, const float* stats,
                                              const void* dx_bf16, float* d_gamma, float* d_beta, float* d_colsum, void* stream) {
  DS_CHECK_ARG(rows > 0 && cols > 0 && cols % 8 == 0, "ds_layernorm_param_grads_mixed: rows %d, cols %d (a multiple of 8)", rows, cols);
  DS_CHECK_ARG(dy_bf16 && x && stats && d_gamma && d_beta && (!d_colsum || dx_bf16),
               "ds_layernorm_param_grads_mixed: null pointer (d_colsum needs dx_bf16)");
  DS_CHECK_ARG(ds_aligned16(dy_bf16) && ds_aligned16(x) && ds_aligned16(dx_bf16),
               "ds_layernorm_param_grads_mixed: tensors must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int strips = (cols + 64 * 8 - 1) / (64 * 8);
  int chunks = 256 / strips;  // about one block per CU
  if (chunks > (rows + 31) / 32) chunks = (rows + 31) / 32;
  if (chunks < 1) chunks = 1;
  const int rpb = (rows + chunks - 1) / chunks;
  dim3 grid(strips, (rows + rpb - 1) / rpb);
  ds_prof_scope prof(s, "layernorm_param_grad_mixed_kernel", (double)rows * cols * (2 + 4 + (d_colsum ? 2 : 0)), "B");
  hipLaunchKernelGGL(layernorm_param_grad_mixed_kernel, grid, dim3(256), 0, s, rows, cols, rpb, (const bf16*)dy_bf16, x, stats,
                     d_colsum ? (const bf16*)dx_bf16 : nullptr, d_gamma, d_beta, d_colsum);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

// The row kernel with the hand-over that loses nothing: an fp32 copy of dy and the two per-row means (see rows_core.h).
extern "C" int ds_layernorm_bwd_mixed_rows(int rows, int cols, const float* dy, const float* x, const float* gamma, const float* stats,
                                           void* dx_bf16, float* dx_f32, float* dy_copy, float* row_sums, void* stream) {
  DS_PROPAGATE(check_mixed("ds_layernorm_bwd_mixed_rows", rows, cols));
  DS_CHECK_ARG(dy && x && gamma && stats && dx_bf16 && dy_copy && row_sums, "ds_layernorm_bwd_mixed_rows: null pointer");
  DS_CHECK_ARG(ds_aligned16(dy) && ds_aligned16(x) && ds_aligned16(dx_bf16) && ds_aligned16(dx_f32) && ds_aligned16(gamma) && ds_aligned16(dy_copy),
               "ds_layernorm_bwd_mixed_rows: tensors must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int need = (cols / 8 + 63) / 64;
  ds_prof_scope prof(s, "layernorm_bwd_mixed_rows_kernel", (double)rows * cols * (4 + 4 + 2 + (dx_f32 ? 4 : 0) + 4), "B");
  DISPATCH_NG(need, hipLaunchKernelGGL((layernorm_bwd_mixed_rows_kernel<NG>), dim3((rows + 3) / 4), dim3(256), 0, s, rows, cols, dy, x, gamma,
                                       stats, (bf16*)dx_bf16, dx_f32, (bf16*)nullptr, dy_copy, row_sums, ds_launch_prio));
  DS_CHECK_LAUNCH();
  return DS_OK;
}

int ds_layernorm_param_grads_exact_seg(int rows, int cols, const float* dy_copy, const float* x, const float* gamma, const float* stats,
                                       const float* row_sums, float* d_gamma, float* d_beta, float* d_colsum, int seg_rows, int64_t x_seg,
                                       int64_t st_seg, void* stream);

extern "C" int ds_layernorm_param_grads_exact(int rows, int cols, const float* dy_copy, const float* x, const float* gamma, const float* stats,
                                              const float* row_sums, float* d_gamma, float* d_beta, float* d_colsum, void* stream) {
  return ds_layernorm_param_grads_exact_seg(rows, cols, dy_copy, x, gamma, stats, row_sums, d_gamma, d_beta, d_colsum, rows, 0, 0, stream);
}

int ds_layernorm_param_grads_exact_seg(int rows, int cols, const float* dy_copy, const float* x, const float* gamma, const float* stats,
                                       const float* row_sums, float* d_gamma, float* d_beta, float* d_colsum, int seg_rows, int64_t x_seg,
                                       int64_t st_seg, void* stream) {
  DS_CHECK_ARG(rows > 0 && cols > 0 && cols % 8 == 0, "ds_layernorm_param_grads_exact: rows %d, cols %d (a multiple of 8)", rows, cols);
  DS_CHECK_ARG(seg_rows > 0 && rows % seg_rows == 0 && x_seg % 4 == 0, "ds_layernorm_param_grads_exact: %d rows in segments of %d", rows, seg_rows);
  DS_CHECK_ARG(dy_copy && x && gamma && stats && row_sums && d_gamma && d_beta, "ds_layernorm_param_grads_exact: null pointer");
  DS_CHECK_ARG(ds_aligned16(dy_copy) && ds_aligned16(x) && ds_aligned16(gamma), "ds_layernorm_param_grads_exact: tensors must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int strips = (cols + 64 * 8 - 1) / (64 * 8);
  int chunks = 256 / strips;  // about one block per CU
  if (chunks > (rows + 31) / 32) chunks = (rows + 31) / 32;
  if (chunks < 1) chunks = 1;
  const int rpb = (rows + chunks - 1) / chunks;
  dim3 grid(strips, (rows + rpb - 1) / rpb);
  ds_prof_scope prof(s, "layernorm_param_grad_exact_kernel", (double)rows * cols * 8, "B");
  hipLaunchKernelGGL(layernorm_param_grad_exact_kernel, grid, dim3(256), 0, s, rows, cols, rpb, dy_copy, x, gamma, stats, row_sums, d_gamma,
                     d_beta, d_colsum, seg_rows, x_seg, st_seg);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

template <typename T>
static int softmax_fwd_t(int64_t rows, int k, int rpb, const float* scores, float scale, const float* mask, float mv,
                         void* p, hipStream_t s) {
  const int need = (k / 4 + 63) / 64;
  dim3 grid((unsigned)((rows + 3) / 4));
  ds_prof_scope prof(s, sizeof(T) == 2 ? "softmax_fwd_kernel<bf16>" : "softmax_fwd_kernel<float>",
                     (double)rows * k * (4 + sizeof(T)), "B");
  DISPATCH_NV(T, need, hipLaunchKernelGGL((softmax_fwd_kernel<T, NV>), grid, dim3(256), 0, s, rows, k, rpb, scores, scale,
                                          mask, mv, (T*)p));
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_softmax_fwd(int dtype, int batch, int heads, int q, int k, const float* scores, float scale,
                              const float* key_mask, float mask_value, void* p, void* stream) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "ds_softmax_fwd: dtype %d", dtype);
  DS_CHECK_ARG(batch > 0 && heads > 0 && q > 0 && k > 0, "ds_softmax_fwd: non-positive shape");
  DS_CHECK_ARG(k % 4 == 0 && k <= 64 * 4 * 8, "ds_softmax_fwd: k=%d must be a multiple of 4 and at most 2048", k);
  DS_CHECK_ARG(scores && p && ds_aligned16(scores), "ds_softmax_fwd: null or unaligned pointer");
  const int64_t rows = (int64_t)batch * heads * q;
  if (dtype == DS_BF16)
    return softmax_fwd_t<bf16>(rows, k, heads * q, scores, scale, key_mask, mask_value, p, (hipStream_t)stream);
  return softmax_fwd_t<float>(rows, k, heads * q, scores, scale, key_mask, mask_value, p, (hipStream_t)stream);
}

template <typename T>
static int softmax_bwd_t(int64_t rows, int k, const void* p, const float* dp, float scale, void* ds, hipStream_t s) {
  const int need = (k / 4 + 63) / 64;
  dim3 grid((unsigned)((rows + 3) / 4));
  ds_prof_scope prof(s, sizeof(T) == 2 ? "softmax_bwd_kernel<bf16>" : "softmax_bwd_kernel<float>",
                     (double)rows * k * (4 + 2 * sizeof(T)), "B");
  DISPATCH_NV(T, need, hipLaunchKernelGGL((softmax_bwd_kernel<T, NV>), grid, dim3(256), 0, s, rows, k, (const T*)p, dp,
                                          scale, (T*)ds));
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_softmax_bwd(int dtype, int64_t rows, int k, const void* p, const float* dp, float scale, void* ds,
                              void* stream) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "ds_softmax_bwd: dtype %d", dtype);
  DS_CHECK_ARG(rows > 0 && k > 0 && k % 4 == 0 && k <= 2048, "ds_softmax_bwd: bad shape rows=%lld k=%d", (long long)rows, k);
  DS_CHECK_ARG(p && dp && ds, "ds_softmax_bwd: null pointer");
  if (dtype == DS_BF16) return softmax_bwd_t<bf16>(rows, k, p, dp, scale, ds, (hipStream_t)stream);
  return softmax_bwd_t<float>(rows, k, p, dp, scale, ds, (hipStream_t)stream);
}

int ds_colsum_accum_multi(int dtype, int rows, int cols, int count, const void* const* xs, int64_t ldx, float* const* outs, void* stream);

extern "C" int ds_colsum_accum(int dtype, int rows, int cols, const void* x, int64_t ldx, float* out, void* stream) {
  return ds_colsum_accum_multi(dtype, rows, cols, 1, &x, ldx, &out, stream);
}

int ds_colsum_accum_multi(int dtype, int rows, int cols, int count, const void* const* xs, int64_t ldx, float* const* outs, void* stream) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "ds_colsum_accum: dtype %d", dtype);
  DS_CHECK_ARG(rows > 0 && cols > 0 && ldx >= cols && count >= 1 && count <= 4, "ds_colsum_accum: bad argument");
  const int vec = dtype == DS_BF16 ? 8 : 4;
  ColsumBatch cb = {};
  for (int i = 0; i < count; ++i) {
    DS_CHECK_ARG(xs[i] && outs[i] && ds_aligned16(xs[i]), "ds_colsum_accum: null or unaligned pointer");
    cb.x[i] = xs[i]; cb.out[i] = outs[i];
  }
  const void* x = xs[0];
  DS_CHECK_ARG(cols % vec == 0 && ldx % vec == 0 && ds_aligned16(x), "ds_colsum_accum: cols and ldx must be multiples of %d and x 16-byte aligned", vec);
  // every block ends in one atomic add per column: keep the number of row chunks in the low thousands
  int fold = 1;
  if (cols < 64 * vec && (64 * vec) % cols == 0 && ldx == cols) fold = 64 * vec / cols;
  const int nsr = (rows + fold - 1) / fold;
  int rpb = 32;
  const int strips = (cols * fold + 64 * vec - 1) / (64 * vec);
  while ((int64_t)strips * ((nsr + rpb - 1) / rpb) > 2048 && rpb < (1 << 20)) rpb *= 2;
  dim3 grid(strips, (nsr + rpb - 1) / rpb, count);
  ds_prof_scope prof((hipStream_t)stream, dtype == DS_BF16 ? "colsum_kernel<bf16>" : "colsum_kernel<float>",
                     (double)rows * cols * (dtype == DS_BF16 ? 2 : 4) * count, "B");
  if (dtype == DS_BF16)
    hipLaunchKernelGGL(colsum_kernel<bf16>, grid, dim3(256), 0, (hipStream_t)stream, rows, cols, cb, ldx, rpb, fold);
  else
    hipLaunchKernelGGL(colsum_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, rows, cols, cb, ldx, rpb, fold);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

// ------------------------------------------------------------------ per-sample column sums, rank-k correction
// out[s][c] = scale * sum over the `seq` rows of sample s of x[s * seq + r][c] (bf16 x, row stride ldx).  Every row of
// the score gradient of a softmax sums to zero, so a query gradient dS K only sees the keys' deviation from their mean,
// and every head's key gradients sum to zero over a sample, so a key-projection weight gradient X^T dK only sees the
// deviation of the layer's inputs from their mean: the means (and the column sums the rounded gradients are left with)
// are what this kernel gives.  A block owns 64 columns of one sample: 8 lanes per row, 32 rows in flight.
namespace {
constexpr int SAMPLE_COLSUM_MAX = 64;
struct SampleColsumArgs {
  const bf16* x[SAMPLE_COLSUM_MAX];
  float* out[SAMPLE_COLSUM_MAX];
  int64_t ldx[SAMPLE_COLSUM_MAX];
  float scale[SAMPLE_COLSUM_MAX];
};
// grid (ceil(cols / 64), samples, problems)
__global__ __launch_bounds__(256) void sample_colsum_kernel(int seq, int cols, SampleColsumArgs a) {
  __shared__ float red[32][65];
  const int cg = threadIdx.x & 7, rg = threadIdx.x >> 3;
  const int c = blockIdx.x * 64 + cg * 8, s = blockIdx.y, z = blockIdx.z;
  const int64_t ldx = a.ldx[z];
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if (c < cols) {
    const bf16* base = a.x[z] + (int64_t)s * seq * ldx + c;
#pragma unroll 4
    for (int r = rg; r < seq; r += 32) {
      const bf16x8 v = *reinterpret_cast<const bf16x8*>(base + (int64_t)r * ldx);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += (float)v[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[rg][cg * 8 + e] = acc[e];
  __syncthreads();
  if (threadIdx.x < 64 && blockIdx.x * 64 + threadIdx.x < cols) {
    float t = 0.f;
#pragma unroll
    for (int r = 0; r < 32; ++r) t += red[r][threadIdx.x];
    a.out[z][(int64_t)s * cols + blockIdx.x * 64 + threadIdx.x] = t * a.scale[z];
  }
}

// For every problem z: w[i][n] -= sum_{s < ns} a[s][i] * b[s][n] and, with v, v[n] -= sum_s b[s][n].
// grid (ceil(cols / 1024), rows, problems), a thread owns 4 consecutive columns.
constexpr int RANK_UPDATE_MAX = 32;
struct RankUpdateArgs {
  const float* a[RANK_UPDATE_MAX];
  const float* b[RANK_UPDATE_MAX];
  float* w[RANK_UPDATE_MAX];
  float* v[RANK_UPDATE_MAX];
};
__global__ __launch_bounds__(256) void rank_update_kernel(int rows, int cols, int ns, int64_t ldw, RankUpdateArgs p) {
  const int i = blockIdx.y, n = (blockIdx.x * 256 + threadIdx.x) * 4, z = blockIdx.z;
  if (n >= cols) return;
  const float* a = p.a[z];
  const float* b = p.b[z];
  f32x4 acc = {0.f, 0.f, 0.f, 0.f}, tot = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < ns; ++s) {
    const float ai = a[(int64_t)s * rows + i];
    const f32x4 bv = *reinterpret_cast<const f32x4*>(b + (int64_t)s * cols + n);
    acc += ai * bv;
    tot += bv;
  }
  f32x4* q = reinterpret_cast<f32x4*>(p.w[z] + (int64_t)i * ldw + n);
  *q = *q - acc;
  if (p.v[z] != nullptr && i == 0) {
    f32x4* r = reinterpret_cast<f32x4*>(p.v[z] + n);
    *r = *r - tot;
  }
}
}  // namespace

// `count` matrices of one shape (samples * seq rows, cols columns) in one launch: outs[i][s][c] = scales[i] * column sum of sample s of xs[i]
int ds_sample_colsum_multi(int count, int samples, int seq, int cols, const void* const* xs, const int64_t* ldxs, const float* scales,
                           float* const* outs, void* stream) {
  DS_CHECK_ARG(count > 0 && samples > 0 && samples <= 65535 && seq > 0 && cols > 0 && cols % 8 == 0, "ds_sample_colsum: bad shape");
  for (int first = 0; first < count; first += SAMPLE_COLSUM_MAX) {
    const int n = count - first < SAMPLE_COLSUM_MAX ? count - first : SAMPLE_COLSUM_MAX;
    SampleColsumArgs a;
    memset(&a, 0, sizeof(a));
    for (int i = 0; i < n; ++i) {
      DS_CHECK_ARG(xs[first + i] && outs[first + i] && ds_aligned16(xs[first + i]) && ldxs[first + i] % 8 == 0 && ldxs[first + i] >= cols,
                   "ds_sample_colsum: null or unaligned pointer, or a bad row stride");
      a.x[i] = (const bf16*)xs[first + i]; a.out[i] = outs[first + i]; a.ldx[i] = ldxs[first + i]; a.scale[i] = scales[first + i];
    }
    ds_prof_scope prof((hipStream_t)stream, "sample_colsum_kernel", (double)n * samples * seq * cols * 2, "B");
    hipLaunchKernelGGL(sample_colsum_kernel, dim3((cols + 63) / 64, samples, n), dim3(256), 0, (hipStream_t)stream, seq, cols, a);
    DS_CHECK_LAUNCH();
  }
  return DS_OK;
}

int ds_sample_colsum(int samples, int seq, int cols, const void* x, int64_t ldx, float scale, float* out, void* stream) {
  return ds_sample_colsum_multi(1, samples, seq, cols, &x, &ldx, &scale, &out, stream);
}

// `count` updates of one shape in one launch; the w (and v) of different problems must not overlap
int ds_rank_update_multi(int count, int rows, int cols, int ns, const float* const* as, const float* const* bs, float* const* ws, int64_t ldw,
                         float* const* vs, void* stream) {
  DS_CHECK_ARG(count > 0 && rows > 0 && rows <= 65535 && cols > 0 && cols % 4 == 0 && ns > 0 && ldw % 4 == 0 && ldw >= cols, "ds_rank_update: bad shape");
  for (int first = 0; first < count; first += RANK_UPDATE_MAX) {
    const int n = count - first < RANK_UPDATE_MAX ? count - first : RANK_UPDATE_MAX;
    RankUpdateArgs p;
    memset(&p, 0, sizeof(p));
    for (int i = 0; i < n; ++i) {
      p.a[i] = as[first + i]; p.b[i] = bs[first + i]; p.w[i] = ws[first + i]; p.v[i] = vs ? vs[first + i] : nullptr;
      DS_CHECK_ARG(p.a[i] && p.b[i] && p.w[i] && ds_aligned16(p.b[i]) && ds_aligned16(p.w[i]) && ds_aligned16(p.v[i]),
                   "ds_rank_update: null or unaligned pointer");
    }
    ds_prof_scope prof((hipStream_t)stream, "rank_update_kernel", (double)n * rows * cols * 8, "B");
    hipLaunchKernelGGL(rank_update_kernel, dim3((cols + 1023) / 1024, rows, n), dim3(256), 0, (hipStream_t)stream, rows, cols, ns, ldw, p);
    DS_CHECK_LAUNCH();
  }
  return DS_OK;
}

int ds_rank_update(int rows, int cols, int ns, const float* a, const float* b, float* w, int64_t ldw, float* v, void* stream) {
  return ds_rank_update_multi(1, rows, cols, ns, &a, &b, &w, ldw, &v, stream);
}
