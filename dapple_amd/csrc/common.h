// Shared device/host helpers for the gfx950 kernels of libdapple_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <atomic>

#include "../../include/dapple_stage.h"

typedef __bf16 bf16;
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define WAVE 64

// ---- error plumbing (host) ----
void ds_set_error(const char* fmt, ...);
#define DS_CHECK_ARG(cond, ...)         \
  do {                                  \
    if (!(cond)) {                      \
      ds_set_error(__VA_ARGS__);        \
      return DS_EINVAL;                 \
    }                                   \
  } while (0)
#define DS_CHECK_HIP(expr)                                                        \
  do {                                                                            \
    hipError_t e_ = (expr);                                                       \
    if (e_ != hipSuccess) {                                                       \
      ds_set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
      return DS_EHIP;                                                             \
    }                                                                             \
  } while (0)
#define DS_CHECK_LAUNCH() DS_CHECK_HIP(hipGetLastError())
#define DS_PROPAGATE(expr)      \
  do {                          \
    int rc_ = (expr);           \
    if (rc_ != DS_OK) return rc_; \
  } while (0)

// ---- optional per-launch timing (host): HIP events around each kernel launch on its own stream
struct ds_prof_scope {
  bool on;
  hipStream_t stream;
  ds_prof_scope(hipStream_t s, const char* tag, double work, const char* unit);
  ~ds_prof_scope();
};

// Wave priority of the kernels launched next from this host thread (0..3, the s_setprio scale).  A stage
// raises it for the passes other work waits on and lowers it for work that only feeds the master gradients,
// so that waves of both sharing a SIMD are issued in that order.
extern thread_local int ds_launch_prio;
struct ds_prio_scope {
  int keep;
  explicit ds_prio_scope(int p) : keep(ds_launch_prio) { ds_launch_prio = p; }
  ~ds_prio_scope() { ds_launch_prio = keep; }
};

static inline bool ds_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// ---- device helpers ----
__device__ __forceinline__ void ds_wave_prio(int p) {  // s_setprio takes an immediate
  if (p == 1) __builtin_amdgcn_s_setprio(1);
  else if (p == 2) __builtin_amdgcn_s_setprio(2);
  else if (p == 3) __builtin_amdgcn_s_setprio(3);
}
template <typename T> struct Vec16;  // 16-byte vector of T
template <> struct Vec16<bf16> { typedef bf16x8 type; static constexpr int N = 8; };
template <> struct Vec16<float> { typedef f32x4 type; static constexpr int N = 4; };

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16 x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float x) { return (bf16)x; }

// Wave reductions: the four steps inside a row of 16 lanes are DPP moves (lane ^ 1, lane ^ 2, mirror of 8, mirror
// of 16 - a few cycles each), only the two steps across rows go through the LDS crossbar.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_move<0x141>(v);  // row_half_mirror
  v += dpp_move<0x140>(v);  // row_mirror
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));
  v = fmaxf(v, dpp_move<0x4E>(v));
  v = fmaxf(v, dpp_move<0x141>(v));
  v = fmaxf(v, dpp_move<0x140>(v));
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  v = fmaxf(v, __shfl_xor(v, 32, 64));
  return v;
}

// Normal CDF and PDF at x from ONE exponential: Phi(x) = 0.5 (1 + erf(x / sqrt 2)) with erf from the rational
// form of Abramowitz & Stegun 7.1.26 (absolute error below 1.5e-7, i.e. at fp32 rounding level for values of
// order one), whose e^{-x^2/2} factor is also the PDF's.  The library erff costs several times more, and the
// GEMM epilogues that apply GELU are not hidden behind anything.
__device__ __forceinline__ void normal_cdf_pdf(float x, float& cdf, float& pdf) {
  const float e = __expf(-0.5f * x * x);
  const float z = fabsf(x) * 0.70710678118654752440f;
  const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * z);
  const float poly = ((((1.061405429f * t - 1.453152027f) * t + 1.421413741f) * t - 0.284496736f) * t + 0.254829592f) * t;
  const float half_tail = 0.5f * poly * e;          // 0.5 * erfc(|x| / sqrt 2)
  cdf = x >= 0.f ? 1.0f - half_tail : half_tail;
  pdf = 0.39894228040143267794f * e;
}
// erf-form GELU of the reference (bert/models/bert/modeling_slice.py:30-43) and its derivative
__device__ __forceinline__ float gelu_erf(float x) {
  float cdf, pdf;
  normal_cdf_pdf(x, cdf, pdf);
  return x * cdf;
}
__device__ __forceinline__ float gelu_erf_grad(float x) {
  float cdf, pdf;
  normal_cdf_pdf(x, cdf, pdf);
  return cdf + x * pdf;
}

// tanh-form GELU of the reference's XLNet layers (xlnet/activations/gelu.py:6-11) and its derivative;
// tanh(z) = 1 - 2 / (1 + e^{2z})
__device__ __forceinline__ float fast_tanh(float z) {
  const float e = __expf(2.0f * z);
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float gelu_tanh(float x) {
  const float t = fast_tanh(0.79788456080286535588f * (x + 0.044715f * x * x * x));
  return 0.5f * x * (1.0f + t);
}
__device__ __forceinline__ float gelu_tanh_grad(float x) {
  const float t = fast_tanh(0.79788456080286535588f * (x + 0.044715f * x * x * x));
  return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * 0.79788456080286535588f * (1.0f + 3.0f * 0.044715f * x * x);
}
__device__ __forceinline__ float gelu_any(float x, bool tanh_form) { return tanh_form ? gelu_tanh(x) : gelu_erf(x); }
__device__ __forceinline__ float gelu_any_grad(float x, bool tanh_form) { return tanh_form ? gelu_tanh_grad(x) : gelu_erf_grad(x); }

// A dense layer over a handful of rows: out[b][j] = act(bias[j] + sum_k in[b][k] W[k][j]), W [K0 + K1, N] row-major,
// in[b] = [in0[b * stride0 .. + K0) | in1[b * stride1 .. + K1)].  grid (ceil(N / 64), rows), 1024 threads: lane = column,
// the 16 waves split k and meet in LDS.  ACT: 0 none, 1 tanh.
template <typename TI, int ACT>
__global__ __launch_bounds__(1024) void ds_small_dense_kernel(int K0, int K1, int N, const TI* __restrict__ in0, int64_t stride0,
                                                              const float* __restrict__ in1, int64_t stride1,
                                                              const float* __restrict__ W, const float* __restrict__ bias,
                                                              float* __restrict__ out) {
  __shared__ float red[16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = blockIdx.x * 64 + lane, b = blockIdx.y;
  const int K = K0 + K1, per = (K + 15) / 16;
  const int k0 = wave * per, k1 = k0 + per < K ? k0 + per : K;
  float a = 0.f;
  if (j < N)
    for (int k = k0; k < k1; ++k) {
      const float x = k < K0 ? (float)in0[(int64_t)b * stride0 + k] : in1[(int64_t)b * stride1 + (k - K0)];
      a += x * W[(int64_t)k * N + j];
    }
  red[wave][lane] = a;
  __syncthreads();
  if (wave == 0 && j < N) {
    float s = bias ? bias[j] : 0.f;
#pragma unroll
    for (int w = 0; w < 16; ++w) s += red[w][lane];
    out[(int64_t)b * N + j] = ACT == 1 ? tanhf(s) : s;
  }
}
