// What the reference runs on the accumulated gradients right after the pipeline unroll: global-norm
// clipping (bert/graph.py:162-165, tf.clip_by_global_norm) and the optimizer's apply_gradients -
// AdamWeightDecayOptimizer (bert/graph_helper.py:213-272: no bias correction, decoupled decay on the
// tensors not excluded by name), tf.train.AdamOptimizer (xlnet/utils/xlnet_utils.py:179-199) and
// tf.train.GradientDescentOptimizer (vgg19/tf-keras-dapple.py:187).  All of it is element-wise over
// the flat fp32 master buffers: one HBM-bound kernel per step (28 B/element for Adam, 12 for SGD)
// plus one 4 B/element reduction for the norm; the clip factor is applied inside the update kernel.
#include <math.h>

#include <vector>

#include "common.h"

struct ds_optim_plan {
  // one entry per chunk of at most CHUNK consecutive elements of one tensor
  int64_t* d_off = nullptr;
  int* d_cnt = nullptr;
  float* d_decay = nullptr;
  int chunks = 0;
  int64_t elements = 0;
};

namespace {

constexpr int CHUNK = 16384;

__global__ __launch_bounds__(256) void sqnorm_kernel(const float* __restrict__ g, size_t n, double* __restrict__ acc) {
  __shared__ float part[4];
  float s = 0.f;
  const size_t n4 = n / 4;
  const f32x4* g4 = reinterpret_cast<const f32x4*>(g);
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256) {
    const f32x4 v = g4[i];
    s += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
  }
  if (blockIdx.x == 0)
    for (size_t i = n4 * 4 + threadIdx.x; i < n; i += 256) s += g[i] * g[i];
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) atomicAdd(acc, (double)part[0] + (double)part[1] + (double)part[2] + (double)part[3]);
}

// tf.clip_by_global_norm: t * clip_norm / max(global_norm, clip_norm)
__device__ __forceinline__ float clip_factor(const double* sqnorm, float clip_norm) {
  if (!sqnorm) return 1.f;
  const float norm = (float)sqrt(*sqnorm);
  return clip_norm / fmaxf(norm, clip_norm);
}

// MODE 0: Adam moments + optional decoupled decay (graph_helper.py:240-261); MODE 1: plain gradient descent
template <int MODE>
__global__ __launch_bounds__(256) void apply_kernel(const int64_t* __restrict__ off, const int* __restrict__ cnt,
                                                    const float* __restrict__ decay, float* __restrict__ w,
                                                    const float* __restrict__ g, float* __restrict__ m, float* __restrict__ v,
                                                    float lr, float b1, float omb1, float b2, float omb2, float eps,
                                                    const double* __restrict__ sqnorm, float clip_norm) {
  const int64_t o = off[blockIdx.x];
  const int n = cnt[blockIdx.x];
  const float wd = decay[blockIdx.x];
  const float cf = clip_factor(sqnorm, clip_norm);
  for (int i = threadIdx.x * 4; i < n; i += 256 * 4) {
    if (i + 4 <= n) {
      f32x4 wv = *reinterpret_cast<f32x4*>(w + o + i);
      const f32x4 gv = *reinterpret_cast<const f32x4*>(g + o + i);
      if (MODE == 0) {
        f32x4 mv = *reinterpret_cast<f32x4*>(m + o + i), vv = *reinterpret_cast<f32x4*>(v + o + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float ge = gv[e] * cf;
          mv[e] = b1 * mv[e] + omb1 * ge;
          vv[e] = b2 * vv[e] + omb2 * ge * ge;
          const float upd = mv[e] / (sqrtf(vv[e]) + eps) + wd * wv[e];
          wv[e] -= lr * upd;
        }
        *reinterpret_cast<f32x4*>(m + o + i) = mv;
        *reinterpret_cast<f32x4*>(v + o + i) = vv;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) wv[e] -= lr * (gv[e] * cf);
      }
      *reinterpret_cast<f32x4*>(w + o + i) = wv;
    } else {
      for (int e = i; e < n; ++e) {
        const float ge = g[o + e] * cf;
        if (MODE == 0) {
          const float mm = b1 * m[o + e] + omb1 * ge;
          const float vv = b2 * v[o + e] + omb2 * ge * ge;
          m[o + e] = mm; v[o + e] = vv;
          w[o + e] -= lr * (mm / (sqrtf(vv) + eps) + wd * w[o + e]);
        } else {
          w[o + e] -= lr * ge;
        }
      }
    }
  }
}

}  // namespace

/* acc (a device double, not cleared here) += sum of squares of g[0..n) */
extern "C" int ds_grad_sqnorm_accum(const float* g, size_t n, double* acc, void* stream) {
  if (n == 0) return DS_OK;
  DS_CHECK_ARG(g && acc, "ds_grad_sqnorm_accum: null pointer");
  DS_CHECK_ARG(ds_aligned16(g), "ds_grad_sqnorm_accum: g must be 16-byte aligned");
  size_t blocks = (n / 4 + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  if (blocks < 1) blocks = 1;
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "sqnorm_kernel", (double)n * 4, "B");
  hipLaunchKernelGGL(sqnorm_kernel, dim3((unsigned)blocks), dim3(256), 0, s, g, n, acc);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_optim_plan_create(int n_tensors, const int64_t* offsets, const int64_t* numels, const float* decay_rates,
                                    ds_optim_plan** out) {
  DS_CHECK_ARG(out != nullptr, "ds_optim_plan_create: null out");
  *out = nullptr;
  DS_CHECK_ARG(n_tensors > 0 && offsets && numels && decay_rates, "ds_optim_plan_create: null or empty tensor list");
  std::vector<int64_t> off;
  std::vector<int> cnt;
  std::vector<float> dec;
  int64_t total = 0;
  for (int t = 0; t < n_tensors; ++t) {
    DS_CHECK_ARG(offsets[t] >= 0 && offsets[t] % 4 == 0, "ds_optim_plan_create: offset of tensor %d must be a non-negative multiple of 4", t);
    DS_CHECK_ARG(numels[t] >= 0, "ds_optim_plan_create: negative element count for tensor %d", t);
    for (int64_t o = 0; o < numels[t]; o += CHUNK) {
      off.push_back(offsets[t] + o);
      cnt.push_back((int)(numels[t] - o < CHUNK ? numels[t] - o : CHUNK));
      dec.push_back(decay_rates[t]);
    }
    total += numels[t];
  }
  ds_optim_plan* p = new ds_optim_plan();
  p->chunks = (int)off.size();
  p->elements = total;
  if (p->chunks) {
    hipError_t e = hipMalloc((void**)&p->d_off, off.size() * sizeof(int64_t));
    if (e == hipSuccess) e = hipMalloc((void**)&p->d_cnt, cnt.size() * sizeof(int));
    if (e == hipSuccess) e = hipMalloc((void**)&p->d_decay, dec.size() * sizeof(float));
    if (e == hipSuccess) e = hipMemcpy(p->d_off, off.data(), off.size() * sizeof(int64_t), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(p->d_cnt, cnt.data(), cnt.size() * sizeof(int), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(p->d_decay, dec.data(), dec.size() * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
      ds_set_error("ds_optim_plan_create: %s", hipGetErrorString(e));
      (void)hipFree(p->d_off); (void)hipFree(p->d_cnt); (void)hipFree(p->d_decay);
      delete p;
      return DS_EHIP;
    }
  }
  *out = p;
  return DS_OK;
}

extern "C" int ds_optim_plan_destroy(ds_optim_plan* p) {
  if (!p) return DS_OK;
  (void)hipFree(p->d_off); (void)hipFree(p->d_cnt); (void)hipFree(p->d_decay);
  delete p;
  return DS_OK;
}

static int check_flat(const char* who, const ds_optim_plan* p, const void* w, const void* g) {
  DS_CHECK_ARG(p != nullptr, "%s: null plan", who);
  DS_CHECK_ARG(w && g, "%s: null buffer", who);
  DS_CHECK_ARG(ds_aligned16(w) && ds_aligned16(g), "%s: buffers must be 16-byte aligned", who);
  return DS_OK;
}

extern "C" int ds_adam_step(const ds_optim_plan* p, float* w, const float* g, float* m, float* v, double lr, double beta1,
                            double beta2, double eps, const double* grad_sqnorm, float clip_norm, void* stream) {
  DS_PROPAGATE(check_flat("ds_adam_step", p, w, g));
  DS_CHECK_ARG(m && v && ds_aligned16(m) && ds_aligned16(v), "ds_adam_step: moment buffers must be non-null and 16-byte aligned");
  DS_CHECK_ARG(!grad_sqnorm || clip_norm > 0.f, "ds_adam_step: clip_norm must be positive");
  if (!p->chunks) return DS_OK;
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "adam_apply_kernel", (double)p->elements * 28, "B");
  hipLaunchKernelGGL(apply_kernel<0>, dim3(p->chunks), dim3(256), 0, s, p->d_off, p->d_cnt, p->d_decay, w, g, m, v, (float)lr, (float)beta1,
                     (float)(1.0 - beta1), (float)beta2, (float)(1.0 - beta2), (float)eps, grad_sqnorm, clip_norm);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_sgd_step(const ds_optim_plan* p, float* w, const float* g, double lr, const double* grad_sqnorm,
                           float clip_norm, void* stream) {
  DS_PROPAGATE(check_flat("ds_sgd_step", p, w, g));
  DS_CHECK_ARG(!grad_sqnorm || clip_norm > 0.f, "ds_sgd_step: clip_norm must be positive");
  if (!p->chunks) return DS_OK;
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "sgd_apply_kernel", (double)p->elements * 12, "B");
  hipLaunchKernelGGL(apply_kernel<1>, dim3(p->chunks), dim3(256), 0, s, p->d_off, p->d_cnt, p->d_decay, w, g, nullptr, nullptr, (float)lr,
                     0.f, 0.f, 0.f, 0.f, 0.f, grad_sqnorm, clip_norm);
  DS_CHECK_LAUNCH();
  return DS_OK;
}
