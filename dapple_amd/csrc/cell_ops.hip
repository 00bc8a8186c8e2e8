// Operators of an AmoebaNet cell (amoeba_net/network_utils_slice.py:124-289, 427-806) in fp32 on NHWC tensors:
// train-mode batch normalisation, 3 x 3 pooling, depthwise k x k convolution, the 1 x k / k x 1 gathers that turn a
// factorised convolution into a GEMM, ReLU, sums and channel slices.  1 x 1 and gathered convolutions run on ds_gemm.
// Every kernel is bound by HBM: an element is read and written once (pooling and depthwise taps come from cache).
#include "common.h"

namespace {

constexpr int TPB = 256;
inline unsigned blocks_for(int64_t n) {
  int64_t b = (n + TPB - 1) / TPB;
  return (unsigned)(b < 1 ? 1 : (b > 1048576 ? 1048576 : b));
}

// ---------------------------------------------------------------- elementwise
__global__ __launch_bounds__(TPB) void relu_fwd_kernel(int64_t n, const float* __restrict__ x, float* __restrict__ y) {
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) y[i] = x[i] > 0.f ? x[i] : 0.f;
}
// dx (+)= dy where x > 0
__global__ __launch_bounds__(TPB) void relu_bwd_kernel(int64_t n, const float* __restrict__ x, const float* __restrict__ dy,
                                                      float* __restrict__ dx, int accumulate) {
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
    const float g = x[i] > 0.f ? dy[i] : 0.f;
    dx[i] = accumulate ? dx[i] + g : g;
  }
}
// (a fill kernel, not a memset: the callers' launches may be captured into a graph)
__global__ __launch_bounds__(TPB) void zero_kernel(int n, float* __restrict__ y) {
  for (int i = blockIdx.x * TPB + threadIdx.x; i < n; i += gridDim.x * TPB) y[i] = 0.f;
}
// y = a + b
__global__ __launch_bounds__(TPB) void add_kernel(int64_t n, const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ y) {
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) y[i] = a[i] + b[i];
}
// dst[r][dst_off + c] (+)= src[r][src_off + c]: channel concatenation, its gradient (a slice) and gradient sums
__global__ __launch_bounds__(TPB) void copy2d_kernel(int64_t rows, int cols, const float* __restrict__ src, int64_t ld_src,
                                                    float* __restrict__ dst, int64_t ld_dst, int accumulate) {
  const int64_t n = rows * cols;
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
    const int64_t r = i / cols;
    const int c = (int)(i - r * cols);
    const float v = src[r * ld_src + c];
    float* d = dst + r * ld_dst + c;
    *d = accumulate ? *d + v : v;
  }
}

// ---------------------------------------------------------------- batch normalisation (training mode)
// Column sums of a [rows, C] matrix: out[c] += sum_r f(x[r][c]) with f = x - shift[c] (MODE 0) or its square (MODE 1).
// One thread per channel, blockIdx.y walks row chunks; neighbouring threads read neighbouring channels.
template <int MODE>
__global__ __launch_bounds__(TPB) void bn_colsum_kernel(int64_t rows, int C, int64_t rows_per_block, const float* __restrict__ x,
                                                       const float* __restrict__ shift, float* __restrict__ out) {
  const int c = blockIdx.x * TPB + threadIdx.x;
  if (c >= C) return;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
  int64_t r1 = r0 + rows_per_block;
  if (r1 > rows) r1 = rows;
  const float s = shift ? shift[c] : 0.f;
  float acc = 0.f;
  for (int64_t r = r0; r < r1; ++r) {
    const float d = x[r * C + c] - s;
    acc += MODE == 0 ? d : d * d;
  }
  atomicAdd(out + c, acc);
}
// sums -> mean, rstd; and the moving averages (tf.nn.fused_batch_norm hands the unbiased variance to the average)
__global__ __launch_bounds__(TPB) void bn_finish_kernel(int C, int64_t rows, float eps, const float* __restrict__ sum, const float* __restrict__ sq,
                                                       float* __restrict__ mean, float* __restrict__ rstd, float* __restrict__ moving_mean,
                                                       float* __restrict__ moving_var, float decay, int phase) {
  const int c = blockIdx.x * TPB + threadIdx.x;
  if (c >= C) return;
  if (phase == 0) {
    mean[c] = sum[c] / (float)rows;
  } else {
    const float var = sq[c] / (float)rows;
    rstd[c] = rsqrtf(var + eps);
    if (moving_mean) moving_mean[c] -= (1.f - decay) * (moving_mean[c] - mean[c]);
    if (moving_var) {
      const float unbiased = rows > 1 ? var * ((float)rows / (float)(rows - 1)) : var;
      moving_var[c] -= (1.f - decay) * (moving_var[c] - unbiased);
    }
  }
}
__global__ __launch_bounds__(TPB) void bn_apply_kernel(int64_t n, int C, const float* __restrict__ x, const float* __restrict__ gamma,
                                                      const float* __restrict__ beta, const float* __restrict__ mean,
                                                      const float* __restrict__ rstd, float* __restrict__ y) {
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
    const int c = (int)(i % C);
    y[i] = (x[i] - mean[c]) * rstd[c] * gamma[c] + beta[c];
  }
}
// s1[c] += sum_r dy, s2[c] += sum_r dy * x_hat
__global__ __launch_bounds__(TPB) void bn_bwd_sums_kernel(int64_t rows, int C, int64_t rows_per_block, const float* __restrict__ dy,
                                                         const float* __restrict__ x, const float* __restrict__ mean,
                                                         const float* __restrict__ rstd, float* __restrict__ s1, float* __restrict__ s2) {
  const int c = blockIdx.x * TPB + threadIdx.x;
  if (c >= C) return;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
  int64_t r1 = r0 + rows_per_block;
  if (r1 > rows) r1 = rows;
  const float m = mean[c], rs = rstd[c];
  float a = 0.f, b = 0.f;
  for (int64_t r = r0; r < r1; ++r) {
    const float g = dy[r * C + c];
    a += g;
    b += g * (x[r * C + c] - m) * rs;
  }
  atomicAdd(s1 + c, a);
  atomicAdd(s2 + c, b);
}
// dx = gamma rstd (dy - s1 / rows - x_hat s2 / rows); dgamma += s2, dbeta += s1 (by the thread of row 0)
__global__ __launch_bounds__(TPB) void bn_bwd_apply_kernel(int64_t n, int C, int64_t rows, const float* __restrict__ dy, const float* __restrict__ x,
                                                          const float* __restrict__ gamma, const float* __restrict__ mean,
                                                          const float* __restrict__ rstd, const float* __restrict__ s1,
                                                          const float* __restrict__ s2, float* __restrict__ dx, float* __restrict__ dgamma,
                                                          float* __restrict__ dbeta, int accumulate) {
  const float inv = 1.f / (float)rows;
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
    const int c = (int)(i % C);
    const float xh = (x[i] - mean[c]) * rstd[c];
    const float g = gamma[c] * rstd[c] * (dy[i] - s1[c] * inv - xh * s2[c] * inv);
    dx[i] = accumulate ? dx[i] + g : g;
    if (i < C) {
      if (dgamma) dgamma[c] += s2[c];
      if (dbeta) dbeta[c] += s1[c];
    }
  }
}

// ---------------------------------------------------------------- 3 x 3 pooling, stride 1, 'SAME'
// kind 0: average over the taps inside the image (what TensorFlow's avg_pool does under 'SAME'); 1: maximum
__global__ __launch_bounds__(TPB) void pool3x3_fwd_kernel(int64_t n, int H, int W, int C, int kind, const float* __restrict__ x, float* __restrict__ y) {
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
    const int c = (int)(i % C);
    const int64_t p = i / C;
    const int w = (int)(p % W), h = (int)((p / W) % H);
    const int64_t img = p / ((int64_t)W * H);
    float acc = kind ? -INFINITY : 0.f;
    int cnt = 0;
    for (int dh = -1; dh <= 1; ++dh)
      for (int dw = -1; dw <= 1; ++dw) {
        const int hh = h + dh, ww = w + dw;
        if (hh < 0 || hh >= H || ww < 0 || ww >= W) continue;
        const float v = x[((img * H + hh) * W + ww) * C + c];
        if (kind) acc = v > acc ? v : acc;
        else acc += v;
        ++cnt;
      }
    y[i] = kind ? acc : acc / (float)cnt;
  }
}
// gather form: the input element looks at the (up to nine) windows that contain it
__global__ __launch_bounds__(TPB) void pool3x3_bwd_kernel(int64_t n, int H, int W, int C, int kind, const float* __restrict__ x,
                                                         const float* __restrict__ dy, float* __restrict__ dx, int accumulate) {
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
    const int c = (int)(i % C);
    const int64_t p = i / C;
    const int w = (int)(p % W), h = (int)((p / W) % H);
    const int64_t img = p / ((int64_t)W * H);
    float g = 0.f;
    for (int dh = -1; dh <= 1; ++dh)
      for (int dw = -1; dw <= 1; ++dw) {
        const int ch = h + dh, cw = w + dw;  // centre of a window that contains (h, w)
        if (ch < 0 || ch >= H || cw < 0 || cw >= W) continue;
        const float up = dy[((img * H + ch) * W + cw) * C + c];
        if (kind == 0) {
          const int nh = (ch > 0) + 1 + (ch < H - 1), nw = (cw > 0) + 1 + (cw < W - 1);
          g += up / (float)(nh * nw);
        } else {
          // the window's maximum, first in row-major order: does it sit at (h, w)?
          float best = -INFINITY;
          int bh = -2, bw = -2;
          for (int eh = -1; eh <= 1; ++eh)
            for (int ew = -1; ew <= 1; ++ew) {
              const int hh = ch + eh, ww = cw + ew;
              if (hh < 0 || hh >= H || ww < 0 || ww >= W) continue;
              const float v = x[((img * H + hh) * W + ww) * C + c];
              if (v > best) { best = v; bh = hh; bw = ww; }
            }
          if (bh == h && bw == w) g += up;
        }
      }
    dx[i] = accumulate ? dx[i] + g : g;
  }
}

// ---------------------------------------------------------------- depthwise k x k, stride 1, 'SAME' (k odd)
// y[n,h,w,c] = sum_ij x[n, h+i-p, w+j-p, c] w[i][j][c]; FLIP: the input gradient, taps mirrored
template <bool FLIP>
__global__ __launch_bounds__(TPB) void depthwise_kernel(int64_t n, int H, int W, int C, int k, const float* __restrict__ x,
                                                       const float* __restrict__ wt, float* __restrict__ y, int accumulate) {
  const int p0 = k / 2;
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
    const int c = (int)(i % C);
    const int64_t p = i / C;
    const int w = (int)(p % W), h = (int)((p / W) % H);
    const int64_t img = p / ((int64_t)W * H);
    float acc = 0.f;
    for (int a = 0; a < k; ++a) {
      const int hh = FLIP ? h - a + p0 : h + a - p0;
      if (hh < 0 || hh >= H) continue;
      for (int b = 0; b < k; ++b) {
        const int ww = FLIP ? w - b + p0 : w + b - p0;
        if (ww < 0 || ww >= W) continue;
        acc += x[((img * H + hh) * W + ww) * C + c] * wt[(a * k + b) * C + c];
      }
    }
    y[i] = accumulate ? y[i] + acc : acc;
  }
}
// dw[a][b][c] += sum_{n,h,w} x[n, h+a-p, w+b-p, c] dy[n,h,w,c]: blockIdx.y = tap, blockIdx.z = chunk of pixels
__global__ __launch_bounds__(TPB) void depthwise_wgrad_kernel(int64_t pixels, int H, int W, int C, int k, int64_t pixels_per_block,
                                                             const float* __restrict__ x, const float* __restrict__ dy, float* __restrict__ dw) {
  const int c = blockIdx.x * TPB + threadIdx.x;
  if (c >= C) return;
  const int a = blockIdx.y / k, b = blockIdx.y % k, p0 = k / 2;
  const int64_t q0 = (int64_t)blockIdx.z * pixels_per_block;
  int64_t q1 = q0 + pixels_per_block;
  if (q1 > pixels) q1 = pixels;
  float acc = 0.f;
  for (int64_t q = q0; q < q1; ++q) {
    const int w = (int)(q % W), h = (int)((q / W) % H);
    const int64_t img = q / ((int64_t)W * H);
    const int hh = h + a - p0, ww = w + b - p0;
    if (hh < 0 || hh >= H || ww < 0 || ww >= W) continue;
    acc += x[((img * H + hh) * W + ww) * C + c] * dy[q * C + c];
  }
  atomicAdd(dw + (int64_t)blockIdx.y * C + c, acc);
}

// ---------------------------------------------------------------- 1 x k / k x 1 gathers (stride 1, 'SAME', k odd)
// col[pixel][t * C + c] = x[pixel shifted by t - k/2 along the axis][c] (0 outside): a 1 x k (axis 1 = width) or k x 1
// (axis 0 = height) convolution is then col [pixels, k*C] x kernel [k*C, Cout]
__global__ __launch_bounds__(TPB) void gather1d_kernel(int64_t n, int H, int W, int C, int k, int axis, const float* __restrict__ x,
                                                      float* __restrict__ col) {
  const int p0 = k / 2;
  const int kc = k * C;
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
    const int j = (int)(i % kc);
    const int64_t p = i / kc;
    const int t = j / C, c = j - t * C;
    const int w = (int)(p % W), h = (int)((p / W) % H);
    const int64_t img = p / ((int64_t)W * H);
    const int hh = axis == 0 ? h + t - p0 : h, ww = axis == 1 ? w + t - p0 : w;
    col[i] = (hh < 0 || hh >= H || ww < 0 || ww >= W) ? 0.f : x[((img * H + hh) * W + ww) * C + c];
  }
}
// its transpose: dx[pixel][c] (+)= sum_t dcol[pixel shifted by p0 - t][t * C + c]
__global__ __launch_bounds__(TPB) void scatter1d_kernel(int64_t n, int H, int W, int C, int k, int axis, const float* __restrict__ dcol,
                                                       float* __restrict__ dx, int accumulate) {
  const int p0 = k / 2;
  const int kc = k * C;
  for (int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x; i < n; i += (int64_t)gridDim.x * TPB) {
    const int c = (int)(i % C);
    const int64_t p = i / C;
    const int w = (int)(p % W), h = (int)((p / W) % H);
    const int64_t img = p / ((int64_t)W * H);
    float g = 0.f;
    for (int t = 0; t < k; ++t) {
      const int hh = axis == 0 ? h - t + p0 : h, ww = axis == 1 ? w - t + p0 : w;
      if (hh < 0 || hh >= H || ww < 0 || ww >= W) continue;
      g += dcol[((img * H + hh) * W + ww) * kc + t * C + c];
    }
    dx[i] = accumulate ? dx[i] + g : g;
  }
}

int chunks_for(int64_t rows, int C, int64_t* per) {
  int64_t chunks = 2048 / ((C + TPB - 1) / TPB);   // enough blocks for every CU to hold several
  if (chunks > (rows + 15) / 16) chunks = (rows + 15) / 16;
  if (chunks < 1) chunks = 1;
  if (chunks > 65535) chunks = 65535;
  *per = (rows + chunks - 1) / chunks;
  return (int)((rows + *per - 1) / *per);
}

}  // namespace

#define CELL_PTRS(name, ...)                                           \
  do {                                                                 \
    const void* ps_[] = {__VA_ARGS__};                                 \
    for (const void* p_ : ps_) DS_CHECK_ARG(p_ != nullptr, name ": null pointer"); \
  } while (0)

extern "C" int ds_relu_fwd(int64_t n, const float* x, float* y, void* stream) {
  DS_CHECK_ARG(n > 0, "ds_relu_fwd: n must be positive");
  CELL_PTRS("ds_relu_fwd", x, y);
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "relu_fwd_kernel", (double)n * 8, "B");
  hipLaunchKernelGGL(relu_fwd_kernel, dim3(blocks_for(n)), dim3(TPB), 0, s, n, x, y);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_relu_bwd(int64_t n, const float* x, const float* dy, float* dx, int accumulate, void* stream) {
  DS_CHECK_ARG(n > 0, "ds_relu_bwd: n must be positive");
  CELL_PTRS("ds_relu_bwd", x, dy, dx);
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "relu_bwd_kernel", (double)n * 12, "B");
  hipLaunchKernelGGL(relu_bwd_kernel, dim3(blocks_for(n)), dim3(TPB), 0, s, n, x, dy, dx, accumulate);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_add(int64_t n, const float* a, const float* b, float* y, void* stream) {
  DS_CHECK_ARG(n > 0, "ds_add: n must be positive");
  CELL_PTRS("ds_add", a, b, y);
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "add_kernel", (double)n * 12, "B");
  hipLaunchKernelGGL(add_kernel, dim3(blocks_for(n)), dim3(TPB), 0, s, n, a, b, y);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_copy2d(int64_t rows, int cols, const float* src, int64_t ld_src, float* dst, int64_t ld_dst, int accumulate, void* stream) {
  DS_CHECK_ARG(rows > 0 && cols > 0 && ld_src >= cols && ld_dst >= cols, "ds_copy2d: bad shape");
  CELL_PTRS("ds_copy2d", src, dst);
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "copy2d_kernel", (double)rows * cols * 8, "B");
  hipLaunchKernelGGL(copy2d_kernel, dim3(blocks_for(rows * cols)), dim3(TPB), 0, s, rows, cols, src, ld_src, dst, ld_dst, accumulate);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" size_t ds_batchnorm_workspace_bytes(int channels) { return (size_t)2 * channels * sizeof(float); }

extern "C" int ds_batchnorm_train_fwd(int64_t rows, int channels, const float* x, const float* gamma, const float* beta, float eps, float* y,
                                      float* save_mean, float* save_rstd, float* moving_mean, float* moving_var, float decay, void* workspace,
                                      void* stream) {
  DS_CHECK_ARG(rows > 0 && channels > 0, "ds_batchnorm_train_fwd: bad shape");
  CELL_PTRS("ds_batchnorm_train_fwd", x, gamma, beta, y, save_mean, save_rstd, workspace);
  hipStream_t s = (hipStream_t)stream;
  float* sum = (float*)workspace;
  float* sq = sum + channels;
  int64_t per;
  const int chunks = chunks_for(rows, channels, &per);
  const dim3 grid((channels + TPB - 1) / TPB, chunks), cgrid((channels + TPB - 1) / TPB);
  ds_prof_scope prof(s, "batchnorm_train_fwd", (double)rows * channels * 16, "B");
  hipLaunchKernelGGL(zero_kernel, dim3(blocks_for(2 * channels)), dim3(TPB), 0, s, 2 * channels, sum);
  hipLaunchKernelGGL(bn_colsum_kernel<0>, grid, dim3(TPB), 0, s, rows, channels, per, x, (const float*)nullptr, sum);
  hipLaunchKernelGGL(bn_finish_kernel, cgrid, dim3(TPB), 0, s, channels, rows, eps, sum, sq, save_mean, save_rstd, moving_mean, moving_var, decay, 0);
  hipLaunchKernelGGL(bn_colsum_kernel<1>, grid, dim3(TPB), 0, s, rows, channels, per, x, (const float*)save_mean, sq);
  hipLaunchKernelGGL(bn_finish_kernel, cgrid, dim3(TPB), 0, s, channels, rows, eps, sum, sq, save_mean, save_rstd, moving_mean, moving_var, decay, 1);
  hipLaunchKernelGGL(bn_apply_kernel, dim3(blocks_for(rows * channels)), dim3(TPB), 0, s, rows * channels, channels, x, gamma, beta, save_mean,
                     save_rstd, y);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_batchnorm_train_bwd(int64_t rows, int channels, const float* dy, const float* x, const float* gamma, const float* save_mean,
                                      const float* save_rstd, float* dx, int accumulate_dx, float* d_gamma, float* d_beta, void* workspace,
                                      void* stream) {
  DS_CHECK_ARG(rows > 0 && channels > 0, "ds_batchnorm_train_bwd: bad shape");
  CELL_PTRS("ds_batchnorm_train_bwd", dy, x, gamma, save_mean, save_rstd, dx, workspace);
  hipStream_t s = (hipStream_t)stream;
  float* s1 = (float*)workspace;
  float* s2 = s1 + channels;
  int64_t per;
  const int chunks = chunks_for(rows, channels, &per);
  const dim3 grid((channels + TPB - 1) / TPB, chunks);
  ds_prof_scope prof(s, "batchnorm_train_bwd", (double)rows * channels * 20, "B");
  hipLaunchKernelGGL(zero_kernel, dim3(blocks_for(2 * channels)), dim3(TPB), 0, s, 2 * channels, s1);
  hipLaunchKernelGGL(bn_bwd_sums_kernel, grid, dim3(TPB), 0, s, rows, channels, per, dy, x, save_mean, save_rstd, s1, s2);
  hipLaunchKernelGGL(bn_bwd_apply_kernel, dim3(blocks_for(rows * channels)), dim3(TPB), 0, s, rows * channels, channels, rows, dy, x, gamma,
                     save_mean, save_rstd, s1, s2, dx, d_gamma, d_beta, accumulate_dx);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_pool3x3_fwd(int kind, int n, int h, int w, int c, const float* x, float* y, void* stream) {
  DS_CHECK_ARG((kind == 0 || kind == 1) && n > 0 && h > 0 && w > 0 && c > 0, "ds_pool3x3_fwd: bad argument");
  CELL_PTRS("ds_pool3x3_fwd", x, y);
  hipStream_t s = (hipStream_t)stream;
  const int64_t total = (int64_t)n * h * w * c;
  ds_prof_scope prof(s, "pool3x3_fwd_kernel", (double)total * 8, "B");
  hipLaunchKernelGGL(pool3x3_fwd_kernel, dim3(blocks_for(total)), dim3(TPB), 0, s, total, h, w, c, kind, x, y);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_pool3x3_bwd(int kind, int n, int h, int w, int c, const float* x, const float* dy, float* dx, int accumulate, void* stream) {
  DS_CHECK_ARG((kind == 0 || kind == 1) && n > 0 && h > 0 && w > 0 && c > 0, "ds_pool3x3_bwd: bad argument");
  CELL_PTRS("ds_pool3x3_bwd", x, dy, dx);
  hipStream_t s = (hipStream_t)stream;
  const int64_t total = (int64_t)n * h * w * c;
  ds_prof_scope prof(s, "pool3x3_bwd_kernel", (double)total * 12, "B");
  hipLaunchKernelGGL(pool3x3_bwd_kernel, dim3(blocks_for(total)), dim3(TPB), 0, s, total, h, w, c, kind, x, dy, dx, accumulate);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_depthwise_conv_fwd(int n, int h, int w, int c, int k, const float* x, const float* kernel, float* y, void* stream) {
  DS_CHECK_ARG(n > 0 && h > 0 && w > 0 && c > 0 && k > 0 && (k & 1), "ds_depthwise_conv_fwd: bad shape (k must be odd)");
  CELL_PTRS("ds_depthwise_conv_fwd", x, kernel, y);
  hipStream_t s = (hipStream_t)stream;
  const int64_t total = (int64_t)n * h * w * c;
  ds_prof_scope prof(s, "depthwise_kernel", (double)total * 8, "B");
  hipLaunchKernelGGL(depthwise_kernel<false>, dim3(blocks_for(total)), dim3(TPB), 0, s, total, h, w, c, k, x, kernel, y, 0);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_depthwise_conv_bwd(int n, int h, int w, int c, int k, const float* x, const float* kernel, const float* dy, float* dx,
                                     int accumulate_dx, float* d_kernel, void* stream) {
  DS_CHECK_ARG(n > 0 && h > 0 && w > 0 && c > 0 && k > 0 && (k & 1), "ds_depthwise_conv_bwd: bad shape (k must be odd)");
  CELL_PTRS("ds_depthwise_conv_bwd", x, kernel, dy);
  hipStream_t s = (hipStream_t)stream;
  const int64_t total = (int64_t)n * h * w * c;
  ds_prof_scope prof(s, "depthwise_bwd", (double)total * 20, "B");
  if (dx) hipLaunchKernelGGL(depthwise_kernel<true>, dim3(blocks_for(total)), dim3(TPB), 0, s, total, h, w, c, k, dy, kernel, dx, accumulate_dx);
  if (d_kernel) {
    const int64_t pixels = (int64_t)n * h * w;
    int64_t chunks = 512 / (k * k);
    if (chunks < 1) chunks = 1;
    if (chunks > (pixels + 63) / 64) chunks = (pixels + 63) / 64;
    const int64_t per = (pixels + chunks - 1) / chunks;
    const dim3 grid((c + TPB - 1) / TPB, k * k, (unsigned)((pixels + per - 1) / per));
    hipLaunchKernelGGL(depthwise_wgrad_kernel, grid, dim3(TPB), 0, s, pixels, h, w, c, k, per, x, dy, d_kernel);
  }
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_gather1d(int n, int h, int w, int c, int k, int axis, const float* x, float* col, void* stream) {
  DS_CHECK_ARG(n > 0 && h > 0 && w > 0 && c > 0 && k > 0 && (k & 1) && (axis == 0 || axis == 1), "ds_gather1d: bad argument");
  CELL_PTRS("ds_gather1d", x, col);
  hipStream_t s = (hipStream_t)stream;
  const int64_t total = (int64_t)n * h * w * c * k;
  ds_prof_scope prof(s, "gather1d_kernel", (double)total * 8, "B");
  hipLaunchKernelGGL(gather1d_kernel, dim3(blocks_for(total)), dim3(TPB), 0, s, total, h, w, c, k, axis, x, col);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_scatter1d(int n, int h, int w, int c, int k, int axis, const float* dcol, float* dx, int accumulate, void* stream) {
  DS_CHECK_ARG(n > 0 && h > 0 && w > 0 && c > 0 && k > 0 && (k & 1) && (axis == 0 || axis == 1), "ds_scatter1d: bad argument");
  CELL_PTRS("ds_scatter1d", dcol, dx);
  hipStream_t s = (hipStream_t)stream;
  const int64_t total = (int64_t)n * h * w * c;
  ds_prof_scope prof(s, "scatter1d_kernel", (double)total * (4.0 * k + 4), "B");
  hipLaunchKernelGGL(scatter1d_kernel, dim3(blocks_for(total)), dim3(TPB), 0, s, total, h, w, c, k, axis, dcol, dx, accumulate);
  DS_CHECK_LAUNCH();
  return DS_OK;
}
