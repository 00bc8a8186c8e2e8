// SQuAD-2 head of the last XLNet stage, xlnet/losses/xlnet_loss.py:36-120 (XLnetLoss.call), forward and backward in
// fp32.  x is time-major [seq, batch, hidden]: row l*batch + b.  Three branches share x:
//   start:  sl[b][l] = x . start_w + start_b; masked log-softmax over l; loss term at start_positions           (:51-54, :78-79)
//   end:    t = tanh(x W0a + x[start_positions[b], b] W0b + b0); LayerNorm; el = . end_w1 + end_b1; same loss   (:57-76, :82-87)
//   answer: a = tanh([sum_l softmax(sl)[b][l] x[l, b], x[cls_index[b], b]] ans_w0 + ans_b0) * dropout;
//           cls = a . ans_w1; sigmoid cross entropy with is_impossible                                          (:90-117)
// The only matrix-sized work is the [seq*batch, hidden] x [hidden, hidden] product of the end branch and its two
// gradients (ds_gemm); the rest is row work over x and batch-sized vectors.
#include <math.h>

#include "common.h"

namespace {

constexpr float LN_EPS = 1e-14f;  // K.epsilon() ** 2, layers/layer_normalization.py:37-38

__global__ __launch_bounds__(256) void xh_clear_kernel(float* __restrict__ p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// one wave per row (l, b): out[b][l] = x[row] . v[b * vstride ..] (+ bias[0])
__global__ __launch_bounds__(256) void xh_rowdot_kernel(int S, int B, int H, const float* __restrict__ x, const float* __restrict__ v,
                                                        int64_t vstride, const float* __restrict__ bias, float* __restrict__ out) {
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= S * B) return;
  const int l = row / B, b = row % B;
  const float* vr = v + (int64_t)b * vstride;
  float a = 0.f;
  for (int c = lane * 4; c < H; c += 256) {
    const f32x4 xv = *reinterpret_cast<const f32x4*>(x + (int64_t)row * H + c);
    const f32x4 vv = *reinterpret_cast<const f32x4*>(vr + c);
    a += xv[0] * vv[0] + xv[1] * vv[1] + xv[2] * vv[2] + xv[3] * vv[3];
  }
  a = wave_sum(a);
  if (lane == 0) out[(int64_t)b * S + l] = a + (bias ? bias[0] : 0.f);
}

// grid (ceil(H/256), B, 2): picked[z][b][c] = x[idx_z[b], b, c], zero when idx is outside [0, S) (tf.one_hot + einsum)
__global__ __launch_bounds__(256) void xh_pick_kernel(int S, int B, int H, const float* __restrict__ x, const int32_t* __restrict__ idx0,
                                                      const int32_t* __restrict__ idx1, float* __restrict__ out0, float* __restrict__ out1) {
  const int c = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
  if (c >= H) return;
  const int pos = blockIdx.z == 0 ? idx0[b] : idx1[b];
  float* out = blockIdx.z == 0 ? out0 : out1;
  out[(int64_t)b * H + c] = (pos >= 0 && pos < S) ? x[((int64_t)pos * B + b) * H + c] : 0.f;
}

// one wave per (b, k): din[b][k] = sum_j dout[b][j] W[k][j]
__global__ __launch_bounds__(256) void xh_dense_din_kernel(int B, int K, int N, const float* __restrict__ dout, const float* __restrict__ W,
                                                           float* __restrict__ din) {
  const int lane = threadIdx.x & 63, k = blockIdx.x * 4 + (threadIdx.x >> 6), b = blockIdx.y;
  if (k >= K) return;
  float a = 0.f;
  for (int j = lane; j < N; j += 64) a += dout[(int64_t)b * N + j] * W[(int64_t)k * N + j];
  a = wave_sum(a);
  if (lane == 0) din[(int64_t)b * K + k] = a;
}

// thread per (k, j): dW[k][j] += sum_b in[b][k] dout[b][j]; row k = 0 also adds dbias[j] += sum_b dout[b][j]
__global__ __launch_bounds__(256) void xh_dense_dw_kernel(int B, int H, int N, const float* __restrict__ in0, const float* __restrict__ in1,
                                                          const float* __restrict__ dout, float* __restrict__ dW, float* __restrict__ dbias) {
  const int j = blockIdx.x * 256 + threadIdx.x, k = blockIdx.y;
  if (j >= N) return;
  const float* in = k < H ? in0 : in1;
  const int kk = k < H ? k : k - H;
  float a = 0.f, s = 0.f;
  for (int b = 0; b < B; ++b) {
    const float d = dout[(int64_t)b * N + j];
    a += in[(int64_t)b * H + kk] * d;
    s += d;
  }
  dW[(int64_t)k * N + j] += a;
  if (k == 0 && dbias) dbias[j] += s;
}

// t[row][c] = tanh(t[row][c] + add[b][c])
__global__ __launch_bounds__(256) void xh_addtanh_kernel(int64_t n4, int B, int H, float* __restrict__ t, const float* __restrict__ add) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  const int64_t e = i * 4;
  const int c = (int)(e % H), b = (int)((e / H) % B);
  f32x4 v = *reinterpret_cast<f32x4*>(t + e);
  const f32x4 a = *reinterpret_cast<const f32x4*>(add + (int64_t)b * H + c);
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = tanhf(v[j] + a[j]);
  *reinterpret_cast<f32x4*>(t + e) = v;
}

// dt[i] *= 1 - t[i]^2
__global__ __launch_bounds__(256) void xh_dtanh_kernel(int64_t n4, float* __restrict__ dt, const float* __restrict__ t) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  f32x4 d = *reinterpret_cast<f32x4*>(dt + i * 4);
  const f32x4 v = *reinterpret_cast<const f32x4*>(t + i * 4);
#pragma unroll
  for (int j = 0; j < 4; ++j) d[j] *= 1.f - v[j] * v[j];
  *reinterpret_cast<f32x4*>(dt + i * 4) = d;
}

__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// one block per b: lm = lg (1 - pm) - 1e30 pm; log-softmax over l; loss += -wgt * log_softmax[pos];
// p_out (nullable) = softmax; g_out[l] = wgt (p - onehot) (times (1 - pm) when masked_grad): d loss / d lm (or / d lg)
__global__ __launch_bounds__(256) void xh_seq_loss_kernel(int S, const float* __restrict__ logits, const float* __restrict__ p_mask,
                                                          const int32_t* __restrict__ positions, float wgt, int masked_grad,
                                                          float* __restrict__ p_out, float* __restrict__ g_out, float* __restrict__ loss) {
  __shared__ float red[4];
  const int b = blockIdx.x;
  const float* lg = logits + (int64_t)b * S;
  const float* pm = p_mask + (int64_t)b * S;
  const int pos = positions[b];
  float mx = -INFINITY;
  for (int l = threadIdx.x; l < S; l += 256) mx = fmaxf(mx, lg[l] * (1.f - pm[l]) - 1e30f * pm[l]);
  mx = block_max(mx, red);
  float sum = 0.f;
  for (int l = threadIdx.x; l < S; l += 256) sum += expf(lg[l] * (1.f - pm[l]) - 1e30f * pm[l] - mx);
  sum = block_sum(sum, red);
  const float lse = mx + logf(sum);
  const bool valid = pos >= 0 && pos < S;
  for (int l = threadIdx.x; l < S; l += 256) {
    const float lm = lg[l] * (1.f - pm[l]) - 1e30f * pm[l];
    const float p = expf(lm - lse);
    if (p_out) p_out[(int64_t)b * S + l] = p;
    float g = valid ? wgt * (p - (l == pos ? 1.f : 0.f)) : 0.f;
    if (masked_grad) g *= 1.f - pm[l];
    g_out[(int64_t)b * S + l] = g;
    if (valid && l == pos) atomicAdd(loss, -wgt * (lm - lse));
  }
}

// grid (ceil(H/256), B, LS): out[b][c] += sum over this block's share of l of p[b][l] x[l, b, c]
__global__ __launch_bounds__(256) void xh_wsum_kernel(int S, int B, int H, const float* __restrict__ x, const float* __restrict__ p,
                                                      float* __restrict__ out) {
  const int c = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
  if (c >= H) return;
  const int per = (S + gridDim.z - 1) / gridDim.z;
  const int l0 = blockIdx.z * per, l1 = l0 + per < S ? l0 + per : S;
  float a = 0.f;
  for (int l = l0; l < l1; ++l) a += p[(int64_t)b * S + l] * x[((int64_t)l * B + b) * H + c];
  atomicAdd(out + (int64_t)b * H + c, a);
}

// one block per b: cls = sum_j a[b][j] drop[b][j] w1[j]; loss += wgt * sigmoid_ce(cls, y[b]);
// dpre[b][j] = wgt (sigmoid(cls) - y) w1[j] drop (1 - a^2); dw1[j] += wgt (sigmoid(cls) - y) a drop
__global__ __launch_bounds__(256) void xh_answer_kernel(int H, const float* __restrict__ a, const float* __restrict__ drop,
                                                        const float* __restrict__ w1, const float* __restrict__ y, float wgt,
                                                        float* __restrict__ cls, float* __restrict__ loss, float* __restrict__ dpre,
                                                        float* __restrict__ dw1) {
  __shared__ float red[4];
  const int b = blockIdx.x;
  float s = 0.f;
  for (int j = threadIdx.x; j < H; j += 256) s += a[(int64_t)b * H + j] * (drop ? drop[(int64_t)b * H + j] : 1.f) * w1[j];
  const float z = block_sum(s, red);
  const float yb = y[b];
  const float sig = 1.f / (1.f + expf(-z));
  const float d = wgt * (sig - yb);
  if (threadIdx.x == 0) {
    cls[b] = z;
    atomicAdd(loss, wgt * (fmaxf(z, 0.f) - z * yb + log1pf(expf(-fabsf(z)))));  // tf.nn.sigmoid_cross_entropy_with_logits
  }
  for (int j = threadIdx.x; j < H; j += 256) {
    const float av = a[(int64_t)b * H + j], dr = drop ? drop[(int64_t)b * H + j] : 1.f;
    if (dpre) dpre[(int64_t)b * H + j] = d * w1[j] * dr * (1.f - av * av);
    if (dw1) atomicAdd(dw1 + j, d * av * dr);
  }
}

// one block per b: dsl[l] = (g[l] + p[l] (dp[l] - sum_l' p dp)) (1 - pm[l])
__global__ __launch_bounds__(256) void xh_start_bwd_kernel(int S, const float* __restrict__ p, const float* __restrict__ dp,
                                                           const float* __restrict__ g, const float* __restrict__ p_mask,
                                                           float* __restrict__ dsl) {
  __shared__ float red[4];
  const int64_t o = (int64_t)blockIdx.x * S;
  float s = 0.f;
  for (int l = threadIdx.x; l < S; l += 256) s += p[o + l] * dp[o + l];
  s = block_sum(s, red);
  for (int l = threadIdx.x; l < S; l += 256) dsl[o + l] = (g[o + l] + p[o + l] * (dp[o + l] - s)) * (1.f - p_mask[o + l]);
}

// block = RPB rows, in place: y[row][c] (the normalised end features) -> d[b][l] w[c];
// dw[c] += sum_rows d y; db += sum_rows d
template <int RPB>
__global__ __launch_bounds__(256) void xh_outer_kernel(int S, int B, int H, float* __restrict__ y, const float* __restrict__ d,
                                                       const float* __restrict__ w, float* __restrict__ dw, float* __restrict__ db) {
  const int rows = S * B, r0 = blockIdx.x * RPB, r1 = r0 + RPB < rows ? r0 + RPB : rows;
  for (int c = threadIdx.x; c < H; c += 256) {
    const float wc = w[c];
    float g = 0.f;
    for (int r = r0; r < r1; ++r) {
      const float dv = d[(int64_t)(r % B) * S + r / B];
      g += dv * y[(int64_t)r * H + c];
      y[(int64_t)r * H + c] = dv * wc;
    }
    if (dw) atomicAdd(dw + c, g);
  }
  if (db && threadIdx.x == 0) {
    float s = 0.f;
    for (int r = r0; r < r1; ++r) s += d[(int64_t)(r % B) * S + r / B];
    atomicAdd(db, s);
  }
}

// block = RPB rows (dxe may be dx itself): dx[row][c] = dxe[row][c] + dsl[b][l] ws[c] + p[b][l] dsf[b][c] + [l == start[b]] dpick0[b][c]
//                               + [l == cls[b]] dpick1[b][c];  dws[c] += sum_rows dsl x;  dbs += sum_rows dsl
template <typename T, int RPB>
__global__ __launch_bounds__(256) void xh_final_kernel(int S, int B, int H, const float* __restrict__ x, const float* dxe,
                                                       const float* __restrict__ dsl, const float* __restrict__ p,
                                                       const float* __restrict__ ws, const float* __restrict__ dcat,
                                                       const float* __restrict__ dpick0, const int32_t* __restrict__ start,
                                                       const int32_t* __restrict__ cls, T* dx, float* __restrict__ dws,
                                                       float* __restrict__ dbs) {
  const int rows = S * B, r0 = blockIdx.x * RPB, r1 = r0 + RPB < rows ? r0 + RPB : rows;
  for (int c = threadIdx.x; c < H; c += 256) {
    const float wc = ws[c];
    float g = 0.f;
    for (int r = r0; r < r1; ++r) {
      const int l = r / B, b = r % B;
      const float d = dsl[(int64_t)b * S + l];
      if (dx) {
        float v = dxe[(int64_t)r * H + c] + d * wc + p[(int64_t)b * S + l] * dcat[(int64_t)b * 2 * H + c];
        if (l == start[b]) v += dpick0[(int64_t)b * H + c];
        if (l == cls[b]) v += dcat[(int64_t)b * 2 * H + H + c];
        dx[(int64_t)r * H + c] = from_f32<T>(v);
      }
      if (dws) g += d * x[(int64_t)r * H + c];
    }
    if (dws) atomicAdd(dws + c, g);
  }
  if (dbs && threadIdx.x == 0) {
    float s = 0.f;
    for (int r = r0; r < r1; ++r) s += dsl[(int64_t)(r % B) * S + r / B];
    atomicAdd(dbs, s);
  }
}

struct Layout {
  size_t xf, t, y, dt, stats, sl_g, p, dp, dsl, del, pick0, pick1, sfeat, sfw, ans, dans, dcat, dsfw, dpick0, lng, total;
};
Layout make_layout(int dtype, int S, int B, int H) {
  Layout L;
  size_t off = 0;
  auto take = [&](size_t n) { size_t o = off; off += (n * sizeof(float) + 255) / 256 * 256; return o; };
  const size_t big = (size_t)S * B * H, bs = (size_t)B * S, bh = (size_t)B * H;
  L.xf = dtype == DS_BF16 ? take(big) : 0;
  L.t = take(big); L.y = take(big); L.dt = take(big); L.stats = take((size_t)S * B * 2);
  L.sl_g = take(bs); L.p = take(bs); L.dp = take(bs); L.dsl = take(bs); L.del = take(bs);
  L.pick0 = take(bh); L.pick1 = take(bh);
  L.sfeat = take(bh); L.dsfw = take(bh);   // the two accumulators cleared at the start, adjacent
  L.sfw = take(bh); L.ans = take(bh); L.dans = take(bh); L.dcat = take(2 * bh); L.dpick0 = take(bh); L.lng = take(2 * (size_t)H);
  L.total = off;
  return L;
}

int gemm_f32(int am, int bm, int m, int n, int k, const float* a, int64_t lda, const float* b, int64_t ldb, float* c, int64_t ldc, int flags,
             hipStream_t s) {
  ds_gemm_desc d = {};
  d.dtype = DS_F32; d.a_major = am; d.b_major = bm; d.m = m; d.n = n; d.k = k; d.lda = lda; d.ldb = ldb; d.ldc = ldc;
  d.batch = 1; d.batch_inner = 1; d.flags = flags; d.alpha = 1.f; d.a = a; d.b = b; d.c = c;
  return ds_gemm(&d, s);
}

inline unsigned cdiv(int64_t a, int64_t b) { return (unsigned)((a + b - 1) / b); }

}  // namespace

extern "C" size_t ds_xlnet_squad_head_workspace_bytes(int dtype, int seq, int batch, int hidden) {
  if (seq <= 0 || batch <= 0 || hidden <= 0) return 0;
  return make_layout(dtype, seq, batch, hidden).total;
}

extern "C" int ds_xlnet_squad_head(int dtype, int seq, int batch, int hidden, const void* x, const ds_xlnet_head_params* w,
                                   const int32_t* cls_index, const int32_t* start_positions, const int32_t* end_positions,
                                   const float* is_impossible, const float* p_mask, const float* dropout_mask, float loss_scale,
                                   float* loss, float* start_logits, float* end_logits, float* cls_logits, void* dx,
                                   const ds_xlnet_head_params* g, void* workspace, size_t workspace_bytes, void* stream) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "ds_xlnet_squad_head: dtype %d", dtype);
  DS_CHECK_ARG(seq > 0 && batch > 0 && hidden > 0 && hidden % 8 == 0, "ds_xlnet_squad_head: seq %d, batch %d, hidden %d (multiple of 8)",
               seq, batch, hidden);
  DS_CHECK_ARG((int64_t)seq * batch * hidden < (int64_t)1 << 31, "ds_xlnet_squad_head: seq * batch * hidden exceeds 2^31");
  DS_CHECK_ARG(batch <= 65535, "ds_xlnet_squad_head: batch %d exceeds 65535", batch);
  DS_CHECK_ARG(x && w && cls_index && start_positions && end_positions && is_impossible && p_mask && loss && start_logits && end_logits &&
               cls_logits && workspace, "ds_xlnet_squad_head: null pointer");
  DS_CHECK_ARG(w->start_w && w->start_b && w->end_w0 && w->end_b0 && w->ln_gamma && w->ln_beta && w->end_w1 && w->end_b1 && w->ans_w0 &&
               w->ans_b0 && w->ans_w1, "ds_xlnet_squad_head: null weight pointer");
  DS_CHECK_ARG(!g || (g->start_w && g->start_b && g->end_w0 && g->end_b0 && g->ln_gamma && g->ln_beta && g->end_w1 && g->end_b1 &&
                      g->ans_w0 && g->ans_b0 && g->ans_w1), "ds_xlnet_squad_head: pass every gradient pointer or no grads struct");
  DS_CHECK_ARG(ds_aligned16(x) && ds_aligned16(dx) && ds_aligned16(workspace) && ds_aligned16(w->start_w) && ds_aligned16(w->end_w0) &&
               ds_aligned16(w->end_w1) && ds_aligned16(w->ln_gamma), "ds_xlnet_squad_head: x, dx, workspace and weights must be 16-byte aligned");
  const int S = seq, B = batch, H = hidden, rows = S * B;
  const Layout L = make_layout(dtype, S, B, H);
  DS_CHECK_ARG(workspace_bytes >= L.total, "ds_xlnet_squad_head: workspace of %zu bytes, %zu needed", workspace_bytes, L.total);
  hipStream_t s = (hipStream_t)stream;
  char* ws = (char*)workspace;
  auto F = [&](size_t off) { return reinterpret_cast<float*>(ws + off); };
  const int64_t big = (int64_t)rows * H;
  const bool bwd = dx || g;
  const float wgt = loss_scale * 0.5f / (float)B;  // each of the three terms enters with 1/2 and a mean over the batch

  // accumulators: the loss, the weighted start feature and the per-sample sums of the end branch's pre-activation gradient
  hipLaunchKernelGGL(xh_clear_kernel, dim3(1), dim3(256), 0, s, loss, (int64_t)1);
  const int64_t nclear = (int64_t)((L.sfw - L.sfeat) / sizeof(float));
  hipLaunchKernelGGL(xh_clear_kernel, dim3(cdiv(nclear, 256)), dim3(256), 0, s, F(L.sfeat), nclear);
  DS_CHECK_LAUNCH();
  const float* xf = (const float*)x;
  if (dtype == DS_BF16) {
    DS_PROPAGATE(ds_cast_bf16_to_f32(F(L.xf), x, (size_t)big, s));
    xf = F(L.xf);
  }
  // ---- start branch
  hipLaunchKernelGGL(xh_rowdot_kernel, dim3(cdiv(rows, 4)), dim3(256), 0, s, S, B, H, xf, w->start_w, (int64_t)0, w->start_b, start_logits);
  hipLaunchKernelGGL(xh_seq_loss_kernel, dim3(B), dim3(256), 0, s, S, start_logits, p_mask, start_positions, wgt, 0, F(L.p), F(L.sl_g), loss);
  // ---- end branch
  hipLaunchKernelGGL(xh_pick_kernel, dim3(cdiv(H, 256), B, 2), dim3(256), 0, s, S, B, H, xf, start_positions, cls_index, F(L.pick0), F(L.pick1));
  hipLaunchKernelGGL((ds_small_dense_kernel<float, 0>), dim3(cdiv(H, 64), B), dim3(1024), 0, s, H, 0, H, (const float*)F(L.pick0), (int64_t)H,
                     (const float*)nullptr, (int64_t)0, (const float*)(w->end_w0 + (int64_t)H * H), (const float*)w->end_b0, F(L.sfw));
  DS_CHECK_LAUNCH();
  DS_PROPAGATE(gemm_f32(DS_K_MAJOR, DS_MN_MAJOR, rows, H, H, xf, H, w->end_w0, H, F(L.t), H, 0, s));
  hipLaunchKernelGGL(xh_addtanh_kernel, dim3(cdiv(big / 4, 256)), dim3(256), 0, s, big / 4, B, H, F(L.t), F(L.sfw));
  DS_CHECK_LAUNCH();
  DS_PROPAGATE(ds_layernorm_fwd(DS_F32, rows, H, F(L.t), w->ln_gamma, w->ln_beta, LN_EPS, F(L.y), F(L.stats), s));
  hipLaunchKernelGGL(xh_rowdot_kernel, dim3(cdiv(rows, 4)), dim3(256), 0, s, S, B, H, F(L.y), w->end_w1, (int64_t)0, w->end_b1, end_logits);
  hipLaunchKernelGGL(xh_seq_loss_kernel, dim3(B), dim3(256), 0, s, S, end_logits, p_mask, end_positions, wgt, 1, (float*)nullptr, F(L.del), loss);
  // ---- answerability branch
  hipLaunchKernelGGL(xh_wsum_kernel, dim3(cdiv(H, 256), B, 16), dim3(256), 0, s, S, B, H, xf, F(L.p), F(L.sfeat));
  hipLaunchKernelGGL((ds_small_dense_kernel<float, 1>), dim3(cdiv(H, 64), B), dim3(1024), 0, s, H, H, H, (const float*)F(L.sfeat), (int64_t)H,
                     (const float*)F(L.pick1), (int64_t)H, (const float*)w->ans_w0, (const float*)w->ans_b0, F(L.ans));
  hipLaunchKernelGGL(xh_answer_kernel, dim3(B), dim3(256), 0, s, H, F(L.ans), dropout_mask, w->ans_w1, is_impossible, wgt, cls_logits, loss,
                     bwd ? F(L.dans) : nullptr, g ? g->ans_w1 : nullptr);
  DS_CHECK_LAUNCH();
  if (!bwd) return DS_OK;

  // ---- backward: answerability branch down to the start probabilities
  hipLaunchKernelGGL(xh_dense_din_kernel, dim3(cdiv(2 * H, 4), B), dim3(256), 0, s, B, 2 * H, H, F(L.dans), w->ans_w0, F(L.dcat));
  if (g)
    hipLaunchKernelGGL(xh_dense_dw_kernel, dim3(cdiv(H, 256), 2 * H), dim3(256), 0, s, B, H, H, F(L.sfeat), F(L.pick1), F(L.dans), g->ans_w0,
                       g->ans_b0);
  hipLaunchKernelGGL(xh_rowdot_kernel, dim3(cdiv(rows, 4)), dim3(256), 0, s, S, B, H, xf, F(L.dcat), (int64_t)2 * H, (const float*)nullptr,
                     F(L.dp));
  hipLaunchKernelGGL(xh_start_bwd_kernel, dim3(B), dim3(256), 0, s, S, F(L.p), F(L.dp), F(L.sl_g), p_mask, F(L.dsl));
  // ---- backward: end branch
  constexpr int RPB = 8;
  hipLaunchKernelGGL((xh_outer_kernel<RPB>), dim3(cdiv(rows, RPB)), dim3(256), 0, s, S, B, H, F(L.y), F(L.del), w->end_w1,
                     g ? g->end_w1 : nullptr, g ? g->end_b1 : nullptr);
  DS_CHECK_LAUNCH();
  DS_PROPAGATE(ds_layernorm_bwd(DS_F32, rows, H, F(L.y), F(L.t), w->ln_gamma, F(L.stats), nullptr, F(L.dt), g ? g->ln_gamma : F(L.lng),
                                g ? g->ln_beta : F(L.lng) + H, nullptr, s));
  hipLaunchKernelGGL(xh_dtanh_kernel, dim3(cdiv(big / 4, 256)), dim3(256), 0, s, big / 4, F(L.dt), F(L.t));
  DS_CHECK_LAUNCH();
  for (int b = 0; b < B; ++b)
    DS_PROPAGATE(ds_colsum_accum(DS_F32, S, H, F(L.dt) + (int64_t)b * H, (int64_t)B * H, F(L.dsfw) + (int64_t)b * H, s));
  hipLaunchKernelGGL(xh_dense_din_kernel, dim3(cdiv(H, 4), B), dim3(256), 0, s, B, H, H, F(L.dsfw), w->end_w0 + (int64_t)H * H, F(L.dpick0));
  if (g) {
    hipLaunchKernelGGL(xh_dense_dw_kernel, dim3(cdiv(H, 256), H), dim3(256), 0, s, B, H, H, F(L.pick0), (const float*)nullptr, F(L.dsfw),
                       g->end_w0 + (int64_t)H * H, g->end_b0);
    DS_CHECK_LAUNCH();
    DS_PROPAGATE(gemm_f32(DS_MN_MAJOR, DS_MN_MAJOR, H, H, rows, xf, H, F(L.dt), H, g->end_w0, H, DS_EPI_ACCUM, s));
  }
  float* dxe = nullptr;
  if (dx) {
    dxe = dtype == DS_F32 ? (float*)dx : F(L.y);
    DS_PROPAGATE(gemm_f32(DS_K_MAJOR, DS_K_MAJOR, rows, H, H, F(L.dt), H, w->end_w0, H, dxe, H, 0, s));
  }
  // ---- everything that lands on x
  if (dtype == DS_BF16)
    hipLaunchKernelGGL((xh_final_kernel<bf16, RPB>), dim3(cdiv(rows, RPB)), dim3(256), 0, s, S, B, H, xf, dxe, F(L.dsl), F(L.p), w->start_w,
                       F(L.dcat), F(L.dpick0), start_positions, cls_index, (bf16*)dx, g ? g->start_w : nullptr, g ? g->start_b : nullptr);
  else
    hipLaunchKernelGGL((xh_final_kernel<float, RPB>), dim3(cdiv(rows, RPB)), dim3(256), 0, s, S, B, H, xf, dxe, F(L.dsl), F(L.p), w->start_w,
                       F(L.dcat), F(L.dpick0), start_positions, cls_index, (float*)dx, g ? g->start_w : nullptr, g ? g->start_b : nullptr);
  DS_CHECK_LAUNCH();
  return DS_OK;
}
