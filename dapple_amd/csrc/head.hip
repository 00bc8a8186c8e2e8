// Last-stage head of the BERT SQuAD model, bert/models/bert/bert.py:669-718 (build_output_layer_squad):
//   logits = X W^T + b  with W [2, hidden] ("cls/squad/output_weights"), transposed to start / end logits
//   [batch, seq]; loss = (CE(start_logits, start_positions) + CE(end_logits, end_positions)) / 2 with
//   CE = -mean_batch(log_softmax(logits)[position]) (compute_loss :699-705, one_hot outside [0, seq) is all
//   zero), and its gradient: dX for the stage's backward pass, dW / db added into the master gradients.
// Everything here is HBM-bound row work: X is read twice (logits, dW) and dX written once.
#include <math.h>
#include <string.h>

#include "common.h"

namespace {

// one wave per row: logits[row][c] = x[row] . w[c] + b[c]
template <typename T>
__global__ __launch_bounds__(256) void squad_logits_kernel(int rows, int H, const T* __restrict__ x, const float* __restrict__ w,
                                                           const float* __restrict__ bias, float* __restrict__ logits,
                                                           float* __restrict__ loss) {
  if (blockIdx.x == 0 && threadIdx.x == 0) *loss = 0.f;  // the loss kernel that follows adds into it
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  constexpr int VEC = Vec16<T>::N;
  typedef typename Vec16<T>::type V;
  float a0 = 0.f, a1 = 0.f;
  for (int c = lane * VEC; c < H; c += 64 * VEC) {
    const V xv = *reinterpret_cast<const V*>(x + (int64_t)row * H + c);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float xe = to_f32(xv[j]);
      a0 += xe * w[c + j];
      a1 += xe * w[H + c + j];
    }
  }
  a0 = wave_sum(a0);
  a1 = wave_sum(a1);
  if (lane == 0) {
    logits[(int64_t)row * 2] = a0 + bias[0];
    logits[(int64_t)row * 2 + 1] = a1 + bias[1];
  }
}

// one block per (batch entry, c): log-softmax over the sequence, loss term, dlogits
__global__ __launch_bounds__(256) void squad_loss_kernel(int B, int S, const float* __restrict__ logits, const int32_t* __restrict__ start,
                                                         const int32_t* __restrict__ end, float scale, float* __restrict__ loss,
                                                         float* __restrict__ dlogits) {
  __shared__ float red[4];
  const int b = blockIdx.x >> 1, c = blockIdx.x & 1;
  const int pos = c == 0 ? start[b] : end[b];
  const float* lg = logits + (int64_t)b * S * 2 + c;
  float mx = -INFINITY;
  for (int s = threadIdx.x; s < S; s += 256) mx = fmaxf(mx, lg[(int64_t)s * 2]);
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float sum = 0.f;
  for (int s = threadIdx.x; s < S; s += 256) sum += expf(lg[(int64_t)s * 2] - mx);
  sum = wave_sum(sum);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
  __syncthreads();
  sum = red[0] + red[1] + red[2] + red[3];
  const float lse = mx + logf(sum);
  const float wgt = scale / (2.f * (float)B);   // mean over the batch, average of the two losses
  const bool valid = pos >= 0 && pos < S;  // tf.one_hot of anything else is an all-zero row: no loss term, no gradient
  for (int s = threadIdx.x; s < S; s += 256) {
    const float p = expf(lg[(int64_t)s * 2] - lse);
    dlogits[((int64_t)b * S + s) * 2 + c] = valid ? (p - (s == pos ? 1.f : 0.f)) * wgt : 0.f;
  }
  if (threadIdx.x == 0 && valid) atomicAdd(loss, -(lg[(int64_t)pos * 2] - lse) * wgt);
}

// block = RPB rows: dx[row] = dl[row][0] w[0] + dl[row][1] w[1];  dw[c] += sum_rows dl[row][c] x[row];  db[c] += sum dl[row][c]
template <typename T, int RPB>
__global__ __launch_bounds__(256) void squad_bwd_kernel(int rows, int H, const T* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ dl, T* __restrict__ dx, float* __restrict__ dw,
                                                        float* __restrict__ db) {
  const int r0 = blockIdx.x * RPB;
  const int r1 = r0 + RPB < rows ? r0 + RPB : rows;
  for (int c = threadIdx.x; c < H; c += 256) {
    const float w0 = w[c], w1 = w[H + c];
    float g0 = 0.f, g1 = 0.f;
    for (int r = r0; r < r1; ++r) {
      const float d0 = dl[(int64_t)r * 2], d1 = dl[(int64_t)r * 2 + 1];
      if (dx) dx[(int64_t)r * H + c] = from_f32<T>(d0 * w0 + d1 * w1);
      if (dw) {
        const float xe = to_f32(x[(int64_t)r * H + c]);
        g0 += d0 * xe;
        g1 += d1 * xe;
      }
    }
    if (dw) { atomicAdd(dw + c, g0); atomicAdd(dw + H + c, g1); }
  }
  if (db && threadIdx.x < 2) {
    float s = 0.f;
    for (int r = r0; r < r1; ++r) s += dl[(int64_t)r * 2 + threadIdx.x];
    atomicAdd(db + threadIdx.x, s);
  }
}

template <typename T>
int squad_head_t(int B, int S, int H, const void* x, const float* w, const float* bias, const int32_t* start, const int32_t* end,
                 float loss_scale, float* loss, float* logits, float* dlogits, void* dx, float* dw, float* db, hipStream_t s) {
  const int rows = B * S;
  {
    ds_prof_scope prof(s, "squad_logits_kernel", (double)rows * H * sizeof(T), "B");
    hipLaunchKernelGGL(squad_logits_kernel<T>, dim3((rows + 3) / 4), dim3(256), 0, s, rows, H, (const T*)x, w, bias, logits, loss);
    DS_CHECK_LAUNCH();
  }
  hipLaunchKernelGGL(squad_loss_kernel, dim3(2 * B), dim3(256), 0, s, B, S, logits, start, end, loss_scale, loss, dlogits);
  DS_CHECK_LAUNCH();
  if (dx || dw || db) {
    constexpr int RPB = 8;
    ds_prof_scope prof(s, "squad_bwd_kernel", (double)rows * H * sizeof(T) * ((dx ? 1 : 0) + (dw ? 1 : 0)), "B");
    hipLaunchKernelGGL((squad_bwd_kernel<T, RPB>), dim3((rows + RPB - 1) / RPB), dim3(256), 0, s, rows, H, (const T*)x, w, dlogits, (T*)dx,
                       dw, db);
    DS_CHECK_LAUNCH();
  }
  return DS_OK;
}

// ------------------------------------------------------------------ pooler + classification head
// modeling_slice.py:849-868 (pooler_stage: tanh dense on the first token) and bert.py:642-664
// (build_output_layer_classification: FC to the labels, mean sparse softmax cross entropy plus the l2
// regulariser of the FC weights).  The batch is a handful of rows: plain one-thread-per-output kernels.

__global__ void head_clear_kernel(float* loss) { *loss = 0.f; }

// one block: logits, loss = scale * (mean CE + l2_scale * sum(Wfc^2) / 2), dlogits = d loss / d logits
__global__ __launch_bounds__(256) void classifier_loss_kernel(int B, int H, int C, const float* __restrict__ pooled,
                                                              const float* __restrict__ wfc, const float* __restrict__ bfc,
                                                              const int32_t* __restrict__ labels, const float* __restrict__ targets,
                                                              float l2_scale, float scale,
                                                              float* __restrict__ logits, float* __restrict__ dlogits,
                                                              float* __restrict__ loss) {
  __shared__ float red[4];
  __shared__ float lg[64];
  for (int o = 0; o < B * C; ++o) {  // B*C dot products over H, the block cooperating on each
    const int b = o / C, c = o % C;
    float a = 0.f;
    for (int j = threadIdx.x; j < H; j += 256) a += pooled[(int64_t)b * H + j] * wfc[(int64_t)j * C + c];
    a = wave_sum(a);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
      const float v = red[0] + red[1] + red[2] + red[3] + bfc[c];
      logits[o] = v;
      if (o < 64) lg[o] = v;
    }
    __syncthreads();
  }
  float sq = 0.f;
  for (int i = threadIdx.x; i < H * C; i += 256) sq += wfc[i] * wfc[i];
  sq = wave_sum(sq);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sq;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = l2_scale * 0.5f * (red[0] + red[1] + red[2] + red[3]);
    if (targets) {
      // regression (bert.py:627-631, C = 1): the prediction is [B, 1] and the labels placeholder is [B]
      // (bert_finetune.py:212), so `prediction - labels` broadcasts to [B, B] and reduce_mean runs over every pair:
      // loss = sum_i sum_j (z_i - y_j)^2 / B^2, d loss / d z_i = 2 (z_i - mean(y)) / B
      float ysum = 0.f;
      for (int j = 0; j < B; ++j) ysum += targets[j];
      for (int i = 0; i < B; ++i) {
        float acc = 0.f;
        for (int j = 0; j < B; ++j) { const float d = logits[i] - targets[j]; acc += d * d; }
        total += acc / ((float)B * (float)B);
        dlogits[i] = 2.f * (logits[i] - ysum / (float)B) * scale / (float)B;
      }
      *loss = total * scale;
      return;
    }
    for (int b = 0; b < B; ++b) {
      const float* l = logits + (int64_t)b * C;
      float mx = l[0];
      for (int c = 1; c < C; ++c) mx = fmaxf(mx, l[c]);
      float sum = 0.f;
      for (int c = 0; c < C; ++c) sum += expf(l[c] - mx);
      const float lse = mx + logf(sum);
      const int y = labels[b];
      const bool ok = y >= 0 && y < C;  // a label outside the classes has no defined loss: NaN, as on TF's GPU kernel
      total += ok ? -(l[y] - lse) / (float)B : NAN;
      for (int c = 0; c < C; ++c)
        dlogits[(int64_t)b * C + c] = ok ? (expf(l[c] - lse) - (c == y ? 1.f : 0.f)) * scale / (float)B : NAN;
    }
    *loss = total * scale;
  }
}

// dWfc[j][c] += sum_b pooled[b][j] dlogits[b][c] + scale*l2_scale*Wfc[j][c]; dbfc[c] += sum_b dlogits[b][c];
// dz[b][j] = (sum_c dlogits[b][c] Wfc[j][c]) * (1 - pooled[b][j]^2)
__global__ __launch_bounds__(256) void classifier_bwd_kernel(int B, int H, int C, const float* __restrict__ pooled,
                                                             const float* __restrict__ wfc, const float* __restrict__ dlogits,
                                                             float l2_scale, float scale, float* __restrict__ dwfc,
                                                             float* __restrict__ dbfc, float* __restrict__ dz) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j < C && dbfc) {
    float s = 0.f;
    for (int b = 0; b < B; ++b) s += dlogits[(int64_t)b * C + j];
    dbfc[j] += s;
  }
  if (j >= H) return;
  for (int c = 0; c < C && dwfc; ++c) {
    float s = scale * l2_scale * wfc[(int64_t)j * C + c];
    for (int b = 0; b < B; ++b) s += pooled[(int64_t)b * H + j] * dlogits[(int64_t)b * C + c];
    dwfc[(int64_t)j * C + c] += s;
  }
  for (int b = 0; b < B; ++b) {
    float dp = 0.f;
    for (int c = 0; c < C; ++c) dp += dlogits[(int64_t)b * C + c] * wfc[(int64_t)j * C + c];
    const float p = pooled[(int64_t)b * H + j];
    dz[(int64_t)b * H + j] = dp * (1.f - p * p);
  }
}

// dWp[i][j] += sum_b x[b, token 0][i] dz[b][j]; dbp[j] += sum_b dz[b][j]
template <typename T>
__global__ __launch_bounds__(256) void pooler_wgrad_kernel(int B, int S, int H, const T* __restrict__ x, const float* __restrict__ dz,
                                                           float* __restrict__ dwp, float* __restrict__ dbp) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)H * H) return;
  const int i = (int)(idx / H), j = (int)(idx % H);
  float s = 0.f;
  for (int b = 0; b < B; ++b) s += to_f32(x[(int64_t)b * S * H + i]) * dz[(int64_t)b * H + j];
  dwp[idx] += s;
  if (i == 0) {
    float t = 0.f;
    for (int b = 0; b < B; ++b) t += dz[(int64_t)b * H + j];
    dbp[j] += t;
  }
}

// dx[b, token 0][i] = sum_j dz[b][j] Wp[i][j] (one wave per (b, i): a row of Wp); every other token gets no gradient
// from this head (zero_rows_kernel)
template <typename T>
__global__ __launch_bounds__(256) void pooler_dgrad_kernel(int B, int S, int H, const float* __restrict__ dz, const float* __restrict__ wp,
                                                           T* __restrict__ dx) {
  const int lane = threadIdx.x & 63, o = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (o >= B * H) return;
  const int b = o / H, i = o % H;
  float v = 0.f;
  for (int j = lane; j < H; j += 64) v += dz[(int64_t)b * H + j] * wp[(int64_t)i * H + j];
  v = wave_sum(v);
  if (lane == 0) dx[(int64_t)b * S * H + i] = from_f32<T>(v);
}
template <typename T>
__global__ __launch_bounds__(256) void zero_rows_kernel(int64_t total, int S, int H, T* __restrict__ dx) {
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256)
    if ((idx / H) % S != 0) dx[idx] = from_f32<T>(0.f);
}

template <typename T>
int classifier_head_t(int B, int S, int H, int C, const void* x, const float* wp, const float* bp, const float* wfc, const float* bfc,
                      const int32_t* labels, const float* targets, float l2_scale, float scale, float* loss, float* pooled, float* logits,
                      float* dlogits, float* dz, void* dx, float* dwp, float* dbp, float* dwfc, float* dbfc, hipStream_t s) {
  // pooled[b][j] = tanh(x[b, token 0] . Wp[:, j] + bp[j])
  hipLaunchKernelGGL(head_clear_kernel, dim3(1), dim3(1), 0, s, loss);
  hipLaunchKernelGGL((ds_small_dense_kernel<T, 1>), dim3((H + 63) / 64, B), dim3(1024), 0, s, H, 0, H, (const T*)x, (int64_t)S * H,
                     (const float*)nullptr, (int64_t)0, wp, bp, pooled);
  DS_CHECK_LAUNCH();
  hipLaunchKernelGGL(classifier_loss_kernel, dim3(1), dim3(256), 0, s, B, H, C, pooled, wfc, bfc, labels, targets, l2_scale, scale, logits,
                     dlogits, loss);
  DS_CHECK_LAUNCH();
  if (!dx && !dwp) return DS_OK;
  hipLaunchKernelGGL(classifier_bwd_kernel, dim3(((H > C ? H : C) + 255) / 256), dim3(256), 0, s, B, H, C, pooled, wfc, dlogits,
                     l2_scale, scale, dwfc, dbfc, dz);
  DS_CHECK_LAUNCH();
  if (dwp) {
    hipLaunchKernelGGL(pooler_wgrad_kernel<T>, dim3((unsigned)(((int64_t)H * H + 255) / 256)), dim3(256), 0, s, B, S, H, (const T*)x,
                       dz, dwp, dbp);
    DS_CHECK_LAUNCH();
  }
  if (dx) {
    const int64_t total = (int64_t)B * S * H;
    hipLaunchKernelGGL(zero_rows_kernel<T>, dim3((unsigned)((total + 255) / 256 > 8192 ? 8192 : (total + 255) / 256)), dim3(256), 0, s,
                       total, S, H, (T*)dx);
    hipLaunchKernelGGL(pooler_dgrad_kernel<T>, dim3((B * H + 3) / 4), dim3(256), 0, s, B, S, H, dz, wp, (T*)dx);
    DS_CHECK_LAUNCH();
  }
  return DS_OK;
}

}  // namespace

// ------------------------------------------------------------------ GNMT output projection + loss
// gnmt/nmt/model.py:685-686 (logits = output_layer(rnn_output), a Dense without bias, :497-499) and _compute_loss
// :824-838: crossent = sparse softmax cross entropy per (step, sample), weighted by sequence_mask(target length),
// summed and divided by the batch size.  The two products with the [units, vocab] kernel are ds_gemm calls; this
// kernel turns a row of logits into its loss term and, in place, into d loss / d logits.
// One block per row r = t*B + b.  Rows past the target length get a zero gradient row and no loss term.
__global__ __launch_bounds__(256) void nmt_xent_kernel(int B, int T, int V, float* __restrict__ logits, const int32_t* __restrict__ target,
                                                       const int32_t* __restrict__ lengths, float wgt, float* __restrict__ loss) {
  __shared__ float red[4];
  const int r = blockIdx.x, t = r / B, b = r % B;
  float* lg = logits + (int64_t)r * V;
  if (t >= lengths[b]) {
    for (int v = threadIdx.x; v < V; v += 256) lg[v] = 0.f;
    return;
  }
  float mx = -INFINITY;
  for (int v = threadIdx.x; v < V; v += 256) mx = fmaxf(mx, lg[v]);
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float sum = 0.f;
  for (int v = threadIdx.x; v < V; v += 256) sum += expf(lg[v] - mx);
  sum = wave_sum(sum);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
  __syncthreads();
  sum = red[0] + red[1] + red[2] + red[3];
  const float lse = mx + logf(sum);
  const int label = target[(int64_t)b * T + t];
  const bool valid = label >= 0 && label < V;
  if (threadIdx.x == 0) atomicAdd(loss, valid ? wgt * (lse - lg[label]) : NAN);
  __syncthreads();  // the label's logit is read before the row is overwritten
  for (int v = threadIdx.x; v < V; v += 256) lg[v] = wgt * (expf(lg[v] - lse) - (v == label ? 1.f : 0.f));
}

__global__ void nmt_clear_kernel(float* loss) { *loss = 0.f; }

extern "C" int ds_classifier_head(int dtype, int batch, int seq, int hidden, int num_labels, const void* x, const float* pooler_w,
                                  const float* pooler_b, const float* fc_w, const float* fc_b, const int32_t* labels, float l2_scale,
                                  float loss_scale, float* loss, float* pooled, float* logits, float* dlogits, float* dz, void* dx,
                                  float* d_pooler_w, float* d_pooler_b, float* d_fc_w, float* d_fc_b, void* stream) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "ds_classifier_head: dtype %d", dtype);
  DS_CHECK_ARG(batch > 0 && seq > 0 && hidden > 0, "ds_classifier_head: non-positive shape");
  DS_CHECK_ARG(num_labels >= 1 && batch * num_labels <= 64, "ds_classifier_head: batch * num_labels (%d) must be at most 64",
               batch * num_labels);
  DS_CHECK_ARG(x && pooler_w && pooler_b && fc_w && fc_b && labels && loss && pooled && logits && dlogits && dz,
               "ds_classifier_head: null pointer");
  const bool wg = d_pooler_w || d_pooler_b || d_fc_w || d_fc_b;
  DS_CHECK_ARG(!wg || (d_pooler_w && d_pooler_b && d_fc_w && d_fc_b), "ds_classifier_head: pass all four weight gradients or none");
  if (dtype == DS_BF16)
    return classifier_head_t<bf16>(batch, seq, hidden, num_labels, x, pooler_w, pooler_b, fc_w, fc_b, labels, nullptr, l2_scale, loss_scale,
                                   loss, pooled, logits, dlogits, dz, dx, d_pooler_w, d_pooler_b, d_fc_w, d_fc_b, (hipStream_t)stream);
  return classifier_head_t<float>(batch, seq, hidden, num_labels, x, pooler_w, pooler_b, fc_w, fc_b, labels, nullptr, l2_scale, loss_scale,
                                  loss, pooled, logits, dlogits, dz, dx, d_pooler_w, d_pooler_b, d_fc_w, d_fc_b, (hipStream_t)stream);
}

extern "C" int ds_pooler(int dtype, int batch, int seq, int hidden, const void* x, const float* pooler_w, const float* pooler_b,
                         float* pooled, void* stream) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "ds_pooler: dtype %d", dtype);
  DS_CHECK_ARG(batch > 0 && seq > 0 && hidden > 0 && batch <= 65535, "ds_pooler: bad shape (%d, %d, %d)", batch, seq, hidden);
  DS_CHECK_ARG(x && pooler_w && pooler_b && pooled, "ds_pooler: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DS_BF16)
    hipLaunchKernelGGL((ds_small_dense_kernel<bf16, 1>), dim3((hidden + 63) / 64, batch), dim3(1024), 0, s, hidden, 0, hidden, (const bf16*)x,
                       (int64_t)seq * hidden, (const float*)nullptr, (int64_t)0, pooler_w, pooler_b, pooled);
  else
    hipLaunchKernelGGL((ds_small_dense_kernel<float, 1>), dim3((hidden + 63) / 64, batch), dim3(1024), 0, s, hidden, 0, hidden, (const float*)x,
                       (int64_t)seq * hidden, (const float*)nullptr, (int64_t)0, pooler_w, pooler_b, pooled);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_regression_head(int dtype, int batch, int seq, int hidden, const void* x, const float* pooler_w, const float* pooler_b,
                                  const float* fc_w, const float* fc_b, const float* targets, float l2_scale, float loss_scale,
                                  float* loss, float* pooled, float* prediction, float* dprediction, float* dz, void* dx,
                                  float* d_pooler_w, float* d_pooler_b, float* d_fc_w, float* d_fc_b, void* stream) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "ds_regression_head: dtype %d", dtype);
  DS_CHECK_ARG(batch > 0 && seq > 0 && hidden > 0, "ds_regression_head: non-positive shape");
  DS_CHECK_ARG(batch <= 64, "ds_regression_head: batch (%d) must be at most 64", batch);
  DS_CHECK_ARG(x && pooler_w && pooler_b && fc_w && fc_b && targets && loss && pooled && prediction && dprediction && dz,
               "ds_regression_head: null pointer");
  const bool wg = d_pooler_w || d_pooler_b || d_fc_w || d_fc_b;
  DS_CHECK_ARG(!wg || (d_pooler_w && d_pooler_b && d_fc_w && d_fc_b), "ds_regression_head: pass all four weight gradients or none");
  if (dtype == DS_BF16)
    return classifier_head_t<bf16>(batch, seq, hidden, 1, x, pooler_w, pooler_b, fc_w, fc_b, nullptr, targets, l2_scale, loss_scale, loss,
                                   pooled, prediction, dprediction, dz, dx, d_pooler_w, d_pooler_b, d_fc_w, d_fc_b, (hipStream_t)stream);
  return classifier_head_t<float>(batch, seq, hidden, 1, x, pooler_w, pooler_b, fc_w, fc_b, nullptr, targets, l2_scale, loss_scale, loss,
                                  pooled, prediction, dprediction, dz, dx, d_pooler_w, d_pooler_b, d_fc_w, d_fc_b, (hipStream_t)stream);
}

extern "C" int ds_squad_head(int dtype, int batch, int seq, int hidden, const void* x, const float* w, const float* bias,
                             const int32_t* start_positions, const int32_t* end_positions, float loss_scale, float* loss,
                             float* logits, float* dlogits, void* dx, float* dw, float* dbias, void* stream) {
  DS_CHECK_ARG(dtype == DS_F32 || dtype == DS_BF16, "ds_squad_head: dtype %d", dtype);
  DS_CHECK_ARG(batch > 0 && seq > 0 && hidden > 0, "ds_squad_head: non-positive shape");
  DS_CHECK_ARG(hidden % (dtype == DS_BF16 ? 8 : 4) == 0, "ds_squad_head: hidden %d must be a multiple of %d", hidden, dtype == DS_BF16 ? 8 : 4);
  DS_CHECK_ARG(x && w && bias && start_positions && end_positions && loss && logits && dlogits, "ds_squad_head: null pointer");
  DS_CHECK_ARG(ds_aligned16(x) && ds_aligned16(dx), "ds_squad_head: x / dx must be 16-byte aligned");
  if (dtype == DS_BF16)
    return squad_head_t<bf16>(batch, seq, hidden, x, w, bias, start_positions, end_positions, loss_scale, loss, logits, dlogits, dx, dw,
                              dbias, (hipStream_t)stream);
  return squad_head_t<float>(batch, seq, hidden, x, w, bias, start_positions, end_positions, loss_scale, loss, logits, dlogits, dx, dw,
                             dbias, (hipStream_t)stream);
}

extern "C" size_t ds_nmt_loss_head_workspace_bytes(int seq, int batch, int vocab) {
  if (seq <= 0 || batch <= 0 || vocab <= 0) return 0;
  return (size_t)seq * batch * vocab * sizeof(float);
}

extern "C" int ds_nmt_loss_head(int seq, int batch, int units, int vocab, const float* x, const float* proj_kernel,
                                const int32_t* target_output, const int32_t* target_sequence_length, int loss_batch_size,
                                float loss_scale, float* loss, float* dx, float* d_proj_kernel, void* workspace,
                                size_t workspace_bytes, void* stream) {
  DS_CHECK_ARG(seq > 0 && batch > 0 && units > 0 && vocab > 0, "ds_nmt_loss_head: non-positive shape");
  DS_CHECK_ARG(units % 4 == 0 && vocab % 4 == 0, "ds_nmt_loss_head: units (%d) and vocab (%d) must be multiples of 4", units, vocab);
  DS_CHECK_ARG(x && proj_kernel && target_output && target_sequence_length && loss && workspace, "ds_nmt_loss_head: null pointer");
  DS_CHECK_ARG(workspace_bytes >= ds_nmt_loss_head_workspace_bytes(seq, batch, vocab), "ds_nmt_loss_head: workspace of %zu bytes, %zu needed",
               workspace_bytes, ds_nmt_loss_head_workspace_bytes(seq, batch, vocab));
  DS_CHECK_ARG(ds_aligned16(x) && ds_aligned16(proj_kernel) && ds_aligned16(workspace) && ds_aligned16(dx) && ds_aligned16(d_proj_kernel),
               "ds_nmt_loss_head: tensors must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int R = seq * batch;
  float* logits = (float*)workspace;
  ds_gemm_desc d;
  memset(&d, 0, sizeof(d));
  d.dtype = DS_F32; d.batch = 1; d.batch_inner = 1; d.alpha = 1.f;
  d.a_major = DS_K_MAJOR; d.b_major = DS_MN_MAJOR; d.m = R; d.n = vocab; d.k = units; d.lda = units; d.ldb = vocab; d.ldc = vocab;
  d.a = x; d.b = proj_kernel; d.c = logits;
  DS_PROPAGATE(ds_gemm(&d, s));
  hipLaunchKernelGGL(nmt_clear_kernel, dim3(1), dim3(1), 0, s, loss);
  {
    ds_prof_scope prof(s, "nmt_xent_kernel", (double)R * vocab * 4 * 4, "B");
    hipLaunchKernelGGL(nmt_xent_kernel, dim3(R), dim3(256), 0, s, batch, seq, vocab, logits, target_output, target_sequence_length,
                       loss_scale / (float)(loss_batch_size > 0 ? loss_batch_size : batch), loss);
  }
  DS_CHECK_LAUNCH();
  if (dx) {  // d loss / d rnn_output = dlogits W^T
    d.a_major = DS_K_MAJOR; d.b_major = DS_K_MAJOR; d.m = R; d.n = units; d.k = vocab; d.lda = vocab; d.ldb = vocab; d.ldc = units;
    d.a = logits; d.b = proj_kernel; d.c = dx; d.flags = 0;
    DS_PROPAGATE(ds_gemm(&d, s));
  }
  if (d_proj_kernel) {  // += rnn_output^T dlogits
    d.a_major = DS_MN_MAJOR; d.b_major = DS_MN_MAJOR; d.m = units; d.n = vocab; d.k = R; d.lda = units; d.ldb = vocab; d.ldc = vocab;
    d.a = x; d.b = logits; d.c = d_proj_kernel; d.flags = DS_EPI_ACCUM;
    DS_PROPAGATE(ds_gemm(&d, s));
  }
  return DS_OK;
}
