// Last-stage head of the BERT SQuAD model, bert/models/bert/bert.py:669-718 (build_output_layer_squad):
//   logits = X W^T + b  with W [2, hidden] ("cls/squad/output_weights"), transposed to start / end logits
//   [batch, seq]; loss = (CE(start_logits, start_positions) + CE(end_logits, end_positions)) / 2 with
//   CE = -mean_batch(log_softmax(logits)[position]) (compute_loss :699-705, one_hot outside [0, seq) is all
//   zero), and its gradient: dX for the stage's backward pass, dW / db added into the master gradients.
// Everything here is HBM-bound row work: X is read twice (logits, dW) and dX written once.
#include <math.h>

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

}  // namespace

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
