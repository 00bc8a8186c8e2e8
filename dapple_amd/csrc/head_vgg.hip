// Classification block and loss of the last VGG19 stage, vgg19/applications/vgg19_slice_model.py:217-220 (flatten, fc1,
// fc2: Dense 4096 + ReLU; predictions: Dense classes + softmax) and :342-356 (the loss).  fp32, as the VGG stages are.
//
// The reference calls K.categorical_crossentropy(x, label) with the arguments swapped: keras' signature is
// (target, output), so the softmax output x [batch, classes] is taken as the TARGET and the label column [batch, 1]
// (a float, vgg19/tf-keras-dapple.py:57-63) as the OUTPUT.  The keras TensorFlow backend then computes
//     output = label / reduce_sum(label, -1)          -> 1 for a non-zero label, 0/0 = NaN for label 0
//     output = clip_by_value(output, 1e-7, 1 - 1e-7)
//     score  = -reduce_sum(x * log(output), -1)       -> -log(1 - 1e-7) * sum_c x[c]
// and the loss is reduce_mean(score): a constant of about 1.2e-7 (fp32: 1 - 1e-7 rounds to 1 - 2^-23) whose gradient with
// respect to x is the same number for every class, i.e. zero behind the softmax up to rounding.  DS_VGG_LOSS_AS_WRITTEN
// evaluates exactly that expression, gradient included; DS_VGG_LOSS_SPARSE_CE is the loss the call was presumably meant
// to be (label = class index, score = -log x[label]) and is what trains the block.
// The products are ds_gemm calls (the dense layers are weight-streaming at batch 32: fc1 reads 411 MB of kernel); the only
// kernel of its own is the row kernel that turns logits into probabilities, loss terms and d logits.
#include <math.h>
#include <string.h>

#include "common.h"

namespace {

__global__ void vgg_head_clear_kernel(float* loss) { *loss = 0.f; }

// one block per row: softmax over the classes, the row's loss term, d logits (in place over the logits)
__global__ __launch_bounds__(256) void vgg_softmax_loss_kernel(int classes, float* __restrict__ z, const float* __restrict__ labels,
                                                               int mode, float scale, float* __restrict__ probs,
                                                               float* __restrict__ loss) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  float* zr = z + (int64_t)row * classes;
  float mx = -INFINITY;
  for (int c = threadIdx.x; c < classes; c += 256) mx = fmaxf(mx, zr[c]);
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float sum = 0.f;
  for (int c = threadIdx.x; c < classes; c += 256) sum += expf(zr[c] - mx);
  sum = wave_sum(sum);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
  __syncthreads();
  sum = red[0] + red[1] + red[2] + red[3];
  __syncthreads();
  const float inv = 1.0f / sum;
  const float label = labels[row];
  if (mode == DS_VGG_LOSS_SPARSE_CE) {
    const int t = (int)label;
    const bool valid = label == (float)t && t >= 0 && t < classes;
    for (int c = threadIdx.x; c < classes; c += 256) {
      const float p = expf(zr[c] - mx) * inv;
      probs[(int64_t)row * classes + c] = p;
      if (c == t || (!valid && c == 0)) atomicAdd(loss, valid ? -scale * (zr[c] - mx - logf(sum)) : NAN);
      zr[c] = scale * (p - (c == t ? 1.f : 0.f));
    }
  } else {
    // the expression of the reference's graph, term by term
    float out = label / label;                             // output /= reduce_sum(output, axis, True)
    out = fminf(fmaxf(out, 1e-7f), 1.0f - 1e-7f);          // clip_by_value (min / max of a NaN stay NaN below)
    if (label != label || label == 0.f || isinf(label)) out = NAN;
    const float g = -logf(out);                            // d score / d x[c], the same for every class
    float psum = 0.f;
    for (int c = threadIdx.x; c < classes; c += 256) {
      const float p = expf(zr[c] - mx) * inv;
      probs[(int64_t)row * classes + c] = p;
      psum += p;
    }
    psum = wave_sum(psum);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = psum;
    __syncthreads();
    psum = red[0] + red[1] + red[2] + red[3];
    if (threadIdx.x == 0) atomicAdd(loss, scale * g * psum);   // -sum_c x[c] log(output)
    // softmax backward of a constant upstream gradient: x[c] * (g - sum_j g x[j])
    for (int c = threadIdx.x; c < classes; c += 256) zr[c] = scale * probs[(int64_t)row * classes + c] * (g - g * psum);
  }
}

}  // namespace

extern "C" size_t ds_vgg_head_workspace_bytes(int batch, int fc, int classes) {
  if (batch <= 0 || fc <= 0 || classes <= 0) return 0;
  // h1, h2, dh1, dh2 [batch, fc]; logits / d logits [batch, classes]
  return ((size_t)4 * batch * fc + (size_t)batch * classes) * sizeof(float) + 256;
}

extern "C" int ds_vgg_head(int batch, int features, int fc, int classes, const float* x, const float* fc1_w, const float* fc1_b,
                           const float* fc2_w, const float* fc2_b, const float* pred_w, const float* pred_b, const float* labels,
                           int loss_mode, float loss_scale, float* loss, float* probs, float* dx, float* d_fc1_w, float* d_fc1_b,
                           float* d_fc2_w, float* d_fc2_b, float* d_pred_w, float* d_pred_b, void* workspace, size_t workspace_bytes,
                           void* stream) {
  DS_CHECK_ARG(batch > 0 && features > 0 && fc > 0 && classes > 0, "ds_vgg_head: non-positive shape");
  DS_CHECK_ARG(features % 4 == 0 && fc % 4 == 0 && classes % 4 == 0,
               "ds_vgg_head: features (%d), fc (%d) and classes (%d) must be multiples of 4", features, fc, classes);
  DS_CHECK_ARG(loss_mode == DS_VGG_LOSS_AS_WRITTEN || loss_mode == DS_VGG_LOSS_SPARSE_CE, "ds_vgg_head: loss_mode %d", loss_mode);
  DS_CHECK_ARG(x && fc1_w && fc1_b && fc2_w && fc2_b && pred_w && pred_b && labels && loss && probs && workspace,
               "ds_vgg_head: null pointer");
  const bool grads = d_fc1_w || d_fc1_b || d_fc2_w || d_fc2_b || d_pred_w || d_pred_b;
  DS_CHECK_ARG(!grads || (d_fc1_w && d_fc1_b && d_fc2_w && d_fc2_b && d_pred_w && d_pred_b),
               "ds_vgg_head: the six weight gradients come together or not at all");
  DS_CHECK_ARG(workspace_bytes >= ds_vgg_head_workspace_bytes(batch, fc, classes), "ds_vgg_head: workspace of %zu bytes, %zu needed",
               workspace_bytes, ds_vgg_head_workspace_bytes(batch, fc, classes));
  DS_CHECK_ARG(ds_aligned16(x) && ds_aligned16(fc1_w) && ds_aligned16(fc2_w) && ds_aligned16(pred_w) && ds_aligned16(probs) &&
               ds_aligned16(dx) && ds_aligned16(d_fc1_w) && ds_aligned16(d_fc2_w) && ds_aligned16(d_pred_w) && ds_aligned16(workspace),
               "ds_vgg_head: tensors must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  float* h1 = (float*)workspace;
  float* h2 = h1 + (size_t)batch * fc;
  float* dh1 = h2 + (size_t)batch * fc;
  float* dh2 = dh1 + (size_t)batch * fc;
  float* z = dh2 + (size_t)batch * fc;
  ds_gemm_desc d;
  auto dense = [&](const float* in, int k, const float* w, const float* b, int n, float* out, int flags) {
    memset(&d, 0, sizeof(d));
    d.dtype = DS_F32; d.batch = 1; d.batch_inner = 1; d.alpha = 1.f;
    d.a_major = DS_K_MAJOR; d.b_major = DS_MN_MAJOR; d.m = batch; d.n = n; d.k = k; d.lda = k; d.ldb = n; d.ldc = n;
    d.a = in; d.b = w; d.c = out; d.bias = b; d.flags = DS_EPI_BIAS | flags;
    return ds_gemm(&d, s);
  };
  DS_PROPAGATE(dense(x, features, fc1_w, fc1_b, fc, h1, DS_EPI_RELU));
  DS_PROPAGATE(dense(h1, fc, fc2_w, fc2_b, fc, h2, DS_EPI_RELU));
  DS_PROPAGATE(dense(h2, fc, pred_w, pred_b, classes, z, 0));
  hipLaunchKernelGGL(vgg_head_clear_kernel, dim3(1), dim3(1), 0, s, loss);
  {
    ds_prof_scope prof(s, "vgg_softmax_loss_kernel", (double)batch * classes * 4 * 3, "B");
    hipLaunchKernelGGL(vgg_softmax_loss_kernel, dim3(batch), dim3(256), 0, s, classes, z, labels, loss_mode, loss_scale / (float)batch,
                       probs, loss);
  }
  DS_CHECK_LAUNCH();
  if (!dx && !grads) return DS_OK;
  // backward: z now holds d logits
  auto dgrad = [&](const float* dy, int k, const float* w, int n, float* out, const float* relu_of) {  // out = dy W^T (masked)
    memset(&d, 0, sizeof(d));
    d.dtype = DS_F32; d.batch = 1; d.batch_inner = 1; d.alpha = 1.f;
    d.a_major = DS_K_MAJOR; d.b_major = DS_K_MAJOR; d.m = batch; d.n = n; d.k = k; d.lda = k; d.ldb = k; d.ldc = n;
    d.a = dy; d.b = w; d.c = out;
    if (relu_of) { d.flags = DS_EPI_MASK; d.c2 = (void*)relu_of; }
    return ds_gemm(&d, s);
  };
  auto wgrad = [&](const float* in, int k_in, const float* dy, int n, float* dw, float* db) {          // dw += in^T dy, db += colsum
    memset(&d, 0, sizeof(d));
    d.dtype = DS_F32; d.batch = 1; d.batch_inner = 1; d.alpha = 1.f;
    d.a_major = DS_MN_MAJOR; d.b_major = DS_MN_MAJOR; d.m = k_in; d.n = n; d.k = batch; d.lda = k_in; d.ldb = n; d.ldc = n;
    d.a = in; d.b = dy; d.c = dw; d.flags = DS_EPI_ACCUM;
    DS_PROPAGATE(ds_gemm(&d, s));
    return ds_colsum_accum(DS_F32, batch, n, dy, n, db, s);
  };
  if (grads) DS_PROPAGATE(wgrad(h2, fc, z, classes, d_pred_w, d_pred_b));
  DS_PROPAGATE(dgrad(z, classes, pred_w, fc, dh2, h2));
  if (grads) DS_PROPAGATE(wgrad(h1, fc, dh2, fc, d_fc2_w, d_fc2_b));
  DS_PROPAGATE(dgrad(dh2, fc, fc2_w, fc, dh1, h1));
  if (grads) DS_PROPAGATE(wgrad(x, features, dh1, fc, d_fc1_w, d_fc1_b));
  if (dx) DS_PROPAGATE(dgrad(dh1, fc, fc1_w, features, dx, nullptr));
  return DS_OK;
}
