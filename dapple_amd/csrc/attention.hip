// Fused softmax attention for bf16, head size 64 (gfx950 MFMA): forward, and backward as two kernels
// (dQ parallel over queries, dK/dV parallel over keys).  Replaces the score matmul, scale, mask adder,
// softmax and context matmul of bert/models/bert/modeling_slice.py:499-533 and their tf.gradients,
// without materialising the [B, N, S, S] probabilities.
//
// Every kernel keeps the MFMA output "transposed": the tile it produces has the softmax axis (keys in
// forward/dQ, queries in dK/dV) running down the 16 accumulator registers of a lane and the other
// axis across lanes.  Row statistics (max, sum, logsumexp, delta) are then per-lane scalars, and the
// accumulator registers, converted to bf16, ARE the B operand of the next MFMA (k = softmax axis) -
// no shuffle, no LDS round trip.  The matching A operands (V^T, K^T, Q^T, dO^T) are read from
// row-major LDS tiles with ds_read_b64_tr_b16.
//
// q, k, v are column blocks of one [B*S, ld] matrix (the fused QKV projection); head h owns columns
// h*64 .. h*64+63 of each block.
#include "stage.h"
#include "attention_core.h"

using namespace dsattn;

namespace {

__global__ __launch_bounds__(NTHREADS) void attn_fwd_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  ds_wave_prio(a.prio);
  attn_fwd_body(a, lds, blockIdx.x + gridDim.x * blockIdx.y);
}
__global__ __launch_bounds__(NTHREADS) void attn_bwd_dq_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  ds_wave_prio(a.prio);
  attn_bwd_dq_body(a, lds, blockIdx.x + gridDim.x * blockIdx.y);
}
__global__ __launch_bounds__(NTHREADS) void attn_bwd_dkv_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  ds_wave_prio(a.prio);
  attn_bwd_dkv_body(a, lds, blockIdx.x + gridDim.x * blockIdx.y);
}

int check(const char* who, int dtype, int B, int N, int S, int D) {
  DS_CHECK_ARG(dtype == DS_BF16, "%s: the fused kernels are bf16 only (dtype %d)", who, dtype);
  DS_CHECK_ARG(D == HD, "%s: head size must be %d (got %d)", who, HD, D);
  DS_CHECK_ARG(B > 0 && N > 0 && S > 0 && S % 64 == 0, "%s: seq (%d) must be a positive multiple of 64", who, S);
  DS_CHECK_ARG(S <= 2048, "%s: seq %d exceeds 2048", who, S);
  DS_CHECK_ARG((int64_t)B * N <= 65535, "%s: batch * heads = %lld exceeds the 65535 a launch grid holds", who, (long long)B * N);
  return DS_OK;
}

}  // namespace

extern "C" int ds_attention_fwd(int dtype, int batch, int heads, int seq, int head_dim, const void* qkv, int64_t ld,
                                const float* key_mask, float scale, float mask_value, void* ctx, float* lse, void* stream) {
  DS_PROPAGATE(check("ds_attention_fwd", dtype, batch, heads, seq, head_dim));
  DS_CHECK_ARG(qkv && ctx && lse, "ds_attention_fwd: null pointer");
  DS_CHECK_ARG(ld >= 3 * heads * head_dim && ld % 8 == 0 && ds_aligned16(qkv) && ds_aligned16(ctx), "ds_attention_fwd: bad ld or alignment");
  AttnArgs a;
  a.qkv = (const bf16*)qkv; a.ld = ld; a.key_mask = key_mask; a.ctx = (bf16*)ctx; a.lse = lse; a.dctx = nullptr; a.dqkv = nullptr;
  a.delta = nullptr; a.B = batch; a.N = heads; a.S = seq; a.H = heads * head_dim; a.scale = scale; a.mask_value = mask_value;
  a.prio = ds_launch_prio; a.kbar = nullptr;
  static std::atomic<bool> attr(false);  // two threads may both set the (idempotent) attribute; neither launches before it is set
  if (!attr) {
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)attn_fwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(2048, 2)));
    attr = true;
  }
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, "attn_fwd_kernel", 4.0 * batch * heads * (double)seq * seq * head_dim, "FLOP");
  hipLaunchKernelGGL(attn_fwd_kernel, dim3(seq / 64, batch * heads), dim3(NTHREADS), lds_bytes(seq, key_mask ? 1 : 0), s, a);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

extern "C" int ds_attention_bwd(int dtype, int batch, int heads, int seq, int head_dim, const void* qkv, int64_t ld,
                                const float* key_mask, float scale, float mask_value, const void* ctx, const float* lse,
                                const void* dctx, void* dqkv, float* delta, void* stream) {
  return ds_attention_bwd_centered(dtype, batch, heads, seq, head_dim, qkv, ld, key_mask, scale, mask_value, ctx, lse, dctx, dqkv, delta,
                                   nullptr, stream);
}

extern "C" int ds_attention_key_mean(int dtype, int batch, int heads, int seq, int head_dim, const void* qkv, int64_t ld, float* key_mean,
                                     void* stream) {
  DS_PROPAGATE(check("ds_attention_key_mean", dtype, batch, heads, seq, head_dim));
  DS_CHECK_ARG(qkv && key_mean && ld >= 3 * heads * head_dim && ld % 8 == 0 && ds_aligned16(qkv) && ds_aligned16(key_mean),
               "ds_attention_key_mean: null pointer, bad ld or alignment");
  const int H = heads * head_dim;
  return ds_sample_colsum(batch, seq, H, (const bf16*)qkv + H, ld, 1.0f / seq, key_mean, stream);
}

extern "C" int ds_attention_bwd_centered(int dtype, int batch, int heads, int seq, int head_dim, const void* qkv, int64_t ld,
                                         const float* key_mask, float scale, float mask_value, const void* ctx, const float* lse,
                                         const void* dctx, void* dqkv, float* delta, const float* key_mean, void* stream) {
  DS_PROPAGATE(check("ds_attention_bwd", dtype, batch, heads, seq, head_dim));
  DS_CHECK_ARG(ds_aligned16(key_mean), "ds_attention_bwd: key_mean must be 16-byte aligned");
  DS_CHECK_ARG(qkv && ctx && lse && dctx && dqkv && delta, "ds_attention_bwd: null pointer");
  DS_CHECK_ARG(ld >= 3 * heads * head_dim && ld % 8 == 0 && ds_aligned16(qkv) && ds_aligned16(ctx) && ds_aligned16(dctx) &&
               ds_aligned16(dqkv), "ds_attention_bwd: bad ld or alignment");
  AttnArgs a;
  a.qkv = (const bf16*)qkv; a.ld = ld; a.key_mask = key_mask; a.ctx = (bf16*)ctx; a.lse = (float*)lse; a.dctx = (const bf16*)dctx;
  a.dqkv = (bf16*)dqkv; a.delta = delta; a.B = batch; a.N = heads; a.S = seq; a.H = heads * head_dim; a.scale = scale;
  a.mask_value = mask_value; a.prio = ds_launch_prio; a.kbar = key_mean;
  static std::atomic<bool> attr(false);  // two threads may both set the (idempotent) attribute; neither launches before it is set
  if (!attr) {
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)attn_bwd_dq_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(2048, 2)));
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)attn_bwd_dkv_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(2048, 2)));
    attr = true;
  }
  hipStream_t s = (hipStream_t)stream;
  {
    ds_prof_scope prof(s, "attn_bwd_dq_kernel", 6.0 * batch * heads * (double)seq * seq * head_dim, "FLOP");
    hipLaunchKernelGGL(attn_bwd_dq_kernel, dim3(seq / 64, batch * heads), dim3(NTHREADS), lds_bytes(seq, key_mask ? 1 : 0), s, a);
    DS_CHECK_LAUNCH();
  }
  {
    ds_prof_scope prof(s, "attn_bwd_dkv_kernel", 8.0 * batch * heads * (double)seq * seq * head_dim, "FLOP");
    hipLaunchKernelGGL(attn_bwd_dkv_kernel, dim3(seq / 64, batch * heads), dim3(NTHREADS), lds_bytes(seq, 2), s, a);
    DS_CHECK_LAUNCH();
  }
  return DS_OK;
}
