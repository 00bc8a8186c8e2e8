// Grouped launches (group.hip): one kernel launch that carries several independent tasks of a stage - GEMMs, the fused
// attention kernels, LayerNorm rows of the fp32 residual stream - each described as the arguments of the entry point
// that would launch it alone.
#pragma once
#include <string.h>

#include "common.h"

enum {
  GOP_GEMM = 0,   // ds_gemm (bf16, k % 64 == 0, operand majors (K, MN), (K, K) or (MN, MN))
  GOP_ATTN_FWD,   // ds_attention_fwd
  GOP_ATTN_DQ,    // the dQ half of ds_attention_bwd (writes delta unless it is null)
  GOP_ATTN_DKV,   // the dK / dV half of ds_attention_bwd (reads delta)
  GOP_LN_FWD,     // ds_layernorm_fwd_mixed
  GOP_LN_BWD,     // ds_layernorm_bwd_mixed without parameter gradients (one wave per row)
};

struct GroupOp {
  int kind = GOP_GEMM;
  int prio = 0;         // wave priority of the task's workgroups (0..3)
  // GOP_GEMM
  ds_gemm_desc gemm;
  int cfg = -1;         // tile shape (0 = 256x256, 1 = 256x128, 2 = 128x128, 3 = 128x64, 4 / 5 = 2 / 3 with two tile buffers); < 0: chosen here
  // with rowdot: rowdot[((row / rowdot_seq) * (n / 64) + col / 64) * rowdot_seq + row % rowdot_seq] = sum over the 64 columns
  // of a column block of bf16(C[row][col]) * c2[row][col] (c2 bf16, layout of C; no other epilogue that reads c2)
  float* rowdot = nullptr;
  int rowdot_seq = 0;
  // with colsum (256x128 tiles, operand majors (MN, MN), batch == batch_inner): colsum[z * colsum_stride + col] += sum over
  // k of B(col, k) for batch entry z - the bias gradient beside the weight gradient X^T dY that reads the same dY
  float* colsum = nullptr;
  int64_t colsum_stride = 0;
  // GOP_ATTN_*: arguments of ds_attention_fwd / ds_attention_bwd (bf16, head size 64)
  int B = 0, N = 0, S = 0;
  const void* qkv = nullptr;
  int64_t ld = 0;
  const float* key_mask = nullptr;
  float scale = 0.f, mask_value = 0.f;
  void* ctx = nullptr;
  float* lse = nullptr;
  const void* dctx = nullptr;
  void* dqkv = nullptr;
  float* delta = nullptr;
  const float* key_mean = nullptr;  // GOP_ATTN_DQ, nullable: ds_attention_bwd_centered
  // GOP_LN_*: arguments of ds_layernorm_fwd_mixed / ds_layernorm_bwd_mixed
  int rows = 0, cols = 0;
  const float* x = nullptr;
  const float* gamma = nullptr;
  const float* beta = nullptr;
  float eps = 0.f;
  void* y16 = nullptr;   // forward: y; backward: dx
  float* y32 = nullptr;  // nullable
  float* stats = nullptr;
  const float* dy = nullptr;
  void* dy16 = nullptr;  // nullable: bf16 copy of dy
  float* dy32 = nullptr;      // nullable: fp32 copy of dy and
  float* row_sums = nullptr;  // the two per-row means (ds_layernorm_bwd_mixed_rows)
  GroupOp() { memset(&gemm, 0, sizeof(gemm)); }
};

constexpr int DS_GROUP_MAX_TASKS = 12;  // (304 bytes of kernel arguments each, 4 KB in all)
// All tasks as one launch; workgroups start in list order.
int ds_group_launch(const GroupOp* ops, int n, hipStream_t stream);
// The tile shape ds_group_launch picks for a GEMM when GroupOp::cfg < 0.
int ds_group_default_cfg(const ds_gemm_desc* d);
