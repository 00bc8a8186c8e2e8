// Several independent tasks in ONE launch (bf16, gfx950).
//
// A pipeline stage in steady state holds work that does not depend on each other: the forward pass of micro-batch
// j+1, the backward pass of micro-batch j (bert/graph.py:126-132 of the reference orders them only through control
// dependencies) and weight gradients nothing waits for.  Launched as kernels of their own they are 2-9 GFLOP apiece:
// too few tiles for 256 CUs unless the tiles are small, and small tiles are short of LDS and L2 bandwidth.  Here the
// workgroups of one launch are dealt out over a list of tasks - GEMMs with their own shapes, operand majors and
// epilogues, the fused attention kernels, LayerNorm rows - so that the launch as a whole fills the CUs with large tiles,
// and a step of the stage is one launch per level of its two chains instead of one per operation and chain.
//
// Workgroup v of the launch belongs to the task whose span [first, first + span) holds v.  Spans start at multiples of
// 8: workgroups go to the 8 XCDs round-robin in launch order, so a task's own XCD-aware order (xcd_tile,
// attn_block_map) stays valid.  Tasks are laid out in the order given; the hardware starts workgroups in index order.
#include "group.h"

#include "attention_core.h"
#include "gemm8_core.h"
#include "rows_core.h"

using namespace dsgemm;

namespace {

struct RowArgs {
  int rows, cols;
  const float* x;
  const float* gamma;
  const float* beta;
  float eps;
  bf16* y16;
  float* y32;
  float* stats;
  const float* dy;
  bf16* dy16;
  float* dy32;
  float* rowsums;
};

enum { ROLE_ATTN_FWD = 64, ROLE_ATTN_DQ, ROLE_ATTN_DKV, ROLE_LN_FWD, ROLE_LN_BWD };
#define GROUP_ROLE(cfg, am, bm) ((cfg) * 4 + (am) * 2 + (bm))

struct GroupTask {
  int role;    // GROUP_ROLE(cfg, amaj, bmaj) of a GEMM, or ROLE_*
  int first;   // first workgroup of the task's span (multiple of 8)
  int count;   // workgroups that do work (the rest of the span returns at once)
  int per_z;   // GEMM: workgroups per batch entry = tiles of one output matrix
  int prio;
  int pad;
  union {
    GemmArgs g;
    dsattn::AttnArgs at;
    RowArgs r;
  };
};
struct GroupArgs {
  int n;
  int pad;
  GroupTask t[DS_GROUP_MAX_TASKS];
};
static_assert(sizeof(GroupArgs) <= 4096, "kernel arguments");
static_assert(sizeof(GroupTask) % 4 == 0, "copied word by word");

struct TileCfg { int bm, bn, stages; };
// cfg: 0 = 256x256, 1 = 256x128, 2 = 128x128, 3 = 128x64; 4 and 5: 128x128 and 128x64 with a two-buffer ring (64 / 48 KB: two
// or three workgroups per CU)
constexpr TileCfg tile_cfg(int cfg) {
  return cfg == 0 ? TileCfg{256, 256, 2} : cfg == 1 ? TileCfg{256, 128, 3} : cfg == 2 ? TileCfg{128, 128, 3} : cfg == 3 ? TileCfg{128, 64, 4}
       : cfg == 4 ? TileCfg{128, 128, 2} : TileCfg{128, 64, 2};
}

template <int CFG, int AMAJ, int BMAJ>
__device__ __forceinline__ void run_tile(const GemmArgs& g, char* lds, int bx, int bz) {
  if (CFG == 0) gemm8_tile<256, 256, 2, 4, 1, 2, AMAJ, BMAJ>(g, lds, bx, bz);
  else if (CFG == 1) {
    if (AMAJ == DS_MN_MAJOR && BMAJ == DS_MN_MAJOR && g.colsum != nullptr) gemm8_tile<256, 128, 2, 2, 2, 3, AMAJ, BMAJ, true>(g, lds, bx, bz);
    else gemm8_tile<256, 128, 2, 2, 2, 3, AMAJ, BMAJ>(g, lds, bx, bz);
  }
  else if (CFG == 2) gemm8_tile<128, 128, 2, 2, 2, 3, AMAJ, BMAJ>(g, lds, bx, bz);
  else if (CFG == 3) gemm8_tile<128, 64, 2, 2, 2, 4, AMAJ, BMAJ>(g, lds, bx, bz);
  else if (CFG == 4) gemm8_tile<128, 128, 2, 2, 2, 2, AMAJ, BMAJ>(g, lds, bx, bz);
  else gemm8_tile<128, 64, 2, 2, 2, 2, AMAJ, BMAJ>(g, lds, bx, bz);
}

template <int NG>
__device__ __forceinline__ void run_rows(const RowArgs& r, bool backward, int row, int lane) {
  if (backward) dsrows::layernorm_bwd_mixed_rows_row<NG>(row, lane, r.rows, r.cols, r.dy, r.x, r.gamma, r.stats, r.y16, r.y32, r.dy16, r.dy32, r.rowsums);
  else dsrows::layernorm_fwd_mixed_row<NG>(row, lane, r.rows, r.cols, r.x, r.gamma, r.beta, r.eps, r.y16, r.y32, r.stats);
}

// WIDE: the launch may hold 256-row GEMM tiles and the attention backward kernels (up to 228 VGPRs: one workgroup per
// CU); otherwise only what fits 128 VGPRs (two workgroups per CU when their LDS fits).
template <bool WIDE>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(WIDE ? 2 : 4, WIDE ? 2 : 4))) void group_kernel(GroupArgs ga) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int v = blockIdx.x;
  int i = 0;
#pragma unroll
  for (int j = 1; j < DS_GROUP_MAX_TASKS; ++j)
    if (j < ga.n && v >= ga.t[j].first) i = j;
  // The task is the same for every lane of the workgroup; its fields are moved to scalar registers word by word so that
  // the tile code - whose loads take scalar base addresses - sees uniform values (an indexed read of the argument block
  // is not one the compiler treats as uniform).
  GroupTask t;
  {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(&ga.t[i]);
    uint32_t* dst = reinterpret_cast<uint32_t*>(&t);
#pragma unroll
    for (int k = 0; k < (int)(sizeof(GroupTask) / 4); ++k) dst[k] = __builtin_amdgcn_readfirstlane(src[k]);
  }
  const int w = v - t.first;
  if (w >= t.count) return;
  ds_wave_prio(t.prio);
  const int bx = w % t.per_z, bz = w / t.per_z;
  // the three operand-major pairs a stage launches: forward (K, MN), input gradient (K, K), weight gradient (MN, MN)
#define GROUP_CASE(cfg, am, bm) \
  case GROUP_ROLE(cfg, am, bm): run_tile<cfg, am, bm>(t.g, lds, bx, bz); break;
#define GROUP_CASES(cfg) \
  GROUP_CASE(cfg, DS_K_MAJOR, DS_MN_MAJOR) GROUP_CASE(cfg, DS_K_MAJOR, DS_K_MAJOR) GROUP_CASE(cfg, DS_MN_MAJOR, DS_MN_MAJOR)
  switch (t.role) {
    GROUP_CASES(2)
    GROUP_CASES(3)
    GROUP_CASES(4)
    GROUP_CASES(5)
    case ROLE_ATTN_FWD: dsattn::attn_fwd_body(t.at, lds, w); break;
    case ROLE_LN_FWD:
    case ROLE_LN_BWD: {
      const int row = w * 8 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
      const bool backward = t.role == ROLE_LN_BWD;
      if (t.r.cols <= 512) run_rows<1>(t.r, backward, row, lane);
      else if (t.r.cols <= 1024) run_rows<2>(t.r, backward, row, lane);
      else run_rows<4>(t.r, backward, row, lane);
      break;
    }
    default:
      if (WIDE) {
        switch (t.role) {
          GROUP_CASES(0)
          GROUP_CASES(1)
          case ROLE_ATTN_DQ: dsattn::attn_bwd_dq_body(t.at, lds, w); break;
          case ROLE_ATTN_DKV: dsattn::attn_bwd_dkv_body(t.at, lds, w); break;
          default: break;
        }
      }
      break;
  }
#undef GROUP_CASES
#undef GROUP_CASE
}

int fill_attention(const GroupOp& op, GroupTask& t, size_t* lds) {
  DS_CHECK_ARG(op.B > 0 && op.N > 0 && op.S > 0 && op.S % 64 == 0 && op.S <= 2048, "ds_group_launch: attention needs seq (%d) a multiple of 64, at most 2048",
               op.S);
  const int64_t H = (int64_t)op.N * 64;
  DS_CHECK_ARG(op.qkv && op.ld >= 3 * H && op.ld % 8 == 0 && ds_aligned16(op.qkv), "ds_group_launch: attention: bad qkv, ld or alignment");
  DS_CHECK_ARG((int64_t)op.B * op.N * (op.S / 64) < (1 << 24), "ds_group_launch: attention: too many workgroups");
  dsattn::AttnArgs& a = t.at;
  a.qkv = (const bf16*)op.qkv; a.ld = op.ld; a.key_mask = op.key_mask; a.ctx = (bf16*)op.ctx; a.lse = op.lse;
  a.dctx = (const bf16*)op.dctx; a.dqkv = (bf16*)op.dqkv; a.delta = op.delta; a.kbar = op.key_mean;
  a.B = op.B; a.N = op.N; a.S = op.S; a.H = (int)H; a.scale = op.scale; a.mask_value = op.mask_value; a.prio = op.prio;
  DS_CHECK_ARG(a.ctx && a.lse && ds_aligned16(a.ctx), "ds_group_launch: attention: ctx and lse are needed");
  int vectors = op.key_mask ? 1 : 0;
  if (op.kind == GOP_ATTN_FWD) {
    t.role = ROLE_ATTN_FWD;
  } else {
    DS_CHECK_ARG(a.dctx && a.dqkv && ds_aligned16(a.dctx) && ds_aligned16(a.dqkv), "ds_group_launch: attention backward: dctx and dqkv are needed");
    DS_CHECK_ARG(a.delta != nullptr || op.kind == GOP_ATTN_DQ, "ds_group_launch: attention backward: the dK / dV task reads delta");
    t.role = op.kind == GOP_ATTN_DQ ? ROLE_ATTN_DQ : ROLE_ATTN_DKV;
    if (op.kind == GOP_ATTN_DKV) vectors = 2;
  }
  t.per_z = 1;
  t.count = (op.S / 64) * op.B * op.N;
  *lds = dsattn::lds_bytes(op.S, vectors);
  return DS_OK;
}

int fill_rows(const GroupOp& op, GroupTask& t) {
  DS_CHECK_ARG(op.rows > 0 && op.cols > 0 && op.cols % 8 == 0 && op.cols <= 2048, "ds_group_launch: LayerNorm: cols (%d) must be a multiple of 8, at most 2048",
               op.cols);
  DS_CHECK_ARG(op.x && op.gamma && op.y16 && op.stats, "ds_group_launch: LayerNorm: null argument");
  DS_CHECK_ARG(ds_aligned16(op.x) && ds_aligned16(op.gamma) && ds_aligned16(op.y16) && ds_aligned16(op.y32) && ds_aligned16(op.dy) &&
               ds_aligned16(op.dy16) && ds_aligned16(op.beta) && ds_aligned16(op.dy32), "ds_group_launch: LayerNorm: operands must be 16-byte aligned");
  RowArgs& r = t.r;
  r.rows = op.rows; r.cols = op.cols; r.x = op.x; r.gamma = op.gamma; r.beta = op.beta; r.eps = op.eps; r.y16 = (bf16*)op.y16;
  r.y32 = op.y32; r.stats = op.stats; r.dy = op.dy; r.dy16 = (bf16*)op.dy16; r.dy32 = op.dy32; r.rowsums = op.row_sums;
  if (op.kind == GOP_LN_FWD) {
    DS_CHECK_ARG(op.beta != nullptr, "ds_group_launch: LayerNorm forward: beta is needed");
    t.role = ROLE_LN_FWD;
  } else {
    DS_CHECK_ARG(op.dy != nullptr, "ds_group_launch: LayerNorm backward: dy is needed");
    t.role = ROLE_LN_BWD;
  }
  t.per_z = 1;
  t.count = (op.rows + 7) / 8;
  return DS_OK;
}

}  // namespace

int ds_group_default_cfg(const ds_gemm_desc* d) {
  const int batch = d->batch > 0 ? d->batch : 1;
  auto tiles = [&](int c) { const TileCfg tc = tile_cfg(c); return (int64_t)((d->m + tc.bm - 1) / tc.bm) * ((d->n + tc.bn - 1) / tc.bn) * batch; };
  if (d->flags & DS_EPI_ACCUM) return tiles(1) >= 96 ? 1 : 2;
  if (tiles(2) >= 160) return 2;
  return 3;
}

int ds_group_launch(const GroupOp* ops, int n, hipStream_t stream) {
  DS_CHECK_ARG(ops != nullptr, "ds_group_launch: null argument");
  DS_CHECK_ARG(n >= 1 && n <= DS_GROUP_MAX_TASKS, "ds_group_launch: %d tasks (1..%d)", n, DS_GROUP_MAX_TASKS);
  GroupArgs ga;
  memset(&ga, 0, sizeof(ga));
  ga.n = n;
  int next = 0;
  size_t lds = 0;
  bool wide = false;
  double flop = 0;
  for (int i = 0; i < n; ++i) {
    const GroupOp& op = ops[i];
    GroupTask& t = ga.t[i];
    size_t need = 0;
    if (op.kind == GOP_GEMM) {
      const ds_gemm_desc* d = &op.gemm;
      const int cfg = op.cfg >= 0 ? op.cfg : ds_group_default_cfg(d);
      DS_CHECK_ARG(cfg >= 0 && cfg <= 5, "ds_group_launch: task %d: tile shape %d (0..5)", i, cfg);
      int batch = 1;
      DS_PROPAGATE(ds_gemm_make_args(d, &t.g, &batch));
      DS_CHECK_ARG(d->dtype == DS_BF16, "ds_group_launch: task %d: bf16 operands only", i);
      DS_CHECK_ARG(t.g.vec_epi && d->k % 64 == 0,
                   "ds_group_launch: task %d: needs k %% 64 == 0, n and ldc multiples of 8 and 16-byte aligned outputs", i);
      const bool fwd = d->a_major == DS_K_MAJOR && d->b_major == DS_MN_MAJOR, dgrad = d->a_major == DS_K_MAJOR && d->b_major == DS_K_MAJOR,
                 wgrad = d->a_major == DS_MN_MAJOR && d->b_major == DS_MN_MAJOR;
      DS_CHECK_ARG(fwd || dgrad || wgrad, "ds_group_launch: task %d: operand majors (MN, K) are not built", i);
      const TileCfg tc = tile_cfg(cfg);
      const int ktiles = d->k / 64;
      DS_CHECK_ARG(ktiles > tc.stages, "ds_group_launch: task %d: k = %d is not longer than the tile ring (%d k-tiles of 64)", i, d->k, tc.stages);
      t.g.prio = op.prio;
      t.g.splitk = 1;
      t.g.ktiles_per_split = ktiles;
      t.g.grid_m = (d->m + tc.bm - 1) / tc.bm;
      t.g.grid_n = (d->n + tc.bn - 1) / tc.bn;
      choose_xcd_block(t.g);
      if (op.rowdot) {
        DS_CHECK_ARG(d->n % 64 == 0 && op.rowdot_seq > 0 && d->m % op.rowdot_seq == 0 && d->c2 != nullptr && batch == 1 &&
                     !(d->flags & (DS_EPI_GELU | DS_EPI_DGELU | DS_EPI_MUL | DS_EPI_MASK | DS_EPI_OUT_F32 | DS_EPI_ACCUM)),
                     "ds_group_launch: task %d: the row-dot epilogue needs n %% 64 == 0, whole samples, c2 and a plain bf16 output", i);
        t.g.flags |= DS_EPI_ROWDOT;
        t.g.rowdot = op.rowdot;
        t.g.rowdot_seq = op.rowdot_seq;
      }
      if (op.colsum) {
        DS_CHECK_ARG(cfg == 1 && wgrad && (batch == 1 || batch == (d->batch_inner > 0 ? d->batch_inner : 1)) && ds_aligned16(op.colsum),
                     "ds_group_launch: task %d: column sums need 256x128 tiles, operand majors (MN, MN) and a batch that is all inner", i);
        t.g.colsum = op.colsum;
        t.g.colsum_si = op.colsum_stride;
      }
      t.role = GROUP_ROLE(cfg, d->a_major, d->b_major);
      t.per_z = t.g.grid_m * t.g.grid_n;
      t.count = t.per_z * batch;
      need = (size_t)tc.stages * (tc.bm + tc.bn) * 128;
      wide = wide || cfg <= 1;
      flop += 2.0 * d->m * d->n * d->k * batch;
    } else if (op.kind == GOP_ATTN_FWD || op.kind == GOP_ATTN_DQ || op.kind == GOP_ATTN_DKV) {
      DS_PROPAGATE(fill_attention(op, t, &need));
      wide = wide || op.kind != GOP_ATTN_FWD;
      flop += (op.kind == GOP_ATTN_FWD ? 4.0 : op.kind == GOP_ATTN_DQ ? 6.0 : 8.0) * op.B * op.N * (double)op.S * op.S * 64;
    } else if (op.kind == GOP_LN_FWD || op.kind == GOP_LN_BWD) {
      DS_PROPAGATE(fill_rows(op, t));
    } else {
      ds_set_error("ds_group_launch: task %d: unknown kind %d", i, op.kind);
      return DS_EINVAL;
    }
    t.prio = op.prio;
    t.first = next;
    next += (t.count + 7) & ~7;
    if (need > lds) lds = need;
  }
  static std::atomic<bool> attr_set(false);  // two threads may both set the (idempotent) attribute; neither launches before it is set
  if (!attr_set) {
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)group_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 147456));
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)group_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 98304));
    attr_set = true;
  }
  DS_CHECK_ARG(lds <= (wide ? 147456u : 98304u), "ds_group_launch: %zu bytes of LDS", lds);
  // the timing log names a launch by what it carries
  char tag[192];
  int off = snprintf(tag, sizeof(tag), "group_kernel<%s>", wide ? "wide" : "narrow");
  for (int i = 0; i < n && off < (int)sizeof(tag) - 40; ++i) {
    const GroupOp& op = ops[i];
    if (op.kind == GOP_GEMM)
      off += snprintf(tag + off, sizeof(tag) - off, " %s%dx%dx%d/%d", (op.gemm.flags & DS_EPI_ACCUM) ? "w" : op.gemm.b_major == DS_K_MAJOR ? "d" : "f",
                      op.gemm.m, op.gemm.n, op.gemm.k, ga.t[i].role >> 2);
    else
      off += snprintf(tag + off, sizeof(tag) - off, " %s", op.kind == GOP_ATTN_FWD ? "att" : op.kind == GOP_ATTN_DQ ? "att_dq" : op.kind == GOP_ATTN_DKV ? "att_dkv"
                                                           : op.kind == GOP_LN_FWD ? "ln" : "ln_bwd");
  }
  ds_prof_scope prof(stream, tag, flop, "FLOP");
  if (wide) hipLaunchKernelGGL(group_kernel<true>, dim3(next), dim3(512), lds, stream, ga);
  else hipLaunchKernelGGL(group_kernel<false>, dim3(next), dim3(512), lds, stream, ga);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

// descs[i] with tile shape cfgs[i], i < n <= 8, in one launch (include/dapple_stage.h).
extern "C" int ds_gemm_grouped(const ds_gemm_desc* descs, const int* cfgs, int n, void* stream) {
  DS_CHECK_ARG(descs != nullptr && cfgs != nullptr, "ds_gemm_grouped: null argument");
  DS_CHECK_ARG(n >= 1 && n <= DS_GROUP_MAX_TASKS, "ds_gemm_grouped: %d tasks (1..%d)", n, DS_GROUP_MAX_TASKS);
  GroupOp ops[DS_GROUP_MAX_TASKS];
  for (int i = 0; i < n; ++i) {
    DS_CHECK_ARG(cfgs[i] >= 0 && cfgs[i] <= 5, "ds_gemm_grouped: task %d: tile shape %d (0..5)", i, cfgs[i]);
    ops[i].kind = GOP_GEMM;
    ops[i].gemm = descs[i];
    ops[i].cfg = cfgs[i];
    ops[i].prio = ds_launch_prio;
  }
  return ds_group_launch(ops, n, (hipStream_t)stream);
}
