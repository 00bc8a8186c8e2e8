/*
 * C ABI of libdapple_hip.so: one DAPPLE pipeline stage on one MI355X.
 *
 * The reference (AlibabaPAI/DAPPLE) has no FFI for this path: src/api/capi.rs is
 * empty and its runtime is TF1 graph construction.  Every entry point below
 * therefore cites the reference Python/TF interface it replaces.  All pointers
 * are device pointers unless the comment says "host"; the caller owns every
 * buffer it passes in; the stage handle owns its compute copies of the weights,
 * its workspace and its K-slot activation stash.  Every function returns 0 on
 * success and a negative DS_E* code on failure, never throws, and leaves a
 * message for ds_last_error() (thread-local).  A handle is used from one host
 * thread at a time.  Launches are asynchronous on the given stream.
 */
#ifndef DAPPLE_STAGE_H
#define DAPPLE_STAGE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DS_OK 0
#define DS_EINVAL (-1)  /* bad argument: shape, alignment, null pointer, unknown enum */
#define DS_EHIP (-2)    /* a HIP runtime call failed */
#define DS_ESTATE (-3)  /* call order: slot not forwarded, weights not bound, ... */

/* element types of activations / compute copies */
#define DS_F32 0
#define DS_BF16 1

/* operand storage for ds_gemm: which index is contiguous in memory */
#define DS_K_MAJOR 0  /* reduction index contiguous: A[m][k] / B[n][k] */
#define DS_MN_MAJOR 1 /* free index contiguous:      A[k][m] / B[k][n] */

/* epilogue flags for ds_gemm */
#define DS_EPI_BIAS 1      /* + bias[n] (fp32) */
#define DS_EPI_RESIDUAL 2  /* + residual[m][n] (element type) */
#define DS_EPI_GELU 4      /* C = pre-activation, C2 = gelu_erf(C) */
#define DS_EPI_DGELU 8     /* C = acc * gelu_erf'(aux[m][n]) */
#define DS_EPI_OUT_F32 16  /* C is fp32 even when dtype is bf16 */
#define DS_EPI_ACCUM 32    /* C (fp32) += acc, split-K allowed (atomic) */
#define DS_EPI_RELU 64     /* C = max(acc + bias, 0) */
#define DS_EPI_TANH_FORM 256 /* GELU / DGELU use the tanh approximation (xlnet/activations/gelu.py:6-11) */
#define DS_EPI_MASK 128    /* C = aux[m][n] > 0 ? acc : 0 (ReLU backward), aux = c2 */
#define DS_EPI_GELU_GRAD 512 /* with DS_EPI_GELU: C = gelu'(pre-activation) instead of the pre-activation */
#define DS_EPI_MUL 1024    /* C = acc * aux[m][n], aux = c2 (backward through a GELU whose derivative was kept) */
#define DS_EPI_RESIDUAL_F32 2048 /* with DS_EPI_RESIDUAL: the residual tensor is fp32 whatever dtype is (a bf16 GEMM adding
                                  * into an fp32 residual stream; combine with DS_EPI_OUT_F32 to keep the sum in fp32) */

const char* ds_last_error(void);

/* Version / build probe; returns the gfx target the library was built for ("gfx950"). */
const char* ds_build_target(void);

/* Per-launch timing for roofline reports (no counterpart in the reference, which relied on
 * tf.train.ProfilerHook, bert/utils/hooks/hooks_helper.py:72-88).  While enabled, every kernel
 * launch made through this library is bracketed by HIP events on the stream it is launched on.
 * ds_profile_dump writes "tag<TAB>launches<TAB>total_ms<TAB>total_work<TAB>unit" lines (work =
 * algorithmic FLOP or bytes) into a host buffer and clears the log.  Not thread safe. */
int ds_profile_enable(int on);
int ds_profile_dump(char* buf, size_t cap);

/* ---------------------------------------------------------------------------
 * Gradient accumulation: acc[i] (fp32) += g[i], i < n.
 * Replaces tf.accumulate_n(grad_i_set) at bert/graph.py:159 (and its copies at
 * vgg19/tf-keras-dapple.py:311, gnmt/nmt/model.py:288, xlnet/main_tf_estimator.py:226),
 * applied in place as each micro-batch's backward finishes: a sum, no 1/M.
 * g_dtype is DS_F32 or DS_BF16.  Pointers must be 16-byte aligned. */
int ds_grad_accumulate(void* acc_fp32, const void* g, size_t n, int g_dtype, void* stream);

/* fp32 -> bf16 copy of n elements (compute copies of the fp32 master weights). */
int ds_cast_f32_to_bf16(void* dst_bf16, const void* src_f32, size_t n, void* stream);
int ds_cast_bf16_to_f32(void* dst_f32, const void* src_bf16, size_t n, void* stream);

/* ---------------------------------------------------------------------------
 * GEMM on the matrix cores: C[m][n] (+)= sum_k A(m,k) * B(n,k), optionally batched.
 * Replaces tf.layers.dense (bert/models/bert/modeling_slice.py:464-485, 974-994),
 * tf.matmul (:499, :533) and their tf.gradients.  Batch index z in [0, batch) is
 * split as (z / batch_inner, z % batch_inner) with separate strides, which
 * addresses [B, heads] views of a [B*S, hidden] matrix without copies. */
typedef struct ds_gemm_desc {
  int dtype;            /* DS_F32 or DS_BF16: element type of A, B (and C unless OUT_F32/ACCUM) */
  int a_major, b_major; /* DS_K_MAJOR / DS_MN_MAJOR */
  int m, n, k;
  int64_t lda, ldb, ldc; /* leading dimensions in elements */
  int batch, batch_inner;
  int64_t a_stride_outer, a_stride_inner;
  int64_t b_stride_outer, b_stride_inner;
  int64_t c_stride_outer, c_stride_inner;
  int flags;            /* DS_EPI_* */
  float alpha;          /* acc is scaled by alpha before the epilogue */
  const void* a;
  const void* b;
  void* c;
  const float* bias;    /* [n] fp32, DS_EPI_BIAS */
  const void* residual; /* same layout and strides as C, DS_EPI_RESIDUAL */
  void* c2;             /* DS_EPI_GELU second output / DS_EPI_DGELU aux input, layout of C */
  void* workspace;      /* optional device scratch for split-K (NULL: never split), see ds_gemm_workspace_bytes */
  size_t workspace_bytes;
  /* Segmented reduction (0: none).  For an MN-major operand the k index may run over k / k_segment segments of k_segment
   * rows each: rows inside a segment are lda / ldb apart as usual, segment s starts a_segment_stride / b_segment_stride
   * elements behind segment s - 1 (a stride of 0 reads the same rows for every segment); a K-major operand beside it runs
   * on along its rows and its stride is ignored; at least one operand must be MN-major.  This is how ONE weight-gradient
   * product X^T dY sums over several micro-batches whose activations sit in different stash slots
   * (tf.accumulate_n over the micro-batches, bert/graph.py:145-161).  k_segment must be a multiple of 64 (bf16) or 32 (fp32). */
  int k_segment;
  int64_t a_segment_stride, b_segment_stride;
} ds_gemm_desc;
int ds_gemm(const ds_gemm_desc* d, void* stream);
/* Split-K: when the output has too few tiles to fill the GPU and k is long (bf16, batch 1), ds_gemm may cut k into
 * slices that run as separate workgroups; every slice leaves its fp32 partial tile in `workspace`, and the workgroup
 * that finishes last adds the slices in index order (bit-reproducible) and runs the epilogue.  The workspace must be
 * at least ds_gemm_workspace_bytes(m, n) bytes, 256-byte aligned, zero-filled once before its first use (the library
 * leaves its counters at zero), and must not be shared by GEMMs that can run at the same time. */
size_t ds_gemm_workspace_bytes(int m, int n);
/* ds_gemm cut into k slices with the library's own scratch as the workspace.  No counterpart in the reference: it is
 * for callers that cannot allocate - code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc - and allocates nothing itself.  Same descriptor and results as ds_gemm with a workspace (d->workspace is
 * ignored).  Limits: an output of at most 16 tiles of 128 x 128 (4 MiB + 4 KiB of scratch per GPU, held until the
 * process ends), bf16, batch 1, and a shape that ds_gemm would cut (DS_EINVAL otherwise, with the reason).  All calls
 * on one GPU share the scratch: calls that overlap in time on one GPU race; calls on one stream do not. */
int ds_gemm_static_scratch(const ds_gemm_desc* d, void* stream);
/* Looks up the scratch's device address on the current device (once per device; launches and allocates nothing).
 * ds_gemm_static_scratch does it on its first call; a caller that captures that call into a HIP graph calls this
 * first, outside the capture. */
int ds_gemm_static_scratch_init(void);
/* Several independent GEMMs as ONE launch (bf16, k % 64 == 0, the operand-major pairs (K, MN), (K, K), (MN, MN); at
 * most 8 problems).  What a stage holds in steady state - a forward product of one micro-batch, an input-gradient
 * product of another (the reference's graph orders them only by control dependencies, bert/graph.py:126-132) and
 * weight-gradient products nothing waits for (bert/graph.py:145-161) - is too small per problem to fill the GPU
 * with large tiles; together it is not.  cfgs[i] is the tile shape of problem i: 0 = 256 x 256, 1 = 256 x 128,
 * 2 = 128 x 128, 3 = 128 x 64.  Workgroups start in the order of the list: put what other work waits for first.
 * Results are those of ds_gemm on each descriptor (d->workspace is ignored: no k slicing). */
int ds_gemm_grouped(const ds_gemm_desc* descs, const int* cfgs, int n, void* stream);

/* ---------------------------------------------------------------------------
 * LayerNorm over the last axis, y = (x - mean) * rsqrt(var + eps) * gamma + beta,
 * biased variance.  Replaces layer_norm() at modeling_slice.py:152-155
 * (tf.contrib.layers.layer_norm, eps 1e-12) and xlnet/layers/layer_normalization.py:69-78.
 * stats receives (mean, rstd) per row for the backward pass. */
int ds_layernorm_fwd(int dtype, int rows, int cols, const void* x, const float* gamma,
                     const float* beta, float eps, void* y, float* stats, void* stream);
/* LayerNorm of a bf16 stage that keeps its residual stream in fp32: x (and dy) fp32 in; the result goes out as the bf16
 * copy the next GEMM reads and, when y_f32 / dx_f32 is given, as the fp32 tensor the next residual sum adds to.
 * Arithmetic, stats, parameter gradients and d_colsum as ds_layernorm_fwd / ds_layernorm_bwd.  cols % 8 == 0, <= 2048. */
int ds_layernorm_fwd_mixed(int rows, int cols, const float* x, const float* gamma, const float* beta, float eps,
                           void* y_bf16, float* y_f32, float* stats, void* stream);
int ds_layernorm_bwd_mixed(int rows, int cols, const float* dy, const float* x, const float* gamma, const float* stats,
                           void* dx_bf16, float* dx_f32, void* dy_bf16, float* d_gamma, float* d_beta, float* d_colsum,
                           void* stream);
/* With d_gamma = d_beta = NULL ds_layernorm_bwd_mixed writes dx only (one wave per row, no atomics: the form for the
 * chain of dependent backward kernels) and, when dy_bf16 is given, a bf16 copy of dy.  From that copy, the fp32 x, stats
 * and dx_bf16 ds_layernorm_param_grads_mixed adds the parameter gradients (and, with d_colsum, the column sums of dx)
 * later, over any number of rows stacked back to back - on another stream, beside the chain. */
int ds_layernorm_param_grads_mixed(int rows, int cols, const void* dy_bf16, const float* x, const float* stats,
                                   const void* dx_bf16, float* d_gamma, float* d_beta, float* d_colsum, void* stream);
/* The same split with nothing rounded on the way: ds_layernorm_bwd_mixed_rows writes dx (bf16, and fp32 when dx_f32 is
 * given), an fp32 copy of dy and, per row, the two means of the backward formula (row_sums [rows][2]); from those, x,
 * stats and gamma ds_layernorm_param_grads_exact adds d_gamma, d_beta and (d_colsum given) the column sums of the fp32 dx,
 * which it rebuilds - the sums ds_layernorm_bwd_mixed itself would have formed, up to the order of the additions. */
int ds_layernorm_bwd_mixed_rows(int rows, int cols, const float* dy, const float* x, const float* gamma, const float* stats,
                                void* dx_bf16, float* dx_f32, float* dy_copy, float* row_sums, void* stream);
int ds_layernorm_param_grads_exact(int rows, int cols, const float* dy_copy, const float* x, const float* gamma, const float* stats,
                                   const float* row_sums, float* d_gamma, float* d_beta, float* d_colsum, void* stream);
/* dx = LN backward; d_gamma/d_beta (fp32, [cols]) are accumulated (+=); d_colsum (nullable,
 * fp32 [cols]) += column sums of dx (the bias gradient of the dense layer that fed x);
 * dx_add (nullable) is added to dx before it is written (gradient of a residual branch). */
int ds_layernorm_bwd(int dtype, int rows, int cols, const void* dy, const void* x,
                     const float* gamma, const float* stats, const void* dx_add, void* dx,
                     float* d_gamma, float* d_beta, float* d_colsum, void* stream);
/* The same backward pass split in two, for callers that keep the parameter gradients off their chain of dependent
 * kernels: ds_layernorm_bwd with d_gamma = d_beta = d_colsum = NULL writes dx only (one wave per row, no atomics), and
 * ds_layernorm_param_grads adds d_gamma += sum_rows dy * x_hat, d_beta += sum_rows dy and, when d_colsum is given,
 * d_colsum += sum_rows dx (dx: the first call's output) - on whatever stream it is given. */
int ds_layernorm_param_grads(int dtype, int rows, int cols, const void* dy, const void* x, const float* stats,
                             const void* dx, float* d_gamma, float* d_beta, float* d_colsum, void* stream);

/* ---------------------------------------------------------------------------
 * Softmax over the last axis of fp32 scores [batch*heads*q, k]:
 *   p = softmax(scores * scale + (1 - key_mask[b][j]) * mask_value)
 * Replaces modeling_slice.py:499-518 (scale 1/sqrt(d), mask_value -10000).
 * key_mask is [batch, k] fp32 of 0/1 or NULL. p has element type dtype. */
int ds_softmax_fwd(int dtype, int batch, int heads, int q, int k, const float* scores,
                   float scale, const float* key_mask, float mask_value, void* p, void* stream);
/* ds = scale * p * (dp - sum_j dp*p), dp fp32, ds element type dtype */
int ds_softmax_bwd(int dtype, int64_t rows, int k, const void* p, const float* dp, float scale,
                   void* ds, void* stream);

/* Fused attention for bf16 and head size 64: ctx = softmax(q k^T * scale + (1 - key_mask) * mask_value) v
 * per (batch, head), without materialising the probabilities (modeling_slice.py:499-533 in one kernel).
 * qkv is the fused projection [batch*seq, ld]: q in columns [0,H), k in [H,2H), v in [2H,3H), H = heads*64;
 * head h owns columns h*64..h*64+63 of each.  lse [batch, heads, seq] receives the row logsumexp for the
 * backward pass; ds_attention_bwd writes dq|dk|dv into dqkv (same layout as qkv) and uses delta
 * [batch, heads, seq] as scratch.  seq must be a multiple of 64, at most 2048. */
int ds_attention_fwd(int dtype, int batch, int heads, int seq, int head_dim, const void* qkv, int64_t ld,
                     const float* key_mask, float scale, float mask_value, void* ctx, float* lse,
                     void* stream);
int ds_attention_bwd(int dtype, int batch, int heads, int seq, int head_dim, const void* qkv, int64_t ld,
                     const float* key_mask, float scale, float mask_value, const void* ctx,
                     const float* lse, const void* dctx, void* dqkv, float* delta, void* stream);
/* The same backward pass with the rounding of the score gradients kept out of dq.  Every row of dS = P (dP - delta) sums to
 * zero, so dq = dS k only depends on the keys' deviation from their mean; the kernel multiplies bf16-rounded dS, whose rows
 * no longer sum to zero, and against keys that share a large common part (token vectors that have grown alike over many
 * layers) that residue times the mean key is the bulk of dq's error.  With key_mean ([batch, heads * 64] fp32, from
 * ds_attention_key_mean on the same qkv; NULL = ds_attention_bwd) the kernel subtracts it: dq -= rowsum(rounded dS) * mean.
 * Same arithmetic otherwise (tf.gradients of modeling_slice.py:499-533). */
int ds_attention_key_mean(int dtype, int batch, int heads, int seq, int head_dim, const void* qkv, int64_t ld, float* key_mean,
                          void* stream);
int ds_attention_bwd_centered(int dtype, int batch, int heads, int seq, int head_dim, const void* qkv, int64_t ld,
                              const float* key_mask, float scale, float mask_value, const void* ctx, const float* lse,
                              const void* dctx, void* dqkv, float* delta, const float* key_mean, void* stream);

/* Column sums: out[n] (fp32) += sum_m x[m][n]; the bias gradient of tf.layers.dense. */
int ds_colsum_accum(int dtype, int rows, int cols, const void* x, int64_t ldx, float* out,
                    void* stream);

/* ---------------------------------------------------------------------------
 * Stage handle: the explicit form of what the reference's unrolled graph implies.
 * ds_stage_forward(slot) = stages[k](prev_output) for every k the planner put on this
 * device (bert/models/bert/bert.py:437-456); ds_stage_backward(slot) =
 * tf.gradients(ys, [prev_y] + vars_i, grad_ys) of bert/graph.py:110-123 with the
 * accumulation of :145-161 fused in (master grads are updated in place). */
#define DS_STAGE_BERT 0
#define DS_STAGE_VGG19 1
#define DS_STAGE_GNMT 2
#define DS_STAGE_XLNET 3

typedef struct ds_stage_cfg {
  int kind;        /* DS_STAGE_* */
  int dtype;       /* compute type: DS_F32 or DS_BF16; master weights/grads are always fp32 */
  int num_layers;  /* encoder layers on this stage */
  int hidden, heads, ffn;
  int batch, seq;  /* micro-batch shape; activations are [batch*seq, hidden] */
  int with_embedding; /* 1: the stage starts at token ids (embedding_stage, modeling_slice.py:794) */
  int vocab, type_vocab, max_pos;
  float ln_eps;
  int stash_slots; /* K: in-flight micro-batches (S - i, bert/graph.py:129) */
  int first_layer; /* index of this stage's first encoder layer in the whole model (names only) */
  int wgrad_group; /* G: weight gradients of G consecutive backward passes are formed by ONE GEMM per weight
                    * (contraction over the G micro-batches' rows, one fp32 read-modify-write of the master
                    * gradient instead of G); 0 or 1: every backward pass accumulates its own.  The sum over
                    * micro-batches is the one tf.accumulate_n forms (bert/graph.py:159).  With G > 1 the
                    * handle keeps K+G stash positions and a 2G-deep ring of the upstream-gradient operands,
                    * and the master gradients are complete only after ds_stage_join / ds_stage_sync. */
  int residual_fp32; /* bf16 stages: 1 keeps the residual stream (the sums in front of both LayerNorms, the LayerNorm
                      * outputs that feed the next sum, and the same chain of gradients in backward) in fp32 and rounds
                      * to bf16 only what a GEMM or the attention kernels read: the reference computes all of it in fp32
                      * (bert/models/bert/modeling_slice.py:942-1001), and the stream's own rounding is what adds up
                      * over 24 layers.  0: every activation is bf16.  Ignored by fp32 stages. */
  int reserved[5];
} ds_stage_cfg;

typedef struct ds_stage ds_stage;

int ds_stage_create(const ds_stage_cfg* cfg, void* stream, ds_stage** out);
int ds_stage_destroy(ds_stage* h);
/* Number of weight tensors and, per tensor, its name (reference variable scope,
 * modeling_slice.py:945-996) and element count. name_buf is host memory. */
int ds_stage_num_weights(const ds_stage* h);
int ds_stage_weight_info(const ds_stage* h, int i, char* name_buf, size_t name_cap, int64_t* numel,
                         int64_t* rows, int64_t* cols);
/* weights[i] / master_grads[i]: fp32 device tensors in ds_stage_weight_info order (host arrays of
 * device pointers).  The handle keeps the pointers; it never frees them. */
int ds_stage_bind_weights(ds_stage* h, int n, const void* const* weights, void* const* master_grads);
/* Refresh the compute copies (bf16 casts, fused QKV packing) after the master weights changed. */
int ds_stage_refresh_weights(ds_stage* h);
/* key_mask: [batch, seq] fp32 0/1 input_mask for this slot's micro-batch, or NULL (all ones). */
int ds_stage_forward(ds_stage* h, int slot, const void* in, const float* key_mask, void* out);
/* token_type_ids [batch, seq] int32 for the micro-batch that will be forwarded into `slot`
 * (segment_ids of bert/models/bert/bert.py:390); NULL or never called: all zeros
 * (modeling_slice.py:785-786).  Only for stages with an embedding. */
int ds_stage_set_token_types(ds_stage* h, int slot, const int32_t* token_type_ids);
/* d_in may be NULL for a first stage (bert/graph.py:121 takes no input gradient there).
 * Ordering of d_out and d_in (the data edges prev_grads -> tf.gradients -> y_grads[0] of bert/graph.py:110-143):
 * on one stream everything follows the stage's stream.  With ds_stage_enable_overlap the pass runs on the handle's
 * backward stream: ds_stage_backward then waits for everything queued on the stage's stream up to the call (whatever
 * produced d_out there - a loss head, the next stage - is honoured, at the price that a forward pass queued before the
 * call also finishes first); ds_stage_backward_after waits only for `ready_event` (a hipEvent_t the caller recorded
 * behind the producer of d_out, on any stream; NULL: d_out is already complete, or was queued before F(slot) on the
 * stage's stream), which keeps a forward pass queued earlier running beside this backward pass.  d_in and the
 * gradients of this pass are ready when the event ds_stage_backward_event returns has completed (NULL on one stream);
 * ds_stage_wait_backward puts `stream` behind it; ds_stage_join does so for the stage's own stream at the end of a step. */
int ds_stage_backward(ds_stage* h, int slot, const void* d_out, void* d_in);
int ds_stage_backward_after(ds_stage* h, int slot, const void* d_out, void* d_in, void* ready_event);
void* ds_stage_backward_event(ds_stage* h, int slot);
int ds_stage_wait_backward(ds_stage* h, int slot, void* stream);
/* The forward pass of one micro-batch into `fslot` and the backward pass of another out of `bslot` as ONE call
 * (arguments of ds_stage_forward and ds_stage_backward).  The reference's graph leaves the two unordered: only the
 * control dependencies of bert/graph.py:126-132 constrain them.  A BERT stage in bf16 with fused attention, the fp32
 * residual stream and wgrad_group > 1 walks both chains together on the stage's stream, one launch per level carrying
 * the next operation of either chain (large tiles for both instead of small ones for each); every other stage runs
 * the two calls one after the other.  d_out must be ordered before the call on the stage's stream; d_in, out and the
 * gradients follow the stage's stream (ds_stage_join / ds_stage_sync at the end of a step, as for separate calls).
 * Results equal those of the separate calls up to the rounding of a different tile order in the GEMMs. */
int ds_stage_forward_backward(ds_stage* h, int fslot, const void* in, const float* key_mask, void* out, int bslot,
                              const void* d_out, void* d_in);
/* Gives up the micro-batch forwarded into `slot` without a backward pass: a forward-only use of the stage (the
 * reference's is_training=False graphs, bert/models/bert/modeling_slice.py:774-776, build no gradients). */
int ds_stage_release_slot(ds_stage* h, int slot);
size_t ds_stage_workspace_bytes(const ds_stage* h);
size_t ds_stage_stash_bytes(const ds_stage* h, int slots);
int ds_stage_sync(ds_stage* h);
/* Forward/backward overlap.  The reference leaves the order of one stage's forward and backward
 * passes of different micro-batches to TensorFlow's inter-op scheduler: only the control
 * dependencies of bert/graph.py:126-132 constrain it (256 inter-op threads,
 * bert/train_flags.py:183-186), so F(j+K) and B(j+1) may run at the same time.
 * ds_stage_enable_overlap(h, 1) puts the backward passes on a second stream owned by the handle and
 * their weight-gradient GEMMs on a third (default priority); per-slot events keep B(slot) after
 * F(slot) and the next F(slot) after B(slot); (h, 0) returns to one stream (no micro-batch may be
 * in flight for either call).
 * ds_stage_join queues the weight-gradient work still deferred (wgrad_group > 1) and orders all queued
 * backward work before what is queued next on the stage's stream (call it at the end of a step, before
 * reading gradients on that stream); ds_stage_sync and
 * ds_stage_refresh_weights join by themselves.  Stages whose forward and backward passes share
 * workspace report 0 from ds_stage_overlap_supported and DS_EINVAL from ds_stage_enable_overlap. */
int ds_stage_overlap_supported(const ds_stage* h);
int ds_stage_enable_overlap(ds_stage* h, int on);
int ds_stage_join(ds_stage* h);

/* ---------------------------------------------------------------------------
 * 3x3, stride 1, 'same' convolution over NHWC fp32 tensors as an implicit GEMM on the matrix cores.
 * Replaces keras Conv2D(C, (3,3), activation='relu', padding='same') of
 * vgg19/applications/vgg19_slice_model.py:137-212 and its tf.gradients.
 *   fwd  : y[n,h,w,co] = epi(sum_{dy,dx,c} x[n,h+dy,w+dx,c] * kernel[dy+1][dx+1][c][co] (+ bias[co]))
 *          flags: DS_EPI_BIAS | DS_EPI_RELU | DS_EPI_MASK (y = mask_src > 0 ? y : 0).  The input
 *          gradient of a convolution is the same call on dz with ds_conv3x3_flip(kernel).
 *   wgrad: dkernel[dy+1][dx+1][c][co] (fp32) += sum_{n,h,w} x[n,h+dy,w+dx,c] * dz[n,h,w,co]
 * cin must be a multiple of 32, cout of 4; wgrad needs n*h*w to be a multiple of 32. */
int ds_conv3x3_fwd(int dtype, int n, int h, int w, int cin, int cout, const void* x,
                   const void* kernel_hwio, const float* bias, int flags, const void* mask_src,
                   void* y, void* stream);
int ds_conv3x3_wgrad(int dtype, int n, int h, int w, int cin, int cout, const void* x,
                     const void* dz, float* dkernel_hwio, void* stream);
/* flipped[8 - tap][co][c] = kernel[tap][c][co]: the kernel of the transposed convolution */
int ds_conv3x3_flip(int cin, int cout, const float* kernel_hwio, float* flipped, void* stream);
/* keras MaxPooling2D((2,2), strides=(2,2)) (vgg19_slice_model.py:145) on NHWC fp32; backward sends
 * the gradient to the first maximum of each window, optionally masked by x > 0 (fused ReLU'). */
int ds_maxpool2x2_fwd(int n, int h, int w, int c, const float* x, float* y, void* stream);
int ds_maxpool2x2_bwd(int n, int h, int w, int c, const float* x, const float* dy, float* dx,
                      int relu_mask, void* stream);

/* VGG19 stage 0 (vgg19_slice_model.py:274-309): ops[i] > 0 is a conv3x3 + bias + ReLU with that many
 * output channels, ops[i] == 0 a 2x2 max-pool.  Weights are named block%d_conv%d/{kernel,bias}
 * (HWIO kernels flattened to [9*cin, cout]).  The handle works with every ds_stage_* call. */
typedef struct ds_vgg_cfg {
  int dtype;  /* DS_F32 */
  int batch, height, width, in_channels;
  int num_ops;
  int ops[40];
  int stash_slots;     /* K = 2S-1-i for this model (vgg19/tf-keras-dapple.py:292) */
  int need_input_grad; /* 0 for a first stage fed with images */
  int reserved[8];
} ds_vgg_cfg;
int ds_vgg_stage_create(const ds_vgg_cfg* cfg, void* stream, ds_stage** out);
/* Copies the stashed output of op `op` (a conv's post-ReLU activation, a pool's output; NHWC fp32) of the micro-batch
 * forwarded into `slot` to dst (device memory, dst_elems = its element count), in the order of the stage's stream: the
 * per-layer outputs a keras model exposes (vgg19/applications/vgg19_slice_model.py:135-213 names every layer). */
int ds_vgg_stage_read_activation(ds_stage* h, int slot, int op, float* dst, size_t dst_elems);

/* GNMT encoder stage (gnmt/nmt/gnmt_model.py:61-221, DAPPLE branch): embedding lookup, one
 * bidirectional BasicLSTMCell layer, then num_layers-1 uni-directional layers, residual from the
 * third layer on (model_helper.py:445-448); ids [batch, seq] int32 in, [seq, batch, units] out
 * (time-major like the reference).  Kernels are TF's [in+units, 4*units] with gate order i, j, f, o.
 * Sequences are full length unless ds_gnmt_stage_set_lengths says otherwise.  The handle works with every
 * ds_stage_* call; it takes no input gradient. */
typedef struct ds_gnmt_cfg {
  int dtype;       /* DS_F32 */
  int num_layers;  /* encoder layers incl. the bidirectional one (8 for GNMT-16's encoder) */
  int units, vocab, batch, seq;
  float forget_bias; /* 1.0 in gnmt/nmt/standard_hparams/wmt16_gnmt_8_layer.json */
  int stash_slots;
  int part;          /* DS_GNMT_ENCODER (0): the encoder stage above; DS_GNMT_DECODER_PART2; DS_GNMT_ATTENTION_CELL (below) */
  int first_layer;   /* DS_GNMT_DECODER_PART2: index of the first decoder cell held (1 in the reference, gnmt_model.py:346-364) */
  int src_seq;       /* DS_GNMT_ATTENTION_CELL: source steps of the memory (seq = target steps) */
  int reserved[5];
} ds_gnmt_cfg;
enum { DS_GNMT_ENCODER = 0, DS_GNMT_DECODER_PART2 = 1, DS_GNMT_ATTENTION_CELL = 2 };
int ds_gnmt_stage_create(const ds_gnmt_cfg* cfg, void* stream, ds_stage** out);
/* iterator.source_sequence_length (gnmt_model.py:103, 223-227) of the micro-batch that will be forwarded
 * into `slot`: lengths [batch] int32 on the device, or NULL for full length.  Every layer's dynamic_rnn
 * gets it: steps t >= lengths[b] emit zeros (residual layers too) and keep the state, the backward
 * direction of the first layer starts at step lengths[b] - 1.  The setting stays with the slot. */
int ds_gnmt_stage_set_lengths(ds_stage* h, int slot, const int32_t* lengths);
/* One time step of BasicLSTMCell (gnmt/nmt/model_helper.py:418-420; TensorFlow's cell: one kernel applied to
 * concat([x, h]), gates split as i, j, f, o) without the matrix product, for unit parity of the stage's cell kernels.
 *   fwd: gates fp32 [batch, 4*units] holds the pre-activations (bias included) and is overwritten with sigmoid(i),
 *        tanh(j), sigmoid(f + forget_bias), sigmoid(o); c = c_prev * f + i * j (c_prev NULL: zero state);
 *        h = tanh(c) * o; with x_residual and y (ResidualWrapper, :445-448) y = h + x_residual.
 *   bwd: gates_act / c / c_prev as the forward step left them; dh fp32 [batch, units] = gradient reaching h at this
 *        step (output plus recurrent); dc in: the cell-state gradient from the step after (ignored when first != 0),
 *        out: dc * f for the step before; dgates fp32 [batch, 4*units] out: gradients of the pre-activations. */
int ds_lstm_cell_fwd(int batch, int units, float forget_bias, float* gates, const float* c_prev, float* c, float* h,
                     const float* x_residual, float* y, void* stream);
int ds_lstm_cell_bwd(int batch, int units, const float* gates_act, const float* c, const float* c_prev, const float* dh, float* dc,
                     int first, float* dgates, void* stream);
/* part = DS_GNMT_DECODER_PART2: decoder cells first_layer .. first_layer + num_layers - 1 as the reference's second device runs
 * them - GNMTAttentionMultiCell_2, gnmt/nmt/gnmt_model.py:489-537, under dynamic_decode with a TrainingHelper on the
 * outputs of cell 0 (gnmt/nmt/model.py:641-656): a scan over all `seq` padded target steps from the zero state
 * (:375).  in / out / d_out / d_in are fp32 [seq, batch, units]; vocab is unused.  Cell l has one kernel
 * [3*units, 4*units] (rows: running input | attention | h; gate order i, j, f, o) and a bias [4*units], and for
 * l >= 2 adds the running input to its output (gnmt_residual_fn :587-613).
 * The attention every cell concatenates to its input (:518, :526) comes from a non-trainable variable in the
 * reference (:456-459), i.e. it is a constant of the graph: here it is a per-slot side input [seq, batch, units]
 * on the device that receives no gradient; NULL (the default) stands for zeros, the variable's initial value. */
int ds_gnmt_stage_set_attention(ds_stage* h, int slot, const float* attention);
/* part = DS_GNMT_ATTENTION_CELL: decoder cell 0 under the attention wrapper, which the reference keeps on the FIRST
 * device behind the encoder (GNMTAttentionMultiCell_1, gnmt/nmt/gnmt_model.py:440-487; built at :309-325, :366-374 as
 * AttentionWrapper(BasicLSTMCell, BahdanauAttention(normalize=True, memory_sequence_length=source_sequence_length),
 * attention_layer_size=None, output_attention=False); driven by dynamic_decode with a TrainingHelper on the embedded
 * target_input, gnmt/nmt/model.py:622-640).  The stage input `in` is the memory = the encoder stage's output, fp32
 * [src_seq, batch, units]; `out` = outputs_1.rnn_output, fp32 [seq, batch, units]; d_in = d loss / d memory (feed it
 * to the encoder stage's backward pass).  Weights, in ds_stage_weight_info order: embedding_decoder [vocab, units],
 * the cell's kernel [3*units, 4*units] (rows: embedded input | previous attention | h) and bias, memory_layer/kernel,
 * query_layer/kernel [units, units], attention_v [units], attention_g [1], attention_b [units].
 * ds_gnmt_stage_set_decoder_inputs gives the slot its side inputs before the forward pass: target_input int32
 * [batch, seq]; source_sequence_length int32 [batch] (NULL = src_seq; every length must be >= 1, an empty source gives
 * NaN in TensorFlow and zeros here); attention_out (nullable) fp32 [seq, batch, units] receives every step's attention
 * vector (what the second device's cells concatenate to their input). */
int ds_gnmt_stage_set_decoder_inputs(ds_stage* h, int slot, const int32_t* target_input,
                                     const int32_t* source_sequence_length, float* attention_out);

/* ---- Operators of an AmoebaNet cell (amoeba_net/network_utils_slice.py), fp32, NHWC ([n, h, w, c] = [rows, c] matrices).
 * The cell itself (BaseCell.__call__, :394-428) is composed from these and ds_gemm on the host side (dapple_amd/amoeba.py).
 * `accumulate` != 0: the result is added to what the output holds (a tensor that feeds several operations collects their
 * gradients). */
/* tf.nn.relu (:321, :353, ...) and its gradient (dx (+)= dy where x > 0) */
int ds_relu_fwd(int64_t n, const float* x, float* y, void* stream);
int ds_relu_bwd(int64_t n, const float* x, const float* dy, float* dx, int accumulate, void* stream);
/* h = h1 + h2 (:418) */
int ds_add(int64_t n, const float* a, const float* b, float* y, void* stream);
/* dst[r][0..cols) (+)= src[r][0..cols) with row strides ld_src / ld_dst: tf.concat of the unused states along the channels
 * (:553-554) writes each state into its column block; the gradient reads the block back */
int ds_copy2d(int64_t rows, int cols, const float* src, int64_t ld_src, float* dst, int64_t ld_dst, int accumulate, void* stream);
/* batch_norm in training mode (:600-806: tf.nn.fused_batch_norm on the batch's own moments, :765-766): per channel
 * mean and biased variance over the rows, y = (x - mean) rsqrt(var + eps) gamma + beta; save_mean / save_rstd [c] are
 * kept for the backward pass; moving_mean / moving_var (nullable) follow assign_moving_average (:779-790):
 * m -= (1 - decay) (m - value), the variance entering as the unbiased estimate.  workspace: ds_batchnorm_workspace_bytes. */
size_t ds_batchnorm_workspace_bytes(int channels);
int ds_batchnorm_train_fwd(int64_t rows, int channels, const float* x, const float* gamma, const float* beta, float eps, float* y,
                           float* save_mean, float* save_rstd, float* moving_mean, float* moving_var, float decay, void* workspace,
                           void* stream);
/* dx (+)= gamma rstd (dy - mean_r dy - x_hat mean_r(dy x_hat)); d_gamma += sum_r dy x_hat, d_beta += sum_r dy (nullable) */
int ds_batchnorm_train_bwd(int64_t rows, int channels, const float* dy, const float* x, const float* gamma, const float* save_mean,
                           const float* save_rstd, float* dx, int accumulate_dx, float* d_gamma, float* d_beta, void* workspace,
                           void* stream);
/* slim.avg_pool2d / slim.max_pool2d, 3 x 3, stride 1, 'SAME' (_pooling, :262-276): kind 0 averages over the taps inside the
 * image, 1 takes the maximum ('min' pooling is max pooling of -x).  The backward call takes the forward INPUT x. */
int ds_pool3x3_fwd(int kind, int n, int h, int w, int c, const float* x, float* y, void* stream);
int ds_pool3x3_bwd(int kind, int n, int h, int w, int c, const float* x, const float* dy, float* dx, int accumulate, void* stream);
/* The depthwise half of slim.separable_conv2d(..., depth_multiplier=1) (_stacked_separable_conv, :213-238): k x k (k odd),
 * stride 1, 'SAME'; kernel [k, k, c] (TensorFlow's [k, k, c, 1]).  The pointwise half is ds_gemm on [rows, c]. */
int ds_depthwise_conv_fwd(int n, int h, int w, int c, int k, const float* x, const float* kernel, float* y, void* stream);
/* dx (nullable) (+)= input gradient; d_kernel (nullable) += kernel gradient */
int ds_depthwise_conv_bwd(int n, int h, int w, int c, int k, const float* x, const float* kernel, const float* dy, float* dx,
                          int accumulate_dx, float* d_kernel, void* stream);
/* The factorised convolutions slim.conv2d(net, f, [1, k]) / [k, 1] (_apply_conv_operation, :446-459) as GEMMs:
 * col[pixel][t * c + ch] = x at the pixel shifted by t - k/2 along the width (axis 1) or the height (axis 0), zero outside
 * the image, so the convolution is col [pixels, k c] x kernel [k c, f] (the kernel as TensorFlow stores it);
 * ds_scatter1d is the transpose of the gather: dx (+)= the input gradient from d col. */
int ds_gather1d(int n, int h, int w, int c, int k, int axis, const float* x, float* col, void* stream);
int ds_scatter1d(int n, int h, int w, int c, int k, int axis, const float* dcol, float* dx, int accumulate, void* stream);

/* XLNet stage (xlnet/models/slice_xlnet.py:164-180 layer body; xlnet/layers/rel_multihead_attn.py:71-149).
 * Activations are sequence-major like the reference: in/out are [streams][seq][batch][hidden] (stream 0 =
 * content stream h, stream 1 = query stream g).  Per-layer weights, in ds_stage_weight_info order:
 * q, k, v, r, o ([hidden, heads*head_dim]), bias_context, bias_relative, bias_segment ([hidden]),
 * seg_emb ([2, hidden]), attn_ln/{gamma,beta}, ff/{W1,b1,W2,b2}, ff_ln/{gamma,beta}.
 * mem_len > 0 and streams == 2 go beyond what the reference builds (it hard-wires memory length 0 and has
 * the content stream only, lambda_funcs.py:20,36) and follow the XLNet formulation. */
enum { DS_XL_ATTN_AUTO = 0, DS_XL_ATTN_SEPARATE = 1 };
typedef struct ds_xlnet_cfg {
  int dtype;
  int num_layers, hidden, heads, ffn;
  int batch, seq, mem_len, streams;
  float ln_eps;     /* 1e-14 = K.epsilon()**2 (layer_normalization.py:37-39) */
  int first_layer;  /* names only */
  int stash_slots;
  int fused_attention; /* how the attention scores are computed; results agree to rounding:
                          DS_XL_ATTN_AUTO (0): where the shape allows (bf16, head size 64, seq and mem_len + seq multiples
                            of 16, mem_len + seq <= 1024) scores, relative shift and softmax are one kernel forward and one
                            backward, and no fp32 score matrix exists; masks then count as 0 / non-zero.  Other shapes run
                            as DS_XL_ATTN_SEPARATE.
                          DS_XL_ATTN_SEPARATE (1): every product and the softmax as launches of their own, fp32 scores
                            in the workspace. */
  int residual_fp32;   /* bf16 only, 1: the residual stream (the sums in front of both LayerNorms, the LayerNorm outputs that
                          feed the next sum, the same chain of gradients) stays in fp32, bf16 is what the GEMMs read: the
                          stream's own rounding no longer adds up over the layers (as ds_stage_cfg.residual_fp32) */
  int wgrad_group;     /* G > 1 (bf16; rows, klen * batch and klen + seq multiples of 64; otherwise taken as 1): weight gradients
                          are formed once per G backward passes, one product per weight over all G micro-batches (as
                          ds_stage_cfg.wgrad_group: the sum tf.accumulate_n forms happens inside the matrix cores).  Master
                          gradients are complete after ds_stage_join / ds_stage_sync; masks, segments and memories then travel
                          with a micro-batch's stash position: ds_xlnet_stage_set_inputs before every forward pass. */
  int reserved[5];
} ds_xlnet_cfg;
int ds_xlnet_stage_create(const ds_xlnet_cfg* cfg, void* stream, ds_stage** out);

/* Scores and softmax of XLNet's relative attention as operators (xlnet/layers/rel_multihead_attn.py:71-115 with the relative
 * shift of lambda_funcs.py:85-93): what an XLNet stage runs per layer under DS_XL_ATTN_AUTO.  bf16, head size 64; seq and klen
 * multiples of 16, klen <= 1024.  rows = streams * seq stacked query rows (row stream*seq + i is position i).  Layouts:
 *   q, qw, qr, qs [rows][batch][heads*64] the projected queries; q + bias_context / bias_relative / bias_segment
 *   de         fp32 [batch][heads][rows]  qs . (seg_emb[1] - seg_emb[0]) per head: the difference of a row's two segment
 *                                         scores (ds_xlnet_bias_q writes qw, qr, qs and de from q)
 *   kv         [klen][batch][2*heads*64] k at column 0, v at column heads*64 of a row
 *   kr         [klen + seq][heads*64]    projected position embeddings
 *   seg_emb    fp32 [2][heads*64];  p, ds bf16 [batch*heads][rows][klen];  dbd bf16 [batch*heads][rows][klen + seq]
 * forward:  p = softmax_j((qw.k[j] + qr.kr[j + seq - i] + qs.seg_emb[seg(i,j,b)]) * scale - 1e30 * mask(i',j,b)),
 *           evaluated with de * seg(i,j,b) in place of the segment score (a softmax row ignores the common qs.seg_emb[0])
 * backward: dp = dvec v^T, ds = scale * p * (dp - sum_j p dp), dbd[i'][j + seq - i] = ds[i'][j] (only that band is written:
 *           clear dbd once), defs fp32 [batch*heads][rows][2] = the sums of ds over the keys of either segment.
 * ds_xlnet_scores_pack turns masks fp32 [rows][klen][batch] (non-zero = masked; may be NULL) and seg_mat uint8
 * [seq][klen][batch] (may be NULL) into the packed bits both kernels read (meta, ds_xlnet_scores_meta_bytes bytes, 16-byte
 * aligned) and nseg fp32 [batch][seq] (keys of the other segment per row; may be NULL when seg_mat is).  meta = NULL in
 * forward / backward means no mask and one segment. */
size_t ds_xlnet_scores_meta_bytes(int rows, int klen, int batch);
int ds_xlnet_scores_pack(int seq, int rows, int klen, int batch, const float* masks, const uint8_t* seg_mat, void* meta,
                         float* nseg, void* stream);
int ds_xlnet_bias_q(int rows, int batch, int heads, const void* q, const float* bias_context, const float* bias_relative,
                    const float* bias_segment, const float* seg_emb, void* qw, void* qr, void* qs, float* de, void* stream);
int ds_xlnet_scores_fwd(int seq, int rows, int klen, int batch, int heads, const void* qw, const void* qr, const float* de,
                        const void* kv, const void* kr, const void* meta, float scale, void* p, void* stream);
int ds_xlnet_scores_bwd(int seq, int rows, int klen, int batch, int heads, const void* kv, const void* p, const void* dvec,
                        const void* meta, const float* nseg, float scale, void* ds, void* dbd, float* defs, void* stream);

/* Side inputs of the micro-batch that will be forwarded into `slot` (copied into the slot):
 *   masks   [streams][seq][mem_len+seq][batch] fp32, 1 = masked (get_attn_mask, lambda_funcs.py:7-44); NULL = none
 *   seg_mat [seq][mem_len+seq][batch] uint8, 1 = different segment (segment_embed.py:41-52); NULL = all equal
 *   mems    [num_layers][mem_len][batch][hidden] in the compute type; required when mem_len > 0 */
int ds_xlnet_stage_set_inputs(ds_stage* h, int slot, const float* masks, const uint8_t* seg_mat, const void* mems);

/* Last-stage head of the SQuAD model, bert/models/bert/bert.py:669-718 (build_output_layer_squad):
 * logits = X W^T + b with W = cls/squad/output_weights [2, hidden], b = cls/squad/output_bias [2];
 * loss = (CE(start) + CE(end)) / 2, CE = -mean_batch log_softmax(logits over seq)[position] (:699-713); a
 * position outside [0, seq) contributes no loss term, like tf.one_hot.
 *   x [batch*seq, hidden] (compute type): the stage's sequence output; logits, dlogits: fp32 [batch*seq, 2]
 *   (column 0 start, 1 end) out; loss: device float, overwritten with loss_scale * loss;
 *   dx (nullable): d loss / d x in the compute type - the d_out of the stage's backward pass;
 *   dw [2, hidden], dbias [2] (nullable): master gradients, added to (tf.accumulate_n over micro-batches). */
int ds_squad_head(int dtype, int batch, int seq, int hidden, const void* x, const float* w, const float* bias,
                  const int32_t* start_positions, const int32_t* end_positions, float loss_scale, float* loss,
                  float* logits, float* dlogits, void* dx, float* dw, float* dbias, void* stream);

/* Pooler and classification head of the last BERT stage: pooler_stage, bert/models/bert/modeling_slice.py:849-868
 * (pooled = tanh(dense(first token)), kernel bert/pooler/dense/kernel [hidden, hidden]) and
 * build_output_layer_classification, bert/models/bert/bert.py:642-664 (fully_connected to num_labels, weights
 * src-output-layer/FC/weights [hidden, num_labels]; loss = mean sparse softmax cross entropy + the l2 regulariser
 * l2_scale * sum(FC weights^2) / 2, 1e-3 in the reference).
 *   x [batch*seq, hidden] (compute type): the stage's sequence output; labels [batch] int32;
 *   out: loss (device float, loss_scale * loss), pooled [batch, hidden], logits [batch, num_labels],
 *   dlogits [batch, num_labels] fp32; dz [batch, hidden] fp32 scratch;
 *   dx (nullable): d loss / d x, zero except on each sample's first token - the d_out of the stage's backward pass;
 *   d_pooler_w, d_pooler_b, d_fc_w, d_fc_b (all or none): master gradients, added to.
 * batch * num_labels <= 64.  A label outside [0, num_labels) gives a NaN loss, as TensorFlow's GPU kernel does. */
int ds_classifier_head(int dtype, int batch, int seq, int hidden, int num_labels, const void* x, const float* pooler_w,
                       const float* pooler_b, const float* fc_w, const float* fc_b, const int32_t* labels, float l2_scale,
                       float loss_scale, float* loss, float* pooled, float* logits, float* dlogits, float* dz, void* dx,
                       float* d_pooler_w, float* d_pooler_b, float* d_fc_w, float* d_fc_b, void* stream);

/* pooler_stage alone (bert/models/bert/modeling_slice.py:849-868), the last entry of BertModelSlice.stages:
 * pooled[b] = tanh(x[b, token 0] . pooler_w + pooler_b), pooled fp32 [batch, hidden]. */
int ds_pooler(int dtype, int batch, int seq, int hidden, const void* x, const float* pooler_w, const float* pooler_b, float* pooled,
              void* stream);

/* Pooler and regression head of the last BERT stage: pooler_stage (bert/models/bert/modeling_slice.py:849-868) and
 * build_output_layer_regression, bert/models/bert/bert.py:615-640: prediction = fully_connected(pooled) to ONE output
 * (weights src-output-layer/FC/weights [hidden, 1]), loss = reduce_mean(pow(prediction - labels, 2)) + the l2 regulariser.
 * The prediction is [batch, 1] and the labels placeholder [batch] (bert_finetune.py:212), so the difference broadcasts to
 * [batch, batch] and the mean runs over every (prediction, label) pair: loss = sum_i sum_j (z_i - y_j)^2 / batch^2 +
 * l2_scale * sum(FC weights^2) / 2.  This is what the reference's graph computes and what is computed here.
 *   targets fp32 [batch]; prediction, dprediction fp32 [batch] out; everything else as ds_classifier_head.  batch <= 64. */
int ds_regression_head(int dtype, int batch, int seq, int hidden, const void* x, const float* pooler_w, const float* pooler_b,
                       const float* fc_w, const float* fc_b, const float* targets, float l2_scale, float loss_scale,
                       float* loss, float* pooled, float* prediction, float* dprediction, float* dz, void* dx,
                       float* d_pooler_w, float* d_pooler_b, float* d_fc_w, float* d_fc_b, void* stream);

/* Classification block and loss of the last VGG19 stage: vgg19/applications/vgg19_slice_model.py:217-220 (flatten; fc1,
 * fc2 = Dense(4096, relu); predictions = Dense(classes, softmax)) applied at :342-347, and the loss of :354-355,
 * score_array = K.categorical_crossentropy(x, label); loss = reduce_mean(score_array).
 *   x fp32 [batch, features]: the flattened NHWC output of block5_pool (keras Flatten keeps the row-major order);
 *   fc1_w [features, fc], fc2_w [fc, fc], pred_w [fc, classes] in keras' [in, out] layout, biases [out]; all fp32;
 *   labels fp32 [batch] (the reference feeds a float column, vgg19/tf-keras-dapple.py:57-63);
 *   loss_mode DS_VGG_LOSS_AS_WRITTEN: the expression of the reference's graph - keras takes its first argument as the
 *     target, so the softmax output is the target and the label column the "output": label / sum(label) = 1 (NaN for a
 *     zero label), clipped to 1 - 1e-7, loss = -log(1 - 1e-7) * mean_rows(sum_c x[c]), a constant of about 1.2e-7 whose
 *     gradient behind the softmax is zero up to rounding;
 *   loss_mode DS_VGG_LOSS_SPARSE_CE: labels are class indices, loss = mean_rows(-log x[label]) (NaN for a label that is
 *     no index in [0, classes));
 *   loss: device float, overwritten with loss_scale * loss; probs fp32 [batch, classes] out;
 *   dx (nullable) fp32 [batch, features]: the d_out of the conv stage's backward pass; the six weight gradients (all or
 *   none, nullable) are master gradients, added to.  features, fc, classes multiples of 4. */
#define DS_VGG_LOSS_AS_WRITTEN 0
#define DS_VGG_LOSS_SPARSE_CE 1
size_t ds_vgg_head_workspace_bytes(int batch, int fc, int classes);
int ds_vgg_head(int batch, int features, int fc, int classes, const float* x, const float* fc1_w, const float* fc1_b,
                const float* fc2_w, const float* fc2_b, const float* pred_w, const float* pred_b, const float* labels,
                int loss_mode, float loss_scale, float* loss, float* probs, float* dx, float* d_fc1_w, float* d_fc1_b,
                float* d_fc2_w, float* d_fc2_b, float* d_pred_w, float* d_pred_b, void* workspace, size_t workspace_bytes,
                void* stream);

/* Output projection and loss of the GNMT model on the last device: gnmt/nmt/model.py:685-686 (logits =
 * output_layer(rnn_output); output_layer is a Dense without bias, :497-499) and _compute_loss :824-838
 * (loss = sum(sparse_softmax_cross_entropy(target_output, logits) * sequence_mask(target_sequence_length)) / batch_size).
 *   x fp32 [seq, batch, units]: the outputs of the last decoder cell; proj_kernel fp32 [units, vocab];
 *   target_output int32 [batch, seq] (the reference transposes it, :827-828), target_sequence_length int32 [batch];
 *   loss_batch_size: the divisor (hparams batch_size; 0 = batch);
 *   loss: device float, overwritten with loss_scale * loss; dx (nullable) fp32 [seq, batch, units]: the d_out of the
 *   decoder stage's backward pass; d_proj_kernel (nullable): master gradient, added to.
 * workspace holds the [seq*batch, vocab] logits (turned into their gradient in place).  A label outside [0, vocab)
 * gives a NaN loss, as TensorFlow's GPU kernel does.  units and vocab must be multiples of 4. */
size_t ds_nmt_loss_head_workspace_bytes(int seq, int batch, int vocab);
int ds_nmt_loss_head(int seq, int batch, int units, int vocab, const float* x, const float* proj_kernel,
                     const int32_t* target_output, const int32_t* target_sequence_length, int loss_batch_size,
                     float loss_scale, float* loss, float* dx, float* d_proj_kernel, void* workspace,
                     size_t workspace_bytes, void* stream);

/* SQuAD-2 head of the last XLNet stage: XLnetLoss.call, xlnet/losses/xlnet_loss.py:36-120 (called at
 * xlnet/models/slice_xlnet.py:238-243 on the content stream).  One struct of device pointers names the eleven
 * tensors of the layer; it is used twice, for the fp32 weights and for their master gradients.
 *   start_w [hidden], start_b [1]                     self.dense      (:19)   start logits
 *   end_w0 [2*hidden, hidden], end_b0 [hidden]        self.dense_0    (:20-23) rows [0, hidden) multiply the
 *                                                     sequence output, rows [hidden, 2*hidden) the start feature
 *   ln_gamma, ln_beta [hidden]                        self.layer_norm (:24; layers/layer_normalization.py, eps 1e-14)
 *   end_w1 [hidden], end_b1 [1]                       self.dense_1    (:25)
 *   ans_w0 [2*hidden, hidden], ans_b0 [hidden]        self.dense_0_1  (:26-29) rows [0, hidden) multiply the
 *                                                     probability-weighted start feature, the rest the cls feature
 *   ans_w1 [hidden]                                   self.dense_1_1  (:30-34, no bias) */
typedef struct ds_xlnet_head_params {
  float* start_w; float* start_b;
  float* end_w0;  float* end_b0;
  float* ln_gamma; float* ln_beta;
  float* end_w1;  float* end_b1;
  float* ans_w0;  float* ans_b0;
  float* ans_w1;
} ds_xlnet_head_params;
/* Bytes of device workspace ds_xlnet_squad_head needs for this shape and element type. */
size_t ds_xlnet_squad_head_workspace_bytes(int dtype, int seq, int batch, int hidden);
/* loss = ((start_loss + end_loss) + regression_loss) / 2 (:88, :117-118) and its gradients.
 *   x [seq, batch, hidden] (compute type, time-major like the stage's output); cls_index, start_positions,
 *   end_positions int32 [batch] (an index outside [0, seq) is an all-zero one-hot row, like tf.one_hot);
 *   is_impossible fp32 [batch]; p_mask fp32 [batch, seq];
 *   dropout_mask fp32 [batch, hidden] or NULL: the factor keras.layers.Dropout(0.1)(., training=True) at :103
 *   applies to each element (0 or 1/0.9 in the reference, drawn by TensorFlow's generator; NULL = all ones);
 *   out: loss (device float, loss_scale * loss), start_logits, end_logits fp32 [batch, seq] (unmasked, :51-52 and
 *   :72-73), cls_logits fp32 [batch];
 *   dx (nullable): d loss / d x in the compute type - the d_out of the stage's backward pass;
 *   grads (nullable): master gradients, added to (tf.accumulate_n over micro-batches).
 * The arithmetic is fp32 whatever the compute type.  hidden must be a multiple of 8. */
int ds_xlnet_squad_head(int dtype, int seq, int batch, int hidden, const void* x, const ds_xlnet_head_params* weights,
                        const int32_t* cls_index, const int32_t* start_positions, const int32_t* end_positions,
                        const float* is_impossible, const float* p_mask, const float* dropout_mask, float loss_scale,
                        float* loss, float* start_logits, float* end_logits, float* cls_logits, void* dx,
                        const ds_xlnet_head_params* grads, void* workspace, size_t workspace_bytes, void* stream);

/* ---- what the reference runs on the accumulated gradients right after the unroll block ----
 *
 * Global-norm clipping, bert/graph.py:162-165 (tf.clip_by_global_norm over all accumulated gradients):
 * ds_grad_sqnorm_accum adds sum(g^2) of a buffer into a device double (clear it first, call once per
 * gradient buffer); the update entry points below take that scalar and clip_norm and scale every
 * gradient by clip_norm / max(sqrt(sum), clip_norm) on the fly (pass NULL for no clipping). */
int ds_grad_sqnorm_accum(const float* g, size_t n, double* acc, void* stream);

/* The tensors of a flat fp32 master buffer (element offsets, multiples of 4; element counts) and the
 * decoupled weight-decay rate of each: 0.01 for BERT's matrices, 0 for the names matching
 * "LayerNorm", "layer_norm", "bias" (bert/graph_helper.py:179-185, _do_use_weight_decay :274-282). */
typedef struct ds_optim_plan ds_optim_plan;
int ds_optim_plan_create(int n_tensors, const int64_t* offsets, const int64_t* numels, const float* decay_rates,
                         ds_optim_plan** out);
int ds_optim_plan_destroy(ds_optim_plan* plan);

/* AdamWeightDecayOptimizer.apply_gradients, bert/graph_helper.py:213-272:
 *   m = b1 m + (1-b1) g;  v = b2 v + (1-b2) g^2;  w -= lr * (m / (sqrt(v) + eps) + decay * w)
 * (no bias correction).  tf.train.AdamOptimizer (xlnet/utils/xlnet_utils.py:195-197) is the same update
 * with decay 0 and lr replaced by lr * sqrt(1 - b2^t) / (1 - b1^t), which the caller computes.
 * The hyper-parameters are doubles like the reference's Python floats: 1 - beta is formed in double
 * and then rounded, as TensorFlow does when it folds `1.0 - self.beta_2` into a float32 constant. */
int ds_adam_step(const ds_optim_plan* plan, float* w, const float* g, float* m, float* v, double lr, double beta1,
                 double beta2, double eps, const double* grad_sqnorm, float clip_norm, void* stream);
/* tf.train.GradientDescentOptimizer (vgg19/tf-keras-dapple.py:187): w -= lr * g */
int ds_sgd_step(const ds_optim_plan* plan, float* w, const float* g, double lr, const double* grad_sqnorm,
                float clip_norm, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DAPPLE_STAGE_H */
