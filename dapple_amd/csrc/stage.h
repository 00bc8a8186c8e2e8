// Stage handle behind ds_stage_*: weights (fp32 masters owned by the caller), compute copies,
// workspace and the K-slot activation stash (owned by the handle).
#pragma once
#include <string>
#include <vector>

#include "common.h"

struct WeightInfo {
  std::string name;
  int64_t rows, cols;  // cols == 1 row vector for biases: rows = 1, cols = n
  int64_t numel() const { return rows * cols; }
};

// Bump allocator over one hipMalloc'd arena; every carve is 256-byte aligned.
struct Arena {
  char* base = nullptr;
  size_t cap = 0, used = 0;
  size_t reserve(size_t bytes) {  // planning pass: returns the offset
    const size_t off = used;
    used += (bytes + 255) & ~size_t(255);
    return off;
  }
};

struct ds_stage {
  ds_stage_cfg cfg;
  hipStream_t stream = nullptr;
  std::vector<WeightInfo> winfo;
  std::vector<const float*> w;  // fp32 masters
  std::vector<float*> g;        // fp32 master grads
  bool bound = false;
  std::vector<char> slot_forwarded;
  // optional forward/backward overlap: backward passes run on a second stream, ordered against the
  // forward passes by one event pair per stash slot
  hipStream_t bwd_stream = nullptr;
  hipStream_t wgrad_stream = nullptr;  // weight-gradient GEMMs of a backward pass (stages that support it)
  hipStream_t bwd_owned = nullptr, wgrad_owned = nullptr;  // created once, kept while overlap is switched off
  std::vector<hipEvent_t> ev_forwarded, ev_released;
  std::vector<char> released_valid;
  hipEvent_t ev_join = nullptr;
  hipEvent_t ev_dout = nullptr;  // marks what was queued on `stream` when a backward pass was issued
  bool bwd_pending = false;
  hipEvent_t ev_pair = nullptr;  // end of the latest ds_stage_forward_backward on `stream`: later backward passes share its workspace
  bool pair_valid = false;
  virtual ~ds_stage() {}
  // true when forward and backward passes of different slots touch disjoint memory (apart from
  // read-only weights), so they may run concurrently
  virtual bool overlap_safe() const { return false; }
  virtual int refresh_weights() = 0;
  virtual int forward(int slot, const void* in, const float* key_mask, void* out) = 0;
  virtual int backward(int slot, const void* d_out, void* d_in) = 0;
  // true when forward_backward runs a forward and a backward pass of different slots as one walk over both chains on
  // `stream` (grouped launches); otherwise the two passes are issued one after the other
  virtual bool pairs_passes() const { return false; }
  virtual int forward_backward(int fslot, const void* in, const float* key_mask, void* out, int bslot, const void* d_out, void* d_in) {
    DS_PROPAGATE(forward(fslot, in, key_mask, out));
    return backward(bslot, d_out, d_in);
  }
  // gives up the micro-batch forwarded into `slot` without a backward pass (inference, a forward-only probe)
  virtual int release(int slot) { (void)slot; return DS_OK; }
  virtual size_t workspace_bytes() const = 0;
  virtual size_t stash_bytes(int slots) const = 0;
  // queues weight-gradient work that backward passes have deferred; `final`: and orders it before what the
  // backward stream (or, without one, the stage's stream) runs next
  virtual int flush_deferred(bool final) { (void)final; return DS_OK; }
};

// Bookkeeping for running a layer's weight-gradient work on ds_stage::wgrad_stream beside the dgrad
// chain of the layers below.  The buffers the weight-gradient kernels read alternate by layer parity;
// per parity one event says "the chain produced them" and one "the weight-gradient kernels are done
// with them".
struct WgradLane {
  hipEvent_t ready[2] = {nullptr, nullptr}, done[2] = {nullptr, nullptr};
  bool valid[2] = {false, false};
  ~WgradLane() {
    for (int p = 0; p < 2; ++p) {
      if (ready[p]) (void)hipEventDestroy(ready[p]);
      if (done[p]) (void)hipEventDestroy(done[p]);
    }
  }
  int ensure() {
    if (ready[0]) return DS_OK;
    for (int p = 0; p < 2; ++p) {
      DS_CHECK_HIP(hipEventCreateWithFlags(&ready[p], hipEventDisableTiming));
      DS_CHECK_HIP(hipEventCreateWithFlags(&done[p], hipEventDisableTiming));
    }
    return DS_OK;
  }
  // chain: before it overwrites the parity's buffers
  int reuse(hipStream_t chain, int par) {
    if (valid[par]) DS_CHECK_HIP(hipStreamWaitEvent(chain, done[par], 0));
    return DS_OK;
  }
  // the parity's buffers are complete on `chain`: the weight-gradient stream may read them
  int begin(hipStream_t chain, hipStream_t ws, int par) {
    DS_CHECK_HIP(hipEventRecord(ready[par], chain));
    DS_CHECK_HIP(hipStreamWaitEvent(ws, ready[par], 0));
    return DS_OK;
  }
  int end(hipStream_t ws, int par) {
    DS_CHECK_HIP(hipEventRecord(done[par], ws));
    valid[par] = true;
    return DS_OK;
  }
  // chain: everything on the weight-gradient stream so far is ordered before what follows
  int finish(hipStream_t chain) {
    for (int p = 0; p < 2; ++p)
      if (valid[p]) DS_CHECK_HIP(hipStreamWaitEvent(chain, done[p], 0));
    return DS_OK;
  }
};

// With overlap on, anything that writes into a stash slot on the stage's stream must first wait for the
// backward pass that last used the slot.
static inline int ds_stage_acquire_slot(ds_stage* h, int slot) {
  if (h->bwd_stream && h->released_valid[slot]) DS_CHECK_HIP(hipStreamWaitEvent(h->stream, h->ev_released[slot], 0));
  return DS_OK;
}

int ds_bert_stage_create(const ds_stage_cfg* cfg, hipStream_t stream, ds_stage** out);

// Scores + softmax of XLNet's relative attention with nothing but bf16 probabilities (forward) or bf16 score gradients
// (backward) leaving the kernel (attention_xl.hip): for every stacked query row i' (stream * Q + i), sample b and head n
//   score[j] = (qw[i'] . k[j] + qr[i'] . kr[j + Q - i] + ef[seg(i, j, b)]) * scale - 1e30 * mask[i'][j][b],  p = softmax_j score
struct XlScoreArgs {
  const void *qw, *qr;        // bf16 [QQ][B][H]: q + bias_context, q + bias_relative; row stride ldq, sample b at column b*H
  int64_t ldq;
  const float* de;            // fp32 [B][N][QQ]: (q + bias_segment) . (seg_emb[1] - seg_emb[0]) per head, from ds_xl_bias_q (forward)
  const void* k;              // bf16 key rows: row stride ldk, sample b at column b*ldk_b, head n at column n*64
  const void* v;              // bf16 value rows, strides of k (backward)
  int64_t ldk, ldk_b;
  const void* kr;             // bf16 [R][H]; row stride ldkr
  int64_t ldkr;
  const void* meta;           // mask / segment bits packed by ds_xl_pack_meta, or null (no mask, one segment)
  const float* nseg;          // fp32 [B][Q]: keys of the other segment per query row, or null (backward)
  void* p;                    // bf16 [B*N][QQ][K]: written by forward, read by backward
  const void* dvec;           // bf16, layout of qw: gradient of the attention vector (backward)
  void* ds;                   // bf16 [B*N][QQ][K] (backward out)
  void* dbd;                  // bf16 [B*N][QQ][R]: ds un-shifted; only the band is written (backward out)
  float* defs;                // fp32 [B*N][QQ][2] (backward out)
  int Q, QQ, K, R, B, N, H;
  float scale;
};
// bf16, head size 64, Q and K multiples of 16, K <= 1024, R = K + Q
bool ds_xl_scores_fit(int dtype, int head_dim, int Q, int K, int R);
size_t ds_xl_meta_bytes(int QQ, int K, int B);
// mask fp32 [QQ][K][B] (non-zero = masked) and seg uint8 [Q][K][B], either may be null -> meta; nseg (may be null) <- seg
int ds_xl_pack_meta(int Q, int QQ, int K, int B, const float* mask, const uint8_t* seg, void* meta, float* nseg, hipStream_t stream);
// q bf16 [rows][B][N*64] -> qw, qr, qs (same layout) and de fp32 [B][N][rows]
int ds_xl_bias_q(int rows, int B, int N, const void* q, const float* rw, const float* rr, const float* rs, const float* seg_emb,
                 void* qw, void* qr, void* qs, float* de, hipStream_t stream);
int ds_xl_scores_fwd(const XlScoreArgs* a, hipStream_t stream);
int ds_xl_scores_bwd(const XlScoreArgs* a, hipStream_t stream);
int ds_gemm_splitk(const ds_gemm_desc* d, int splitk, void* stream);
// out[s][c] = scale * sum over the seq rows of sample s of the bf16 matrix x (row stride ldx): per-sample column sums / means
int ds_sample_colsum(int samples, int seq, int cols, const void* x, int64_t ldx, float scale, float* out, void* stream);
// the same for `count` matrices of one shape in one launch
int ds_sample_colsum_multi(int count, int samples, int seq, int cols, const void* const* xs, const int64_t* ldxs, const float* scales,
                           float* const* outs, void* stream);
// w[i][n] -= sum_{s < ns} a[s][i] * b[s][n] and, with v, v[n] -= sum_s b[s][n]   (a [ns][rows], b [ns][cols], w fp32 with row stride ldw)
int ds_rank_update(int rows, int cols, int ns, const float* a, const float* b, float* w, int64_t ldw, float* v, void* stream);
// `count` such updates of one shape in one launch (no two of them on the same w)
int ds_rank_update_multi(int count, int rows, int cols, int ns, const float* const* as, const float* const* bs, float* const* ws, int64_t ldw,
                         float* const* vs, void* stream);
// ds_layernorm_param_grads_exact with x and stats in segments of seg_rows rows, x_seg / st_seg elements apart
int ds_layernorm_param_grads_exact_seg(int rows, int cols, const float* dy_copy, const float* x, const float* gamma, const float* stats,
                                       const float* row_sums, float* d_gamma, float* d_beta, float* d_colsum, int seg_rows, int64_t x_seg,
                                       int64_t st_seg, void* stream);
// ds_colsum_accum for up to 4 matrices of one shape in one launch
int ds_colsum_accum_multi(int dtype, int rows, int cols, int count, const void* const* xs, int64_t ldx, float* const* outs, void* stream);
