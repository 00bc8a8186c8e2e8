// BERT pipeline stage: [embedding] + encoder layers, forward and hand-derived backward, with
// the weight gradients accumulated in place into the caller's fp32 master gradients.
//
// Follows bert/models/bert/modeling_slice.py of the reference: embedding_stage :794-821,
// encoder_layer :942-1001 (attention_layer :357-549, dense+residual+layer_norm, gelu FFN).
// Dropout is the identity (is_training=False zeroes it, :774-776).
#include <stdlib.h>
#include <string.h>

#include <functional>
#include <memory>

#include "group.h"
#include "stage.h"

namespace {

enum LayerW {
  W_Q = 0, W_K, W_V, B_Q, B_K, B_V, W_AO, B_AO, LN1_G, LN1_B, W_FF1, B_FF1, W_FF2, B_FF2, LN2_G, LN2_B, LAYER_NW
};
enum EmbW { E_WORD = 0, E_TYPE, E_POS, E_LN_G, E_LN_B, EMB_NW };

template <typename T>
__global__ __launch_bounds__(256) void pack_qkv_kernel(int H, const float* __restrict__ wq, const float* __restrict__ wk,
                                                      const float* __restrict__ wv, const float* __restrict__ bq,
                                                      const float* __restrict__ bk, const float* __restrict__ bv,
                                                      T* __restrict__ wqkv, float* __restrict__ bqkv) {
  const int64_t total = (int64_t)H * 3 * H;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int h = (int)(i / (3 * H)), j = (int)(i % (3 * H));
    const float* src = j < H ? wq : (j < 2 * H ? wk : wv);
    wqkv[i] = from_f32<T>(src[(int64_t)h * H + (j % H)]);
    if (i < 3 * H) bqkv[i] = (i < H ? bq[i] : (i < 2 * H ? bk[i - H] : bv[i - 2 * H]));
  }
}

// e[r] = word[ids[r]] + type[tt[r]] + pos[r % seq]
template <typename T>
__global__ __launch_bounds__(256) void embed_fwd_kernel(int rows, int H, int seq, int vocab, int type_vocab,
                                                       const int32_t* __restrict__ ids, const int32_t* __restrict__ tt,
                                                       const float* __restrict__ word, const float* __restrict__ type,
                                                       const float* __restrict__ pos, T* __restrict__ e) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  int id = ids[row];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  int t = tt ? tt[row] : 0;
  t = t < 0 ? 0 : (t >= type_vocab ? type_vocab - 1 : t);
  const int s = row % seq;
  for (int c = (threadIdx.x & 63); c < H; c += 64)
    e[(int64_t)row * H + c] = from_f32<T>(word[(int64_t)id * H + c] + type[(int64_t)t * H + c] + pos[(int64_t)s * H + c]);
}

// scatter-add of the embedding-sum gradient into the three tables (repeated ids accumulate)
template <typename T>
__global__ __launch_bounds__(256) void embed_bwd_kernel(int rows, int H, int seq, int vocab, int type_vocab,
                                                       const int32_t* __restrict__ ids, const int32_t* __restrict__ tt,
                                                       const T* __restrict__ de, float* __restrict__ dword,
                                                       float* __restrict__ dtype, float* __restrict__ dpos) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  int id = ids[row];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  int t = tt ? tt[row] : 0;
  t = t < 0 ? 0 : (t >= type_vocab ? type_vocab - 1 : t);
  const int s = row % seq;
  for (int c = (threadIdx.x & 63); c < H; c += 64) {
    const float v = to_f32(de[(int64_t)row * H + c]);
    atomicAdd(dword + (int64_t)id * H + c, v);
    atomicAdd(dtype + (int64_t)t * H + c, v);
    atomicAdd(dpos + (int64_t)s * H + c, v);
  }
}

// A stashed tensor: `size` bytes per stash position, the positions back to back from byte `off` of the stash.
// Consecutive positions of a [rows, cols] tensor therefore read as one [n*rows, cols] matrix.
struct Ten {
  size_t off = 0, size = 0;
};
struct LayerStash {
  Ten x, qkv, p, ctx, z1, a, u, h, z2, st1, st2, lse, kbar, xbar;
};
// Upstream-gradient operands of a layer's weight-gradient GEMMs when those are deferred: per tensor a ring
// of positions back to back, byte offsets into dy_base.
struct LayerDy {
  size_t dz2, du, dz1, dqkv;
  size_t dyn2, dyn1;  // fp32 residual stream: fp32 copies of the gradients that entered the two LayerNorms
  size_t rs2, rs1;    // and the two per-row means of each LayerNorm's backward pass
  size_t dksum;       // fused attention: per sample, the column sums of the pass's key gradients (fp32 [B][H])
};
struct Deferred {
  int xpos, dypos;
};
struct Run {  // n micro-batches back to back in the stash and in the operand ring
  int xpos, dypos, n;
};

struct BertStage : ds_stage {
  int L, H, F, NH, D, B, S, rows;
  int dtype;
  size_t esz;
  bool emb;
  bool fused_attn;  // bf16, head size 64: fused attention kernels, no [B,N,S,S] tensors at all
  // fused attention: query gradients through ds_attention_bwd_centered, key parameter gradients from key gradients
  // centred over each sample (DS_BERT_CENTRED=0 switches both off, for measurements)
  bool centred = false, centre_q = false, centre_k = false;
  // bf16 with cfg.residual_fp32: the residual stream - the sums in front of both LayerNorms, the LayerNorm outputs that
  // feed the next sum, and the same chain of gradients in backward - stays in fp32; bf16 is only what a GEMM or the
  // attention kernels read.  The rounding of the stream itself, which otherwise adds up over the layers, is gone.
  bool rs32 = false;
  size_t fw_xf[2] = {0, 0}, fw_af = 0, bw_dxf[2] = {0, 0}, bw_dz2f = 0, bw_daf = 0, bw_dz1f = 0;
  // the forward pass writes its stash slot, its output and (unfused attention) its own score buffer; the rest
  // of the workspace belongs to backward
  bool overlap_safe() const override { return true; }
  // compute copies
  char* wc_base = nullptr;
  std::vector<char*> wqkv, wo, w1, w2;  // element type T
  std::vector<float*> bqkv;
  // stash: the tensors live at stash positions; with per-pass weight gradients position = slot
  char* stash_base = nullptr;
  size_t pos_bytes = 0;  // all tensors of one position
  Ten emb_e, emb_st;
  std::vector<LayerStash> ls;
  // small per-slot inputs (mask, token ids, token types)
  char* small_base = nullptr;
  size_t small_bytes = 0;
  size_t emb_ids = 0, emb_tt = 0, mask_off = 0;
  // Deferred weight gradients (cfg.wgrad_group = G > 1).  A backward pass leaves its upstream-gradient operands
  // in position (count of backward passes) % 2G of a per-layer ring and the activations where the forward
  // pass put them; after G passes ONE GEMM per weight contracts over all G micro-batches' rows.  Forward
  // passes take stash positions round-robin out of K+G, so that G consecutive micro-batches sit back to back.
  int G = 1, KP = 0, NDY = 0;
  char* dy_base = nullptr;
  std::vector<LayerDy> ld;
  size_t dy_act = 0, dy_actF = 0, dy_act32 = 0;
  std::vector<int> slot_pos, pos_owner;
  std::vector<char> pos_deferred;
  int next_pos = 0;
  long n_backward = 0;
  std::vector<Deferred> deferred;
  hipEvent_t ev_chain = nullptr, ev_wg_done = nullptr, ev_refresh = nullptr;
  std::vector<hipEvent_t> ev_cast;   // compute copies of layer l written (refresh_weights on the weight-gradient stream)
  std::vector<char> cast_pending;
  std::vector<hipEvent_t> ev_x_bwd, ev_x_wg, ev_dy_wg;
  std::vector<char> x_bwd_valid, x_wg_valid, dy_wg_valid;
  bool wg_outstanding = false;
  size_t out_off = 0;  // last layer's y is written straight to the caller's buffer
  std::vector<char> slot_has_mask, slot_has_tt;
  // workspace
  char* ws_base = nullptr;
  size_t ws_bytes = 0;
  size_t ws_scores, ws_fscores, ws_ds, ws_dz2[2], ws_du[2], ws_da, ws_dz1[2], ws_dctx, ws_dqkv[2], ws_dx[2];
  size_t ws_dksum = 0;
  WgradLane lane;

  ~BertStage() override {
    if (wc_base) (void)hipFree(wc_base);
    if (stash_base) (void)hipFree(stash_base);
    if (small_base) (void)hipFree(small_base);
    if (dy_base) (void)hipFree(dy_base);
    if (ev_chain) (void)hipEventDestroy(ev_chain);
    if (ev_wg_done) (void)hipEventDestroy(ev_wg_done);
    if (ev_refresh) (void)hipEventDestroy(ev_refresh);
    for (hipEvent_t e : ev_cast) (void)hipEventDestroy(e);
    for (hipEvent_t e : ev_x_bwd) (void)hipEventDestroy(e);
    for (hipEvent_t e : ev_x_wg) (void)hipEventDestroy(e);
    for (hipEvent_t e : ev_dy_wg) (void)hipEventDestroy(e);
    if (ws_base) (void)hipFree(ws_base);
  }
  int base(int l) const { return (emb ? EMB_NW : 0) + l * LAYER_NW; }
  char* at(const Ten& t, int pos) const { return stash_base + t.off + (size_t)pos * t.size; }
  char* smallp(int slot) const { return small_base + (size_t)slot * small_bytes; }

  int init() {
    const ds_stage_cfg& c = cfg;
    L = c.num_layers; H = c.hidden; F = c.ffn; NH = c.heads; B = c.batch; S = c.seq;
    D = H / NH; rows = B * S; dtype = c.dtype; esz = dtype == DS_BF16 ? 2 : 4; emb = c.with_embedding != 0;
    fused_attn = dtype == DS_BF16 && D == 64 && S % 64 == 0 && S <= 2048;
    {
      const char* env = getenv("DS_BERT_CENTRED");
      centred = fused_attn && !(env && atoi(env) == 0);
      centre_q = centred && !(env && atoi(env) == 3);
      centre_k = centred && !(env && atoi(env) == 2);
    }
    rs32 = dtype == DS_BF16 && c.residual_fp32 != 0 && L > 0 && H % 8 == 0 && H <= 2048;
    char name[160];
    if (emb) {
      winfo.push_back({"bert/embeddings/word_embeddings", c.vocab, H});
      winfo.push_back({"bert/embeddings/token_type_embeddings", c.type_vocab, H});
      winfo.push_back({"bert/embeddings/position_embeddings", c.max_pos, H});
      winfo.push_back({"bert/embeddings/LayerNorm/gamma", 1, H});
      winfo.push_back({"bert/embeddings/LayerNorm/beta", 1, H});
    }
    const int first = c.first_layer;
    for (int l = 0; l < L; ++l) {
      auto add = [&](const char* suffix, int64_t r, int64_t cc) {
        snprintf(name, sizeof(name), "bert/encoder/layer_%d/%s", first + l, suffix);
        winfo.push_back({name, r, cc});
      };
      add("attention/self/query/kernel", H, H);
      add("attention/self/key/kernel", H, H);
      add("attention/self/value/kernel", H, H);
      add("attention/self/query/bias", 1, H);
      add("attention/self/key/bias", 1, H);
      add("attention/self/value/bias", 1, H);
      add("attention/output/dense/kernel", H, H);
      add("attention/output/dense/bias", 1, H);
      add("attention/output/LayerNorm/gamma", 1, H);
      add("attention/output/LayerNorm/beta", 1, H);
      add("intermediate/dense/kernel", H, F);
      add("intermediate/dense/bias", 1, F);
      add("output/dense/kernel", F, H);
      add("output/dense/bias", 1, H);
      add("output/LayerNorm/gamma", 1, H);
      add("output/LayerNorm/beta", 1, H);
    }
    // ---- compute copies
    Arena wa;
    std::vector<size_t> o_qkv(L), o_b(L), o_wo(L), o_w1(L), o_w2(L);
    for (int l = 0; l < L; ++l) {
      o_qkv[l] = wa.reserve((size_t)H * 3 * H * esz);
      o_b[l] = wa.reserve((size_t)3 * H * 4);
      if (dtype == DS_BF16) {
        o_wo[l] = wa.reserve((size_t)H * H * esz);
        o_w1[l] = wa.reserve((size_t)H * F * esz);
        o_w2[l] = wa.reserve((size_t)F * H * esz);
      }
    }
    if (wa.used) DS_CHECK_HIP(hipMalloc((void**)&wc_base, wa.used));
    wqkv.resize(L); wo.resize(L); w1.resize(L); w2.resize(L); bqkv.resize(L);
    for (int l = 0; l < L; ++l) {
      wqkv[l] = wc_base + o_qkv[l];
      bqkv[l] = (float*)(wc_base + o_b[l]);
      if (dtype == DS_BF16) { wo[l] = wc_base + o_wo[l]; w1[l] = wc_base + o_w1[l]; w2[l] = wc_base + o_w2[l]; }
    }
    // ---- stash layout
    const int K = c.stash_slots;
    G = c.wgrad_group > 1 ? c.wgrad_group : 1;
    // (a multiple of G: the G micro-batches of a group then always sit back to back, one GEMM per weight and group)
    KP = G > 1 ? (K + G + G - 1) / G * G : K;
    NDY = 2 * G;
    const size_t act = (size_t)rows * H * esz, actF = (size_t)rows * F * esz;
    const size_t probs = (size_t)B * NH * S * S * esz, stats = (size_t)rows * 2 * 4;
    size_t ring_used = 0;
    auto ring = [&](size_t bytes) {  // rows of 16-byte multiples: no padding between positions
      Ten t;
      t.size = (bytes + 15) & ~size_t(15);
      t.off = ring_used;
      ring_used += t.size * (size_t)KP;
      ring_used = (ring_used + 255) & ~size_t(255);
      pos_bytes += t.size;
      return t;
    };
    Arena sm;
    mask_off = sm.reserve((size_t)B * S * 4);
    if (emb) {
      emb_ids = sm.reserve((size_t)rows * 4);
      emb_tt = sm.reserve((size_t)rows * 4);
      emb_e = ring(act);
      emb_st = ring(stats);
    }
    small_bytes = sm.used;
    ls.resize(L);
    Ten next_x = L ? ring(act) : Ten();
    for (int l = 0; l < L; ++l) {
      LayerStash& t = ls[l];
      t.x = next_x;
      t.qkv = ring(3 * act);
      if (fused_attn) {
        t.lse = ring((size_t)B * NH * S * 4);
        t.kbar = ring((size_t)B * H * 4);  // mean key per sample and head
        t.xbar = ring((size_t)B * H * 4);  // mean input row per sample
      }
      else t.p = ring(probs);
      t.ctx = ring(act);
      t.z1 = ring(rs32 ? (size_t)rows * H * 4 : act);
      t.a = ring(act);
      t.u = ring(actF);
      t.h = ring(actF);
      t.z2 = ring(rs32 ? (size_t)rows * H * 4 : act);
      t.st1 = ring(stats);
      t.st2 = ring(stats);
      if (l + 1 < L) next_x = ring(act);
    }
    DS_CHECK_HIP(hipMalloc((void**)&stash_base, ring_used ? ring_used : 256));
    DS_CHECK_HIP(hipMalloc((void**)&small_base, small_bytes * K));
    slot_forwarded.assign(K, 0);
    slot_has_mask.assign(K, 0);
    slot_has_tt.assign(K, 0);
    slot_pos.assign(K, 0);
    for (int i = 0; i < K; ++i) slot_pos[i] = i;
    if (G > 1) {
      pos_owner.assign(KP, -1);
      pos_deferred.assign(KP, 0);
      Arena da;
      ld.resize(L);
      dy_act = act; dy_actF = actF; dy_act32 = (size_t)rows * H * 4;
      for (int l = 0; l < L; ++l) {
        ld[l].dz2 = da.reserve(act * NDY);
        ld[l].du = da.reserve(actF * NDY);
        ld[l].dz1 = da.reserve(act * NDY);
        ld[l].dqkv = da.reserve(3 * act * NDY);
        if (rs32) {
          ld[l].dyn2 = da.reserve(dy_act32 * NDY);
          ld[l].dyn1 = da.reserve(dy_act32 * NDY);
          ld[l].rs2 = da.reserve((size_t)rows * 8 * NDY);
          ld[l].rs1 = da.reserve((size_t)rows * 8 * NDY);
        }
        ld[l].dksum = da.reserve((size_t)B * H * 4 * NDY);
      }
      if (da.used) DS_CHECK_HIP(hipMalloc((void**)&dy_base, da.used));
      DS_CHECK_HIP(hipEventCreateWithFlags(&ev_chain, hipEventDisableTiming));
      DS_CHECK_HIP(hipEventCreateWithFlags(&ev_wg_done, hipEventDisableTiming));
      ev_x_bwd.assign(KP, nullptr); ev_x_wg.assign(KP, nullptr); ev_dy_wg.assign(NDY, nullptr);
      for (auto& e : ev_x_bwd) DS_CHECK_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
      for (auto& e : ev_x_wg) DS_CHECK_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
      for (auto& e : ev_dy_wg) DS_CHECK_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
      x_bwd_valid.assign(KP, 0); x_wg_valid.assign(KP, 0); dy_wg_valid.assign(NDY, 0);
    }
    // ---- workspace
    Arena w;
    ws_scores = w.reserve(fused_attn ? (size_t)B * NH * S * 4 : (size_t)B * NH * S * S * 4);  // fused: delta
    ws_fscores = fused_attn ? 0 : w.reserve((size_t)B * NH * S * S * 4);  // forward's own scores: backward keeps ws_scores
    ws_ds = fused_attn ? 0 : w.reserve(probs);
    for (int p = 0; p < 2; ++p) {  // the operands of the weight-gradient GEMMs alternate by layer parity
      ws_dz2[p] = w.reserve(act);
      ws_du[p] = w.reserve(actF);
      ws_dz1[p] = w.reserve(act);
      ws_dqkv[p] = w.reserve(3 * act);
    }
    ws_da = w.reserve(act);
    ws_dctx = w.reserve(act);
    ws_dx[0] = w.reserve(act);
    ws_dx[1] = w.reserve(act);
    if (rs32) {
      const size_t act32 = (size_t)rows * H * 4;
      fw_xf[0] = w.reserve(act32); fw_xf[1] = w.reserve(act32); fw_af = w.reserve(act32);
      bw_dxf[0] = w.reserve(act32); bw_dxf[1] = w.reserve(act32);
      bw_dz2f = w.reserve(act32); bw_daf = w.reserve(act32); bw_dz1f = w.reserve(act32);
    }
    if (fused_attn) {  // per-sample means of a layer's inputs and column sums of its key gradients (weight-gradient side)
      const size_t ns = (size_t)(G > 1 ? G : 1) * B;
      ws_dksum = w.reserve(ns * H * 4);
    }
    ws_bytes = w.used;
    DS_CHECK_HIP(hipMalloc((void**)&ws_base, ws_bytes));
    return DS_OK;
  }

  size_t workspace_bytes() const override { return ws_bytes; }
  size_t stash_bytes(int slots) const override {
    return (pos_bytes + small_bytes) * (size_t)slots + (G > 1 ? pos_bytes * (size_t)G : 0);
  }

  const void* weight_T(int l, int which) const {  // kernel in the element type
    if (dtype == DS_BF16) return which == W_AO ? wo[l] : (which == W_FF1 ? w1[l] : w2[l]);
    return w[base(l) + which];
  }

  // The compute copies of layer l are only needed when the next forward pass reaches layer l.  With a weight-gradient
  // stream at hand (idle between steps) the copies of layers 1.. are made there, one event per layer, and the first
  // forward pass after the refresh waits for each layer's event as it gets to it: the pass starts after one layer's
  // casts instead of after all of them.
  int refresh_weights() override {
    hipStream_t side = wgrad_stream;
    if (side) {
      if (ev_cast.empty()) {
        ev_cast.resize(L);
        for (int l = 0; l < L; ++l) DS_CHECK_HIP(hipEventCreateWithFlags(&ev_cast[l], hipEventDisableTiming));
        DS_CHECK_HIP(hipEventCreateWithFlags(&ev_refresh, hipEventDisableTiming));
      }
      // everything queued before this call (the master weights' last update among it) precedes the casts
      DS_CHECK_HIP(hipEventRecord(ev_refresh, stream));
      DS_CHECK_HIP(hipStreamWaitEvent(side, ev_refresh, 0));
    }
    cast_pending.assign(L, 0);
    for (int l = 0; l < L; ++l) {
      const int b = base(l);
      hipStream_t cs = (side && l > 0) ? side : stream;
      if (dtype == DS_BF16) {
        hipLaunchKernelGGL(pack_qkv_kernel<bf16>, dim3(1024), dim3(256), 0, cs, H, w[b + W_Q], w[b + W_K], w[b + W_V],
                           w[b + B_Q], w[b + B_K], w[b + B_V], (bf16*)wqkv[l], bqkv[l]);
        DS_CHECK_LAUNCH();
        DS_PROPAGATE(ds_cast_f32_to_bf16(wo[l], w[b + W_AO], (size_t)H * H, cs));
        DS_PROPAGATE(ds_cast_f32_to_bf16(w1[l], w[b + W_FF1], (size_t)H * F, cs));
        DS_PROPAGATE(ds_cast_f32_to_bf16(w2[l], w[b + W_FF2], (size_t)F * H, cs));
      } else {
        hipLaunchKernelGGL(pack_qkv_kernel<float>, dim3(1024), dim3(256), 0, cs, H, w[b + W_Q], w[b + W_K], w[b + W_V],
                           w[b + B_Q], w[b + B_K], w[b + B_V], (float*)wqkv[l], bqkv[l]);
        DS_CHECK_LAUNCH();
      }
      if (cs != stream) {
        DS_CHECK_HIP(hipEventRecord(ev_cast[l], cs));
        cast_pending[l] = 1;
      }
    }
    return DS_OK;
  }
  // called by whatever reads layer l's compute copies first on `s`
  int await_cast(int l, hipStream_t s) {
    if (!cast_pending.empty() && cast_pending[l]) {
      DS_CHECK_HIP(hipStreamWaitEvent(s, ev_cast[l], 0));
      cast_pending[l] = 0;
    }
    return DS_OK;
  }

  // C[rows_m, n] = A[rows_m, k] (K-major) x W[k, n] (MN-major) with an epilogue
  ds_gemm_desc desc_fwd(int m, int n, int k, const void* a, const void* wt, void* c, int flags, const float* bias,
                        const void* residual, void* c2) const {
    ds_gemm_desc d;
    memset(&d, 0, sizeof(d));
    d.dtype = dtype; d.a_major = DS_K_MAJOR; d.b_major = DS_MN_MAJOR;
    d.m = m; d.n = n; d.k = k; d.lda = k; d.ldb = n; d.ldc = n; d.batch = 1; d.batch_inner = 1;
    d.flags = flags; d.alpha = 1.f; d.a = a; d.b = wt; d.c = c; d.bias = bias; d.residual = residual; d.c2 = c2;
    return d;
  }
  // dX[m, k] = dY[m, n] x W[k, n]^T (+ residual) (* gelu'(aux))
  ds_gemm_desc desc_dgrad(int m, int n, int k, const void* dy, const void* wt, void* dx, int flags, const void* residual,
                          void* aux) const {
    ds_gemm_desc d;
    memset(&d, 0, sizeof(d));
    d.dtype = dtype; d.a_major = DS_K_MAJOR; d.b_major = DS_K_MAJOR;
    d.m = m; d.n = k; d.k = n; d.lda = n; d.ldb = n; d.ldc = k; d.batch = 1; d.batch_inner = 1;
    d.flags = flags; d.alpha = 1.f; d.a = dy; d.b = wt; d.c = dx; d.residual = residual; d.c2 = aux;
    return d;
  }
  // dW[k, n] (fp32) += X[m, k]^T x dY[m, n]
  ds_gemm_desc desc_wgrad(int m, int n, int k, const void* x, int64_t ldx, const void* dy, int64_t ldy, float* dw, int64_t lddw) const {
    ds_gemm_desc d;
    memset(&d, 0, sizeof(d));
    d.dtype = dtype; d.a_major = DS_MN_MAJOR; d.b_major = DS_MN_MAJOR;
    d.m = k; d.n = n; d.k = m; d.lda = ldx; d.ldb = ldy; d.ldc = lddw; d.batch = 1; d.batch_inner = 1;
    d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.a = x; d.b = dy; d.c = dw;
    return d;
  }
  int gemm_wgrad(int m, int n, int k, const void* x, int64_t ldx, const void* dy, int64_t ldy, float* dw, int64_t lddw) {
    const ds_gemm_desc d = desc_wgrad(m, n, k, x, ldx, dy, ldy, dw, lddw);
    return ds_gemm(&d, stream);
  }
  // per-(batch, head) GEMM on [rows, ld] matrices whose head h owns columns h*D..h*D+D-1
  int gemm_heads(int am, int bm, int m, int n, int k, const void* a, int64_t lda, int64_t a_so, int64_t a_si,
                 const void* b, int64_t ldb, int64_t b_so, int64_t b_si, void* c, int64_t ldc, int64_t c_so, int64_t c_si,
                 int flags) {
    ds_gemm_desc d;
    memset(&d, 0, sizeof(d));
    d.dtype = dtype; d.a_major = am; d.b_major = bm;
    d.m = m; d.n = n; d.k = k; d.lda = lda; d.ldb = ldb; d.ldc = ldc; d.batch = B * NH; d.batch_inner = NH;
    d.a_stride_outer = a_so; d.a_stride_inner = a_si; d.b_stride_outer = b_so; d.b_stride_inner = b_si;
    d.c_stride_outer = c_so; d.c_stride_inner = c_si;
    d.flags = flags; d.alpha = 1.f; d.a = a; d.b = b; d.c = c;
    return ds_gemm(&d, stream);
  }

  // A stash position for the next forward pass: round-robin, skipping positions whose micro-batch has not
  // been through backward; a position that deferred weight-gradient work still reads is flushed first.
  int take_pos(int* out) {
    for (int tries = 0; tries < KP; ++tries) {
      const int p = next_pos;
      next_pos = next_pos + 1 == KP ? 0 : next_pos + 1;
      if (pos_owner[p] >= 0) continue;
      if (pos_deferred[p]) DS_PROPAGATE(flush_deferred(false));
      *out = p;
      return DS_OK;
    }
    ds_set_error("ds_stage_forward: no free stash position");
    return DS_ESTATE;
  }

  // ---- a pass as a sequence of steps
  // A step is one link of a pass's chain of dependent kernels.  `solo` launches it as kernels of its own on `stream`;
  // `ops` describe the same work as tasks of a grouped launch (group.h) where the stage's configuration allows - then
  // a forward and a backward pass of different micro-batches advance level by level, one launch per level carrying a
  // step of each.  `before` / `after` are the host's work around the step: event waits, launches on other streams.
  struct Step {
    std::function<int()> before, solo, after;
    int nops = 0;
    GroupOp ops[2];
  };
  typedef std::vector<Step> Steps;
  // grouped launches exist for the bf16 kernels of the benchmarked configuration: fused attention, fp32 residual stream
  // and deferred weight gradients (whose backward LayerNorm is the row kernel)
  bool groupable() const { return fused_attn && rs32 && G > 1 && H % 64 == 0 && F % 64 == 0 && H >= 192 && F >= 192; }
  bool pairs_passes() const override { return groupable(); }

  static Step& add(Steps& st, std::function<int()> solo) {
    st.emplace_back();
    st.back().solo = std::move(solo);
    return st.back();
  }
  Step& add_gemm(Steps& st, const ds_gemm_desc& d, int prio) {
    Step& s = add(st, [this, d]() { return ds_gemm(&d, stream); });
    if (groupable()) {
      s.nops = 1;
      s.ops[0].kind = GOP_GEMM;
      s.ops[0].gemm = d;
      s.ops[0].prio = prio;
    }
    return s;
  }
  Step& add_ln_fwd(Steps& st, int prio, const float* x, const float* gamma, const float* beta, void* y16, float* y32, float* stats) {
    Step& s = add(st, [=]() { return ds_layernorm_fwd_mixed(rows, H, x, gamma, beta, cfg.ln_eps, y16, y32, stats, stream); });
    if (groupable()) {
      GroupOp& o = s.ops[0];
      s.nops = 1;
      o.kind = GOP_LN_FWD; o.prio = prio; o.rows = rows; o.cols = H; o.x = x; o.gamma = gamma; o.beta = beta; o.eps = cfg.ln_eps;
      o.y16 = y16; o.y32 = y32; o.stats = stats;
    }
    return s;
  }
  Step& add_ln_bwd_rows(Steps& st, int prio, const float* dy, const float* x, const float* gamma, const float* stats, void* dx16, float* dx32,
                        float* dy32, float* row_sums) {
    Step& s = add(st, [=]() { return ds_layernorm_bwd_mixed_rows(rows, H, dy, x, gamma, stats, dx16, dx32, dy32, row_sums, stream); });
    if (groupable()) {
      GroupOp& o = s.ops[0];
      s.nops = 1;
      o.kind = GOP_LN_BWD; o.prio = prio; o.rows = rows; o.cols = H; o.x = x; o.gamma = gamma; o.stats = (float*)stats; o.dy = dy;
      o.y16 = dx16; o.y32 = dx32; o.dy32 = dy32; o.row_sums = row_sums;
    }
    return s;
  }
  void attn_op(GroupOp& o, int kind, int prio, const void* qkv, const float* mask, void* ctx, float* lse, const void* dctx, void* dqkv,
               float* delta) const {
    o.kind = kind; o.prio = prio; o.B = B; o.N = NH; o.S = S; o.qkv = qkv; o.ld = 3 * H; o.key_mask = mask;
    o.scale = 1.0f / sqrtf((float)D); o.mask_value = -10000.0f; o.ctx = ctx; o.lse = lse; o.dctx = dctx; o.dqkv = dqkv; o.delta = delta;
  }

  // one pass alone: every step as launches of its own, in order
  int play(const Steps& st) {
    for (const Step& s : st) {
      if (s.before) DS_PROPAGATE(s.before());
      DS_PROPAGATE(s.solo());
      if (s.after) DS_PROPAGATE(s.after());
    }
    return DS_OK;
  }

  // Tile shapes of the grouped launches (DS_GROUP_CFG_WIDE / _NARROW: tuning overrides, group.h numbering).
  void choose_cfg(GroupOp& o) const {
    if (o.kind != GOP_GEMM || o.cfg >= 0) return;
    static const char* env_w = getenv("DS_GROUP_CFG_WIDE");
    static const char* env_n = getenv("DS_GROUP_CFG_NARROW");
    const bool narrow = o.gemm.n <= 1024 && o.gemm.m <= 1024;
    if (narrow) o.cfg = env_n ? atoi(env_n) : 3;
    else o.cfg = env_w ? atoi(env_w) : 4;
    // a tile ring must be shorter than the reduction: the two-buffer shapes take anything from three k-tiles on
    const int ktiles = o.gemm.k / 64;
    if (o.cfg == 3 && ktiles <= 4) o.cfg = 5;
    if ((o.cfg == 1 || o.cfg == 2) && ktiles <= 3) o.cfg = 4;
  }

  // A forward and a backward pass of different micro-batches side by side on `stream`: steps that exist as tasks go
  // out as ONE launch per level - the next step of either chain - the others as launches of their own.  The backward
  // chain runs `lead` levels ahead so that steps of different kinds meet (DS_GROUP_LEAD).
  int play_pair(Steps& f, Steps& b) {
    static const char* env_lead = getenv("DS_GROUP_LEAD");
    int lead = env_lead ? atoi(env_lead) : 1;
    size_t fi = 0, bi = 0;
    while (fi < f.size() || bi < b.size()) {
      // steps that only exist as launches of their own go first, forward chain first
      if (fi < f.size() && f[fi].nops == 0) {
        DS_PROPAGATE(play_one(f[fi++], 1));
        continue;
      }
      if (bi < b.size() && b[bi].nops == 0) {
        DS_PROPAGATE(play_one(b[bi++], 3));
        continue;
      }
      Step* sf = fi < f.size() ? &f[fi] : nullptr;
      Step* sb = bi < b.size() ? &b[bi] : nullptr;
      if (lead > 0 && sb) { sf = nullptr; --lead; }
      GroupOp ops[4];
      int n = 0;
      if (sb) {
        if (sb->before) DS_PROPAGATE(sb->before());
        for (int i = 0; i < sb->nops; ++i) ops[n++] = sb->ops[i];
      }
      if (sf) {
        if (sf->before) DS_PROPAGATE(sf->before());
        for (int i = 0; i < sf->nops; ++i) ops[n++] = sf->ops[i];
      }
      for (int i = 0; i < n; ++i) choose_cfg(ops[i]);
      DS_PROPAGATE(ds_group_launch(ops, n, stream));
      if (sb) {
        if (sb->after) DS_PROPAGATE(sb->after());
        ++bi;
      }
      if (sf) {
        if (sf->after) DS_PROPAGATE(sf->after());
        ++fi;
      }
    }
    return DS_OK;
  }
  int play_one(const Step& s, int prio) {
    ds_prio_scope scope(prio);
    if (s.before) DS_PROPAGATE(s.before());
    DS_PROPAGATE(s.solo());
    if (s.after) DS_PROPAGATE(s.after());
    return DS_OK;
  }

  // Per sample, the mean key of every head (what ds_attention_bwd_centered wants) and the mean input row (for the key
  // kernel's weight gradient) of every layer, in one launch at the end of the forward pass that wrote them.  (On the
  // weight-gradient stream it would queue behind a whole group's GEMMs, and the slot's backward pass would wait for it.)
  int sample_means(int pos) {
    std::vector<const void*> xs;
    std::vector<int64_t> lds;
    std::vector<float> scales;
    std::vector<float*> outs;
    for (int l = 0; l < L; ++l) {
      xs.push_back(at(ls[l].qkv, pos) + (size_t)H * esz); lds.push_back(3 * H); outs.push_back((float*)at(ls[l].kbar, pos));
      xs.push_back(at(ls[l].x, pos)); lds.push_back(H); outs.push_back((float*)at(ls[l].xbar, pos));
      scales.push_back(1.0f / S); scales.push_back(1.0f / S);
    }
    return ds_sample_colsum_multi((int)xs.size(), B, S, H, xs.data(), lds.data(), scales.data(), outs.data(), stream);
  }

  int forward(int slot, const void* in, const float* key_mask, void* out) override {
    ds_prio_scope prio(1);
    Steps st;
    DS_PROPAGATE(forward_steps(slot, in, key_mask, out, st));
    return play(st);
  }

  int forward_steps(int slot, const void* in, const float* key_mask, void* out, Steps& st) {
    const int prio = 1;
    int pos = slot;
    if (G > 1) {
      DS_PROPAGATE(take_pos(&pos));
      pos_owner[pos] = slot;
      slot_pos[slot] = pos;
      // the backward pass and the weight-gradient GEMMs that last read this position
      if (x_bwd_valid[pos]) DS_CHECK_HIP(hipStreamWaitEvent(stream, ev_x_bwd[pos], 0));
      if (x_wg_valid[pos]) DS_CHECK_HIP(hipStreamWaitEvent(stream, ev_x_wg[pos], 0));
    }
    char* sm = smallp(slot);
    const size_t act = (size_t)rows * H * esz;
    const float scale = 1.0f / sqrtf((float)D);
    const float* mask = key_mask ? (const float*)(sm + mask_off) : nullptr;
    slot_has_mask[slot] = key_mask != nullptr;
    char* x0 = L ? at(ls[0].x, pos) : nullptr;
    add(st, [=]() {  // the micro-batch's inputs into the slot, the embedding if the stage has it
      if (key_mask) DS_CHECK_HIP(hipMemcpyAsync(sm + mask_off, key_mask, (size_t)B * S * 4, hipMemcpyDeviceToDevice, stream));
      if (emb) {
        DS_CHECK_HIP(hipMemcpyAsync(sm + emb_ids, in, (size_t)rows * 4, hipMemcpyDeviceToDevice, stream));
        const int32_t* tt = slot_has_tt[slot] ? (const int32_t*)(sm + emb_tt) : nullptr;
        dim3 grid((rows + 3) / 4);
        if (dtype == DS_BF16)
          hipLaunchKernelGGL(embed_fwd_kernel<bf16>, grid, dim3(256), 0, stream, rows, H, S, cfg.vocab, cfg.type_vocab,
                             (const int32_t*)(sm + emb_ids), tt, w[E_WORD], w[E_TYPE], w[E_POS], (bf16*)(at(emb_e, pos)));
        else
          hipLaunchKernelGGL(embed_fwd_kernel<float>, grid, dim3(256), 0, stream, rows, H, S, cfg.vocab, cfg.type_vocab,
                             (const int32_t*)(sm + emb_ids), tt, w[E_WORD], w[E_TYPE], w[E_POS], (float*)(at(emb_e, pos)));
        DS_CHECK_LAUNCH();
        DS_PROPAGATE(ds_layernorm_fwd(dtype, rows, H, at(emb_e, pos), w[E_LN_G], w[E_LN_B], cfg.ln_eps, L ? (void*)x0 : out,
                                      (float*)(at(emb_st, pos)), stream));
      } else {
        DS_CHECK_HIP(hipMemcpyAsync(x0, in, act, hipMemcpyDeviceToDevice, stream));
      }
      if (rs32) DS_PROPAGATE(ds_cast_bf16_to_f32(ws_base + fw_xf[0], x0, (size_t)rows * H, stream));
      return DS_OK;
    });
    for (int l = 0; l < L; ++l) {
      const LayerStash& t = ls[l];
      const int b = base(l);
      char* x = at(t.x, pos);
      char* y = (l + 1 < L) ? at(ls[l + 1].x, pos) : (char*)out;
      char* qkv = at(t.qkv, pos);
      // fused Q|K|V projection (modeling_slice.py:464-485)
      {
        Step& s = add_gemm(st, desc_fwd(rows, 3 * H, H, x, wqkv[l], qkv, DS_EPI_BIAS, bqkv[l], nullptr, nullptr), prio);
        s.before = [this, l]() { return await_cast(l, stream); };
      }
      if (fused_attn) {
        // scores, scale, mask adder, softmax and context in one kernel (:499-533)
        char* ctx = at(t.ctx, pos);
        float* lse = (float*)(at(t.lse, pos));
        Step& s = add(st, [=]() { return ds_attention_fwd(dtype, B, NH, S, D, qkv, 3 * H, mask, scale, -10000.0f, ctx, lse, stream); });
        if (groupable()) {
          s.nops = 1;
          attn_op(s.ops[0], GOP_ATTN_FWD, prio, qkv, mask, ctx, lse, nullptr, nullptr, nullptr);
        }
      } else {
        char* p = at(t.p, pos);
        char* ctx = at(t.ctx, pos);
        add(st, [=]() {
          // scores = Q K^T (:499), fp32
          DS_PROPAGATE(gemm_heads(DS_K_MAJOR, DS_K_MAJOR, S, S, D, qkv, 3 * H, (int64_t)S * 3 * H, D, qkv + (size_t)H * esz, 3 * H,
                                  (int64_t)S * 3 * H, D, ws_base + ws_fscores, S, (int64_t)NH * S * S, (int64_t)S * S, DS_EPI_OUT_F32));
          // scale, mask adder, softmax (:500-518)
          DS_PROPAGATE(ds_softmax_fwd(dtype, B, NH, S, S, (const float*)(ws_base + ws_fscores), scale, mask, -10000.0f, p, stream));
          // ctx = P V (:533), written head-interleaved as [rows, H] (:536-542)
          return gemm_heads(DS_K_MAJOR, DS_MN_MAJOR, S, D, S, p, S, (int64_t)NH * S * S, (int64_t)S * S, qkv + (size_t)2 * H * esz, 3 * H,
                            (int64_t)S * 3 * H, D, ctx, H, (int64_t)S * H, D, 0);
        });
      }
      const int res32 = DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32 | DS_EPI_OUT_F32;  // fp32 stream: fp32 residual in, fp32 sum out
      float* xf = (float*)(ws_base + fw_xf[l & 1]);
      float* af = (float*)(ws_base + fw_af);
      // attention output dense + residual (:974-978), then layer_norm (:979)
      add_gemm(st, desc_fwd(rows, H, H, at(t.ctx, pos), weight_T(l, W_AO), at(t.z1, pos), DS_EPI_BIAS | (rs32 ? res32 : DS_EPI_RESIDUAL),
                            w[b + B_AO], rs32 ? (const void*)xf : (const void*)x, nullptr), prio);
      if (rs32) {
        add_ln_fwd(st, prio, (const float*)at(t.z1, pos), w[b + LN1_G], w[b + LN1_B], at(t.a, pos), af, (float*)(at(t.st1, pos)));
      } else {
        char *z1 = at(t.z1, pos), *a = at(t.a, pos), *st1 = at(t.st1, pos);
        add(st, [=]() { return ds_layernorm_fwd(dtype, rows, H, z1, w[b + LN1_G], w[b + LN1_B], cfg.ln_eps, a, (float*)st1, stream); });
      }
      // intermediate dense + gelu (:983-987)
      add_gemm(st, desc_fwd(rows, F, H, at(t.a, pos), weight_T(l, W_FF1), at(t.u, pos), DS_EPI_BIAS | DS_EPI_GELU | DS_EPI_GELU_GRAD,
                            w[b + B_FF1], nullptr, at(t.h, pos)), prio);
      // output dense + residual + layer_norm (:991-996)
      add_gemm(st, desc_fwd(rows, H, F, at(t.h, pos), weight_T(l, W_FF2), at(t.z2, pos), DS_EPI_BIAS | (rs32 ? res32 : DS_EPI_RESIDUAL),
                            w[b + B_FF2], rs32 ? (const void*)af : (const void*)at(t.a, pos), nullptr), prio);
      if (rs32) {
        add_ln_fwd(st, prio, (const float*)at(t.z2, pos), w[b + LN2_G], w[b + LN2_B], y,
                   l + 1 < L ? (float*)(ws_base + fw_xf[(l + 1) & 1]) : nullptr, (float*)(at(t.st2, pos)));
      } else {
        char *z2 = at(t.z2, pos), *st2 = at(t.st2, pos);
        add(st, [=]() { return ds_layernorm_fwd(dtype, rows, H, z2, w[b + LN2_G], w[b + LN2_B], cfg.ln_eps, y, (float*)st2, stream); });
      }
    }
    if (centred && L > 0) st.back().after = [this, pos]() { return sample_means(pos); };
    return DS_OK;
  }

  int release(int slot) override {
    if (G > 1) {  // the stash position goes back to the pool; nothing was deferred for it
      const int pos = slot_pos[slot];
      pos_owner[pos] = -1;
      x_bwd_valid[pos] = 0;
    }
    return DS_OK;
  }

  int backward(int slot, const void* d_out, void* d_in) override {
    ds_prio_scope prio(3);  // the chain every later pass waits on
    Steps st;
    DS_PROPAGATE(backward_steps(slot, d_out, d_in, st));
    return play(st);
  }

  // A forward pass (slot fslot) and a backward pass (slot bslot) of different micro-batches as one walk over both
  // chains on `stream`: the reference's graph leaves them unordered (bert/graph.py:126-132).
  int forward_backward(int fslot, const void* in, const float* key_mask, void* out, int bslot, const void* d_out, void* d_in) override {
    if (!groupable()) {
      {
        ds_prio_scope prio(1);
        Steps f;
        DS_PROPAGATE(forward_steps(fslot, in, key_mask, out, f));
        DS_PROPAGATE(play(f));
      }
      return backward(bslot, d_out, d_in);
    }
    Steps f, b;
    DS_PROPAGATE(forward_steps(fslot, in, key_mask, out, f));
    DS_PROPAGATE(backward_steps(bslot, d_out, d_in, b));
    return play_pair(f, b);
  }

  int backward_steps(int slot, const void* d_out, void* d_in, Steps& st) {
    const int prio = 3;
    const int pos = slot_pos[slot];
    char* sm = smallp(slot);
    const int dypos = (int)(n_backward % NDY);
    if (G > 1 && dy_wg_valid[dypos]) DS_CHECK_HIP(hipStreamWaitEvent(stream, ev_dy_wg[dypos], 0));
    const float scale = 1.0f / sqrtf((float)D);
    // With a weight-gradient stream the wgrad GEMMs and bias column sums of a layer run beside the
    // dgrad chain of the layers below it: they only feed the master gradients.
    hipStream_t ws = G > 1 ? nullptr : wgrad_stream;
    // Grouped weight gradients: the pass that completes a group issues the group's GEMMs layer by layer as its own
    // chain passes each layer, so that they run beside the chain of the layers below instead of after the pass.
    const bool closing = G > 1 && (int)deferred.size() + 1 >= G;
    std::shared_ptr<std::vector<Run>> runs = std::make_shared<std::vector<Run>>();
    hipStream_t gws = nullptr;
    if (closing) {
      std::vector<Deferred> all = deferred;
      all.push_back({pos, dypos});
      *runs = make_runs(all);
      gws = wgrad_stream ? wgrad_stream : stream;
    }
    if (ws || (gws && gws != stream)) DS_PROPAGATE(lane.ensure());
    // fp32 stream: the gradient that travels down the layers is fp32 (dyf); its bf16 copies feed the GEMMs
    const float* dyf = nullptr;
    if (rs32) {
      float* dst = (float*)(ws_base + bw_dxf[L & 1]);
      add(st, [=]() { return ds_cast_bf16_to_f32(dst, d_out, (size_t)rows * H, stream); });
      dyf = dst;
    }
    const char* dy = (const char*)d_out;
    for (int l = L - 1; l >= 0; --l) {
      const LayerStash& t = ls[l];
      const int b = base(l);
      const int par = l & 1;
      char* dz2 = G > 1 ? dy_base + ld[l].dz2 + dypos * dy_act : ws_base + ws_dz2[par];
      char* du = G > 1 ? dy_base + ld[l].du + dypos * dy_actF : ws_base + ws_du[par];
      char* da = ws_base + ws_da;
      char* dz1 = G > 1 ? dy_base + ld[l].dz1 + dypos * dy_act : ws_base + ws_dz1[par];
      char* dctx = ws_base + ws_dctx;
      char* dqkv = G > 1 ? dy_base + ld[l].dqkv + dypos * 3 * dy_act : ws_base + ws_dqkv[par];
      float* dp = (float*)(ws_base + ws_scores);
      char* dsm = ws_base + ws_ds;
      const int res32 = DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32 | DS_EPI_OUT_F32;
      float* dz2f = (float*)(ws_base + bw_dz2f);
      float* daf = (float*)(ws_base + bw_daf);
      float* dz1f = (float*)(ws_base + bw_dz1f);
      const float* z2 = (const float*)at(t.z2, pos);
      const float* z1 = (const float*)at(t.z1, pos);
      const float* st2 = (const float*)(at(t.st2, pos));
      const float* st1 = (const float*)(at(t.st1, pos));
      // output LayerNorm; the column sums of dz2 are the gradient of output/dense/bias
      // (fp32 stream with grouped weight gradients: the chain only computes dz; gamma, beta and bias gradients follow
      // with the group's weight gradients, from bf16 copies of dy kept beside dz in the operand ring)
      const bool ln_deferred = rs32 && G > 1;
      Step* first_step;
      if (ln_deferred) {
        first_step = &add_ln_bwd_rows(st, prio, dyf, z2, w[b + LN2_G], st2, dz2, dz2f, (float*)(dy_base + ld[l].dyn2 + dypos * dy_act32),
                                      (float*)(dy_base + ld[l].rs2 + (size_t)dypos * rows * 8));
      } else if (rs32) {
        const float* dyin = dyf;
        first_step = &add(st, [=]() {
          return ds_layernorm_bwd_mixed(rows, H, dyin, z2, w[b + LN2_G], st2, dz2, dz2f, nullptr, g[b + LN2_G], g[b + LN2_B], g[b + B_FF2], stream);
        });
      } else {
        const char* dyin = dy;
        first_step = &add(st, [=]() {
          return ds_layernorm_bwd(dtype, rows, H, dyin, z2, w[b + LN2_G], st2, nullptr, dz2, g[b + LN2_G], g[b + LN2_B], g[b + B_FF2], stream);
        });
      }
      // the wgrads that read this parity's buffers two layers up must have run
      if (ws) first_step->before = [this, par]() { return lane.reuse(stream, par); };
      // du = (dz2 W2^T) * gelu'(u)
      add_gemm(st, desc_dgrad(rows, H, F, dz2, weight_T(l, W_FF2), du, DS_EPI_MUL, nullptr, at(t.u, pos)), prio);
      // da = du W1^T + dz2 (a also feeds the residual into z2)
      if (rs32) add_gemm(st, desc_dgrad(rows, F, H, du, weight_T(l, W_FF1), daf, res32, dz2f, nullptr), prio);
      else add_gemm(st, desc_dgrad(rows, F, H, du, weight_T(l, W_FF1), da, DS_EPI_RESIDUAL, dz2, nullptr), prio);
      // attention-output LayerNorm; column sums of dz1 = gradient of attention/output/dense/bias
      if (ln_deferred) {
        add_ln_bwd_rows(st, prio, daf, z1, w[b + LN1_G], st1, dz1, dz1f, (float*)(dy_base + ld[l].dyn1 + dypos * dy_act32),
                        (float*)(dy_base + ld[l].rs1 + (size_t)dypos * rows * 8));
      } else if (rs32) {
        add(st, [=]() {
          return ds_layernorm_bwd_mixed(rows, H, daf, z1, w[b + LN1_G], st1, dz1, dz1f, nullptr, g[b + LN1_G], g[b + LN1_B], g[b + B_AO], stream);
        });
      } else {
        add(st, [=]() {
          return ds_layernorm_bwd(dtype, rows, H, da, z1, w[b + LN1_G], st1, nullptr, dz1, g[b + LN1_G], g[b + LN1_B], g[b + B_AO], stream);
        });
      }
      // d ctx = dz1 Wo^T; as a task of a grouped launch it also leaves delta = rowsum(d ctx * ctx) per head, which lets the
      // two attention-backward kernels run side by side (alone, the dQ kernel computes delta and the dK/dV kernel waits for it)
      {
        Step& s = add_gemm(st, desc_dgrad(rows, H, H, dz1, weight_T(l, W_AO), dctx, 0, nullptr, nullptr), prio);
        if (s.nops) {
          s.ops[0].gemm.c2 = at(t.ctx, pos);
          s.ops[0].rowdot = dp;
          s.ops[0].rowdot_seq = S;
        }
      }
      // attention backward per (batch, head)
      const char* q = at(t.qkv, pos);
      const char* k = q + (size_t)H * esz;
      const char* v = q + (size_t)2 * H * esz;
      const int64_t so3 = (int64_t)S * 3 * H, soH = (int64_t)S * H, soP = (int64_t)NH * S * S, siP = (int64_t)S * S;
      Step* attn_step;
      if (fused_attn) {
        const float* mask = slot_has_mask[slot] ? (const float*)(sm + mask_off) : nullptr;
        char* ctx = at(t.ctx, pos);
        const float* lse = (const float*)(at(t.lse, pos));
        const float* kbar = centre_q ? (const float*)at(t.kbar, pos) : nullptr;
        attn_step = &add(st, [=]() {
          return ds_attention_bwd_centered(dtype, B, NH, S, D, q, 3 * H, mask, scale, -10000.0f, ctx, lse, dctx, dqkv, dp, kbar, stream);
        });
        if (groupable()) {
          attn_step->nops = 2;
          attn_op(attn_step->ops[0], GOP_ATTN_DKV, prio, q, mask, ctx, (float*)lse, dctx, dqkv, dp);
          attn_op(attn_step->ops[1], GOP_ATTN_DQ, prio, q, mask, ctx, (float*)lse, dctx, dqkv, nullptr);
          attn_step->ops[1].key_mean = kbar;
        }
      } else {
        char* p = at(t.p, pos);
        attn_step = &add(st, [=]() {
          // dP = dctx V^T (fp32)
          DS_PROPAGATE(gemm_heads(DS_K_MAJOR, DS_K_MAJOR, S, S, D, dctx, H, soH, D, v, 3 * H, so3, D, dp, S, soP, siP, DS_EPI_OUT_F32));
          // dV = P^T dctx
          DS_PROPAGATE(gemm_heads(DS_MN_MAJOR, DS_MN_MAJOR, S, D, S, p, S, soP, siP, dctx, H, soH, D, dqkv + (size_t)2 * H * esz, 3 * H, so3, D, 0));
          // dS = scale * P * (dP - rowsum(dP * P))
          DS_PROPAGATE(ds_softmax_bwd(dtype, (int64_t)B * NH * S, S, p, dp, scale, dsm, stream));
          // dQ = dS K ; dK = dS^T Q
          DS_PROPAGATE(gemm_heads(DS_K_MAJOR, DS_MN_MAJOR, S, D, S, dsm, S, soP, siP, k, 3 * H, so3, D, dqkv, 3 * H, so3, D, 0));
          return gemm_heads(DS_MN_MAJOR, DS_MN_MAJOR, S, D, S, dsm, S, soP, siP, q, 3 * H, so3, D, dqkv + (size_t)H * esz, 3 * H, so3, D, 0);
        });
      }
      // ---- weight gradients of this layer (on the weight-gradient stream when there is one)
      if (G == 1) {
        const char *x = at(t.x, pos), *ctx = at(t.ctx, pos), *a = at(t.a, pos), *h = at(t.h, pos);
        const float* xbar = centred ? (const float*)at(t.xbar, pos) : nullptr;
        attn_step->after = [=]() {
          hipStream_t chain = stream;
          if (ws) {
            DS_PROPAGATE(lane.begin(chain, ws, par));
            stream = ws;  // the GEMMs and column sums of layer_wgrad launch on `stream`
          }
          const int rc = layer_wgrad(l, rows, x, xbar, ctx, a, h, dz2, du, dz1, dqkv);
          stream = chain;
          if (rc != DS_OK) return rc;
          if (ws) DS_PROPAGATE(lane.end(ws, par));
          return (int)DS_OK;
        };
      } else if (closing) {
        attn_step->after = [=]() {
          hipStream_t chain = stream;
          hipStream_t side = wgrad_stream ? wgrad_stream : chain;
          if (side != chain) DS_PROPAGATE(lane.begin(chain, side, par));
          stream = side;
          const int rc = layer_wgrad_runs(l, *runs);
          stream = chain;
          return rc;
        };
      }
      // dx = dqkv Wqkv^T + dz1 (x also feeds the residual into z1)
      const bool first = (l == 0);
      if (first && !emb && d_in == nullptr) break;  // a first stage takes no input gradient
      char* dx = first ? (emb ? ws_base + ws_dx[0] : (char*)d_in) : ws_base + ws_dx[l & 1];
      if (rs32 && !first) {
        float* dxf = (float*)(ws_base + bw_dxf[l & 1]);
        add_gemm(st, desc_dgrad(rows, 3 * H, H, dqkv, wqkv[l], dxf, res32, dz1f, nullptr), prio);
        dyf = dxf;
      } else if (rs32) {  // the stage's input gradient leaves as bf16
        add_gemm(st, desc_dgrad(rows, 3 * H, H, dqkv, wqkv[l], dx, DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32, dz1f, nullptr), prio);
      } else {
        add_gemm(st, desc_dgrad(rows, 3 * H, H, dqkv, wqkv[l], dx, DS_EPI_RESIDUAL, dz1, nullptr), prio);
      }
      dy = dx;
    }
    // the stash slot and the master gradients are released to the caller in the order of `stream`
    const char* dy_last = dy;
    add(st, [=]() {
      if (ws) DS_PROPAGATE(lane.finish(stream));
      if (G > 1) {
        deferred.push_back({pos, dypos});
        pos_deferred[pos] = 1;
        pos_owner[pos] = -1;
        ++n_backward;
      }
      if (emb) {
        // embedding LayerNorm backward, then scatter-add into the three tables
        char* de = ws_base + ws_dz2[0];
        DS_PROPAGATE(ds_layernorm_bwd(dtype, rows, H, dy_last, at(emb_e, pos), w[E_LN_G], (const float*)(at(emb_st, pos)), nullptr, de,
                                      g[E_LN_G], g[E_LN_B], nullptr, stream));
        const int32_t* tt = slot_has_tt[slot] ? (const int32_t*)(sm + emb_tt) : nullptr;
        dim3 grid((rows + 3) / 4);
        if (dtype == DS_BF16)
          hipLaunchKernelGGL(embed_bwd_kernel<bf16>, grid, dim3(256), 0, stream, rows, H, S, cfg.vocab, cfg.type_vocab,
                             (const int32_t*)(sm + emb_ids), tt, (const bf16*)de, g[E_WORD], g[E_TYPE], g[E_POS]);
        else
          hipLaunchKernelGGL(embed_bwd_kernel<float>, grid, dim3(256), 0, stream, rows, H, S, cfg.vocab, cfg.type_vocab,
                             (const int32_t*)(sm + emb_ids), tt, (const float*)de, g[E_WORD], g[E_TYPE], g[E_POS]);
        DS_CHECK_LAUNCH();
      }
      if (G > 1 && centre_k) DS_PROPAGATE(key_gradient_sums(dypos));
      if (G > 1) {
        if (bwd_stream) {
          DS_CHECK_HIP(hipEventRecord(ev_x_bwd[pos], stream));
          x_bwd_valid[pos] = 1;
        } else {
          x_bwd_valid[pos] = 0;
        }
        if (closing) {
          hipStream_t side = wgrad_stream ? wgrad_stream : stream;
          {
            hipStream_t chain = stream;
            stream = side;
            const int rc = launch_pending_wgrads();
            stream = chain;
            if (rc != DS_OK) return rc;
          }
          if (centre_k) {
            hipStream_t chain = stream;
            if (side != chain) {  // the key-gradient sums this pass has just queued
              DS_CHECK_HIP(hipEventRecord(ev_chain, chain));
              DS_CHECK_HIP(hipStreamWaitEvent(side, ev_chain, 0));
            }
            stream = side;
            const int rc = key_corrections(*runs);
            stream = chain;
            if (rc != DS_OK) return rc;
          }
          DS_PROPAGATE(retire_deferred(side, stream));
        }
      }
      return (int)DS_OK;
    });
    return DS_OK;
  }

  // runs of micro-batches that sit back to back in both rings: one set of GEMMs per run
  static std::vector<Run> make_runs(const std::vector<Deferred>& d) {
    std::vector<Run> runs;
    size_t i = 0;
    while (i < d.size()) {
      size_t j = i + 1;
      while (j < d.size() && d[j].xpos == d[j - 1].xpos + 1 && d[j].dypos == d[j - 1].dypos + 1) ++j;
      runs.push_back({d[i].xpos, d[i].dypos, (int)(j - i)});
      i = j;
    }
    return runs;
  }
  // Deferred weight gradients: per sample, the column sums of the key gradients a backward pass left in the operand ring,
  // all layers in one launch at the end of the pass; and, when the group's GEMMs have been queued, the centring of the
  // key projections' parameter gradients (see layer_wgrad) for all layers in one launch per run.
  int key_gradient_sums(int dypos) {
    std::vector<const void*> xs;
    std::vector<int64_t> lds(L, 3 * H);
    std::vector<float> scales(L, 1.0f);
    std::vector<float*> outs;
    for (int l = 0; l < L; ++l) {
      xs.push_back(dy_base + ld[l].dqkv + (size_t)dypos * 3 * dy_act + (size_t)H * esz);
      outs.push_back((float*)(dy_base + ld[l].dksum + (size_t)dypos * B * H * 4));
    }
    return ds_sample_colsum_multi(L, B, S, H, xs.data(), lds.data(), scales.data(), outs.data(), stream);
  }
  int key_corrections(const std::vector<Run>& runs) {
    for (const Run& r : runs) {
      std::vector<const float*> as, bs;
      std::vector<float*> ws, vs;
      for (int l = 0; l < L; ++l) {
        as.push_back((const float*)at(ls[l].xbar, r.xpos));
        bs.push_back((const float*)(dy_base + ld[l].dksum + (size_t)r.dypos * B * H * 4));
        ws.push_back(g[base(l) + W_K]);
        vs.push_back(g[base(l) + B_K]);
      }
      DS_PROPAGATE(ds_rank_update_multi(L, H, H, r.n * B, as.data(), bs.data(), ws.data(), H, vs.data(), stream));
    }
    return DS_OK;
  }
  // weight-gradient GEMMs collected for one grouped launch (on `stream`, the stream they were collected for)
  std::vector<GroupOp> wg_pending;
  int launch_pending_wgrads() {
    if (wg_pending.empty()) return DS_OK;
    const int rc = ds_group_launch(wg_pending.data(), (int)wg_pending.size(), stream);
    wg_pending.clear();
    return rc;
  }
  int layer_wgrad_runs(int l, const std::vector<Run>& runs) {
    const LayerStash& t = ls[l];
    const int b = base(l);
    for (const Run& r : runs) {
      const int m = r.n * rows;
      const char* dz2 = dy_base + ld[l].dz2 + r.dypos * dy_act;
      const char* dz1 = dy_base + ld[l].dz1 + r.dypos * dy_act;
      DS_PROPAGATE(layer_wgrad(l, m, at(t.x, r.xpos), centred ? (const float*)at(t.xbar, r.xpos) : nullptr, at(t.ctx, r.xpos), at(t.a, r.xpos),
                               at(t.h, r.xpos), dz2,
                               dy_base + ld[l].du + r.dypos * dy_actF, dz1, dy_base + ld[l].dqkv + r.dypos * 3 * dy_act));
      if (rs32) {  // the LayerNorm parameter gradients and the two bias gradients the chain left out, from its fp32 hand-over
        DS_PROPAGATE(ds_layernorm_param_grads_exact(m, H, (const float*)(dy_base + ld[l].dyn2 + r.dypos * dy_act32), (const float*)at(t.z2, r.xpos),
                                                    w[b + LN2_G], (const float*)at(t.st2, r.xpos),
                                                    (const float*)(dy_base + ld[l].rs2 + (size_t)r.dypos * rows * 8), g[b + LN2_G], g[b + LN2_B],
                                                    g[b + B_FF2], stream));
        DS_PROPAGATE(ds_layernorm_param_grads_exact(m, H, (const float*)(dy_base + ld[l].dyn1 + r.dypos * dy_act32), (const float*)at(t.z1, r.xpos),
                                                    w[b + LN1_G], (const float*)at(t.st1, r.xpos),
                                                    (const float*)(dy_base + ld[l].rs1 + (size_t)r.dypos * rows * 8), g[b + LN1_G], g[b + LN1_B],
                                                    g[b + B_AO], stream));
      }
    }
    return DS_OK;
  }
  // the weight-gradient work of every deferred pass has been queued on `ws`
  int retire_deferred(hipStream_t ws, hipStream_t chain) {
    for (const Deferred& e : deferred) {
      if (ws != chain) {
        DS_CHECK_HIP(hipEventRecord(ev_x_wg[e.xpos], ws));
        DS_CHECK_HIP(hipEventRecord(ev_dy_wg[e.dypos], ws));
      }
      x_wg_valid[e.xpos] = dy_wg_valid[e.dypos] = ws != chain;
      pos_deferred[e.xpos] = 0;
    }
    deferred.clear();
    if (ws != chain) wg_outstanding = true;
    return DS_OK;
  }

  // Weight and bias gradients of layer l over m rows (one micro-batch, or several back to back), on `stream`.
  int layer_wgrad(int l, int m, const char* x, const float* xbar, const char* ctx, const char* a, const char* h, const char* dz2,
                  const char* du, const char* dz1, const char* dqkv) {
    const int b = base(l);
    ds_prio_scope prio(0);  // feeds only the master gradients
    // projection gradients: three [H,H] kernels and three biases fed by the columns of dqkv
    const bool adjacent = g[b + B_K] == g[b + B_Q] + H && g[b + B_V] == g[b + B_Q] + 2 * H &&
                          g[b + W_K] == g[b + W_Q] + (size_t)H * H && g[b + W_V] == g[b + W_Q] + (size_t)2 * H * H;
    // Long reductions (several micro-batches' rows per weight): the layer's four weight-gradient GEMMs are independent, so
    // one launch carries all their 256 x 128 tiles - no hand-over between them, their tails fill each other - and, with
    // deferred weight gradients, those of two layers (measured on the BERT-48 half-stage: 40.25 -> 38.3 ms per step with
    // all 8 micro-batches in one group).  DS_BERT_GROUP_WGRAD = -1 switches it off, 0..5 forces a tile shape.
    static const char* env_gw = getenv("DS_BERT_GROUP_WGRAD");
    const int group_cfg = env_gw ? atoi(env_gw) : (m >= 2048 ? 1 : -1);
    if (group_cfg >= 0 && adjacent && dtype == DS_BF16 && m % 64 == 0 && m > 256 && H % 8 == 0 && F % 8 == 0) {
      GroupOp ops[4];
      ops[0].gemm = desc_wgrad(m, H, F, h, F, dz2, H, g[b + W_FF2], H);
      ops[1].gemm = desc_wgrad(m, F, H, a, H, du, F, g[b + W_FF1], F);
      ops[2].gemm = desc_wgrad(m, H, H, ctx, H, dz1, H, g[b + W_AO], H);
      ds_gemm_desc& d = ops[3].gemm;
      d = desc_wgrad(m, H, H, x, H, dqkv, 3 * H, g[b + W_Q], H);
      d.batch = 3; d.batch_inner = 3; d.b_stride_inner = H; d.c_stride_inner = (int64_t)H * H;
      // the two bias gradients that are column sums of a GEMM's dY operand come out of that GEMM (256x128 tiles only)
      static const char* env_cs = getenv("DS_BERT_GROUP_COLSUM");
      const bool fused_colsum = group_cfg == 1 && !(env_cs && atoi(env_cs) == 0);
      if (fused_colsum) {
        ops[1].colsum = g[b + B_FF1];
        ops[3].colsum = g[b + B_Q];
        ops[3].colsum_stride = H;
      }
      for (GroupOp& o : ops) { o.kind = GOP_GEMM; o.cfg = group_cfg; o.prio = 0; wg_pending.push_back(o); }
      static const char* env_gl = getenv("DS_BERT_GROUP_LAYERS");
      // (per-pass weight gradients hand their operand buffers back layer by layer: nothing is held over)
      const size_t per_launch = G > 1 && !(env_gl && atoi(env_gl) == 1) ? 8 : 4;
      if (wg_pending.size() >= per_launch) DS_PROPAGATE(launch_pending_wgrads());
      if (!fused_colsum) {
        DS_PROPAGATE(ds_colsum_accum(dtype, m, F, du, F, g[b + B_FF1], stream));
        DS_PROPAGATE(ds_colsum_accum(dtype, m, 3 * H, dqkv, 3 * H, g[b + B_Q], stream));
      }
      return DS_OK;
    }
    DS_PROPAGATE(gemm_wgrad(m, H, F, h, F, dz2, H, g[b + W_FF2], H));
    DS_PROPAGATE(ds_colsum_accum(dtype, m, F, du, F, g[b + B_FF1], stream));
    DS_PROPAGATE(gemm_wgrad(m, F, H, a, H, du, F, g[b + W_FF1], F));
    DS_PROPAGATE(gemm_wgrad(m, H, H, ctx, H, dz1, H, g[b + W_AO], H));
    if (adjacent) {
      // q, k, v master gradients lie back to back: one column sum over [m, 3H] and one GEMM batched
      // over the three column blocks of dqkv
      DS_PROPAGATE(ds_colsum_accum(dtype, m, 3 * H, dqkv, 3 * H, g[b + B_Q], stream));
      ds_gemm_desc d;
      memset(&d, 0, sizeof(d));
      d.dtype = dtype; d.a_major = DS_MN_MAJOR; d.b_major = DS_MN_MAJOR;
      d.m = H; d.n = H; d.k = m; d.lda = H; d.ldb = 3 * H; d.ldc = H; d.batch = 3; d.batch_inner = 3;
      d.b_stride_inner = H; d.c_stride_inner = (int64_t)H * H;
      d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.a = x; d.b = dqkv; d.c = g[b + W_Q];
      DS_PROPAGATE(ds_gemm(&d, stream));
    } else {
      for (int j = 0; j < 3; ++j) {
        DS_PROPAGATE(ds_colsum_accum(dtype, m, H, dqkv + (size_t)j * H * esz, 3 * H, g[b + B_Q + j], stream));
        DS_PROPAGATE(gemm_wgrad(m, H, H, x, H, dqkv + (size_t)j * H * esz, 3 * H, g[b + W_Q + j], H));
      }
    }
    if (centre_k && G == 1) {
      // The key gradients of a sample sum to zero per head (every row of dS does, and dK = dS^T Q adds the rows up), so
      // X^T dK only depends on the inputs' deviation from their per-sample mean and the key bias gets no gradient at all.
      // The stored dK are rounded to bf16 (from bf16-rounded dS) and sum to a residue instead; against inputs that share a
      // large common part, mean (x) residue is the bulk of the key kernel's gradient error.  The residue is known: the
      // parameter gradients are those of dK centred over each sample's keys - the mean's share goes out again.
      const int ns = m / S;
      float* dksum = (float*)(ws_base + ws_dksum);
      DS_PROPAGATE(ds_sample_colsum(ns, S, H, dqkv + (size_t)H * esz, 3 * H, 1.0f, dksum, stream));
      DS_PROPAGATE(ds_rank_update(H, H, ns, xbar, dksum, g[b + W_K], H, g[b + B_K], stream));
    }
    return DS_OK;
  }

  int flush_deferred(bool final) override {
    if (G <= 1) return DS_OK;
    hipStream_t chain = bwd_stream ? bwd_stream : stream;
    hipStream_t ws = wgrad_stream ? wgrad_stream : chain;
    if (!deferred.empty()) {
      if (ws != chain) {  // the operands the last backward pass wrote
        DS_CHECK_HIP(hipEventRecord(ev_chain, chain));
        DS_CHECK_HIP(hipStreamWaitEvent(ws, ev_chain, 0));
      }
      hipStream_t keep = stream;
      stream = ws;
      int rc = DS_OK;
      const std::vector<Run> runs = make_runs(deferred);
      for (int l = L - 1; l >= 0 && rc == DS_OK; --l) rc = layer_wgrad_runs(l, runs);
      if (rc == DS_OK) rc = launch_pending_wgrads();
      if (rc == DS_OK && centre_k) rc = key_corrections(runs);
      stream = keep;
      if (rc != DS_OK) return rc;
      DS_PROPAGATE(retire_deferred(ws, chain));
    }
    if (final && wg_outstanding) {
      DS_CHECK_HIP(hipEventRecord(ev_wg_done, wgrad_owned));
      DS_CHECK_HIP(hipStreamWaitEvent(chain, ev_wg_done, 0));
      wg_outstanding = false;
    }
    return DS_OK;
  }

  int set_token_types(int slot, const int32_t* tt) {
    if (!emb) { ds_set_error("ds_stage_set_token_types: stage has no embedding"); return DS_ESTATE; }
    if (tt) DS_CHECK_HIP(hipMemcpyAsync(smallp(slot) + emb_tt, tt, (size_t)rows * 4, hipMemcpyDeviceToDevice, stream));
    slot_has_tt[slot] = tt != nullptr;
    return DS_OK;
  }
};

}  // namespace

int ds_bert_stage_create(const ds_stage_cfg* c, hipStream_t stream, ds_stage** out) {
  DS_CHECK_ARG(c->dtype == DS_F32 || c->dtype == DS_BF16, "ds_stage_create: dtype %d", c->dtype);
  DS_CHECK_ARG(c->num_layers >= 0 && c->hidden > 0 && c->heads > 0 && c->ffn > 0 && c->batch > 0 && c->seq > 0,
               "ds_stage_create: non-positive shape");
  DS_CHECK_ARG(c->num_layers > 0 || c->with_embedding, "ds_stage_create: empty stage");
  DS_CHECK_ARG(c->hidden % c->heads == 0, "ds_stage_create: hidden size (%d) is not a multiple of the number of attention heads (%d)",
               c->hidden, c->heads);
  const int vec = c->dtype == DS_BF16 ? 8 : 4;
  const int d = c->hidden / c->heads;
  DS_CHECK_ARG(d % vec == 0 && c->seq % vec == 0 && c->hidden % vec == 0 && c->ffn % vec == 0,
               "ds_stage_create: head size %d, seq %d, hidden %d and ffn %d must be multiples of %d", d, c->seq, c->hidden, c->ffn, vec);
  DS_CHECK_ARG(c->seq <= 2048, "ds_stage_create: seq %d exceeds 2048", c->seq);
  DS_CHECK_ARG(c->hidden <= 64 * vec * 8, "ds_stage_create: hidden %d too large for the LayerNorm kernel", c->hidden);
  DS_CHECK_ARG(c->stash_slots >= 1, "ds_stage_create: stash_slots must be >= 1");
  if (c->with_embedding) {
    DS_CHECK_ARG(c->vocab > 0 && c->type_vocab > 0 && c->max_pos > 0, "ds_stage_create: embedding table sizes");
    DS_CHECK_ARG(c->seq <= c->max_pos, "ds_stage_create: The seq length (%d) cannot be greater than `max_position_embeddings` (%d)",
                 c->seq, c->max_pos);
  }
  BertStage* s = new BertStage();
  s->cfg = *c;
  s->stream = stream;
  const int rc = s->init();
  if (rc != DS_OK) { delete s; return rc; }
  *out = s;
  return DS_OK;
}

extern "C" int ds_stage_set_token_types(ds_stage* h, int slot, const int32_t* token_type_ids) {
  DS_CHECK_ARG(h != nullptr, "ds_stage_set_token_types: null handle");
  DS_CHECK_ARG(h->cfg.kind == DS_STAGE_BERT, "ds_stage_set_token_types: not a BERT stage");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_stage_set_token_types: slot %d out of range", slot);
  DS_PROPAGATE(ds_stage_acquire_slot(h, slot));
  return static_cast<BertStage*>(h)->set_token_types(slot, token_type_ids);
}
