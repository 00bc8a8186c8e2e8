// BERT pipeline stage: [embedding] + encoder layers, forward and hand-derived backward, with
// the weight gradients accumulated in place into the caller's fp32 master gradients.
//
// Follows bert/models/bert/modeling_slice.py of the reference: embedding_stage :794-821,
// encoder_layer :942-1001 (attention_layer :357-549, dense+residual+layer_norm, gelu FFN).
// Dropout is the identity (is_training=False zeroes it, :774-776).
#include <string.h>

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

struct LayerStash {  // byte offsets into a slot
  size_t x, qkv, p, ctx, z1, a, u, h, z2, st1, st2, lse;
};

struct BertStage : ds_stage {
  int L, H, F, NH, D, B, S, rows;
  int dtype;
  size_t esz;
  bool emb;
  bool fused_attn;  // bf16, head size 64: fused attention kernels, no [B,N,S,S] tensors at all
  // the forward pass writes its stash slot, its output and (unfused attention) its own score buffer; the rest
  // of the workspace belongs to backward
  bool overlap_safe() const override { return true; }
  // compute copies
  char* wc_base = nullptr;
  std::vector<char*> wqkv, wo, w1, w2;  // element type T
  std::vector<float*> bqkv;
  // stash
  char* stash_base = nullptr;
  size_t slot_bytes = 0;
  size_t emb_e = 0, emb_st = 0, emb_ids = 0, emb_tt = 0, mask_off = 0;
  std::vector<LayerStash> ls;
  size_t out_off = 0;  // last layer's y is written straight to the caller's buffer
  std::vector<char> slot_has_mask, slot_has_tt;
  // workspace
  char* ws_base = nullptr;
  size_t ws_bytes = 0;
  size_t ws_scores, ws_fscores, ws_ds, ws_dz2[2], ws_du[2], ws_da, ws_dz1[2], ws_dctx, ws_dqkv[2], ws_dx[2];
  WgradLane lane;

  ~BertStage() override {
    if (wc_base) (void)hipFree(wc_base);
    if (stash_base) (void)hipFree(stash_base);
    if (ws_base) (void)hipFree(ws_base);
  }
  int base(int l) const { return (emb ? EMB_NW : 0) + l * LAYER_NW; }
  char* slotp(int slot) const { return stash_base + (size_t)slot * slot_bytes; }

  int init() {
    const ds_stage_cfg& c = cfg;
    L = c.num_layers; H = c.hidden; F = c.ffn; NH = c.heads; B = c.batch; S = c.seq;
    D = H / NH; rows = B * S; dtype = c.dtype; esz = dtype == DS_BF16 ? 2 : 4; emb = c.with_embedding != 0;
    fused_attn = dtype == DS_BF16 && D == 64 && S % 64 == 0 && S <= 2048;
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
    // ---- stash layout of one slot
    Arena sa;
    const size_t act = (size_t)rows * H * esz, actF = (size_t)rows * F * esz;
    const size_t probs = (size_t)B * NH * S * S * esz, stats = (size_t)rows * 2 * 4;
    mask_off = sa.reserve((size_t)B * S * 4);
    if (emb) {
      emb_ids = sa.reserve((size_t)rows * 4);
      emb_tt = sa.reserve((size_t)rows * 4);
      emb_e = sa.reserve(act);
      emb_st = sa.reserve(stats);
    }
    ls.resize(L);
    size_t next_x = L ? sa.reserve(act) : 0;
    for (int l = 0; l < L; ++l) {
      LayerStash& t = ls[l];
      t.x = next_x;
      t.qkv = sa.reserve(3 * act);
      t.p = fused_attn ? 0 : sa.reserve(probs);
      t.lse = fused_attn ? sa.reserve((size_t)B * NH * S * 4) : 0;
      t.ctx = sa.reserve(act);
      t.z1 = sa.reserve(act);
      t.a = sa.reserve(act);
      t.u = sa.reserve(actF);
      t.h = sa.reserve(actF);
      t.z2 = sa.reserve(act);
      t.st1 = sa.reserve(stats);
      t.st2 = sa.reserve(stats);
      if (l + 1 < L) next_x = sa.reserve(act);
    }
    slot_bytes = sa.used;
    const int K = c.stash_slots;
    DS_CHECK_HIP(hipMalloc((void**)&stash_base, slot_bytes * K));
    slot_forwarded.assign(K, 0);
    slot_has_mask.assign(K, 0);
    slot_has_tt.assign(K, 0);
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
    ws_bytes = w.used;
    DS_CHECK_HIP(hipMalloc((void**)&ws_base, ws_bytes));
    return DS_OK;
  }

  size_t workspace_bytes() const override { return ws_bytes; }
  size_t stash_bytes(int slots) const override { return slot_bytes * (size_t)slots; }

  const void* weight_T(int l, int which) const {  // kernel in the element type
    if (dtype == DS_BF16) return which == W_AO ? wo[l] : (which == W_FF1 ? w1[l] : w2[l]);
    return w[base(l) + which];
  }

  int refresh_weights() override {
    for (int l = 0; l < L; ++l) {
      const int b = base(l);
      if (dtype == DS_BF16) {
        hipLaunchKernelGGL(pack_qkv_kernel<bf16>, dim3(1024), dim3(256), 0, stream, H, w[b + W_Q], w[b + W_K], w[b + W_V],
                           w[b + B_Q], w[b + B_K], w[b + B_V], (bf16*)wqkv[l], bqkv[l]);
        DS_CHECK_LAUNCH();
        DS_PROPAGATE(ds_cast_f32_to_bf16(wo[l], w[b + W_AO], (size_t)H * H, stream));
        DS_PROPAGATE(ds_cast_f32_to_bf16(w1[l], w[b + W_FF1], (size_t)H * F, stream));
        DS_PROPAGATE(ds_cast_f32_to_bf16(w2[l], w[b + W_FF2], (size_t)F * H, stream));
      } else {
        hipLaunchKernelGGL(pack_qkv_kernel<float>, dim3(1024), dim3(256), 0, stream, H, w[b + W_Q], w[b + W_K], w[b + W_V],
                           w[b + B_Q], w[b + B_K], w[b + B_V], (float*)wqkv[l], bqkv[l]);
        DS_CHECK_LAUNCH();
      }
    }
    return DS_OK;
  }

  // C[rows_m, n] = A[rows_m, k] (K-major) x W[k, n] (MN-major) with an epilogue
  int gemm_fwd(int m, int n, int k, const void* a, const void* wt, void* c, int flags, const float* bias,
               const void* residual, void* c2) {
    ds_gemm_desc d;
    memset(&d, 0, sizeof(d));
    d.dtype = dtype; d.a_major = DS_K_MAJOR; d.b_major = DS_MN_MAJOR;
    d.m = m; d.n = n; d.k = k; d.lda = k; d.ldb = n; d.ldc = n; d.batch = 1; d.batch_inner = 1;
    d.flags = flags; d.alpha = 1.f; d.a = a; d.b = wt; d.c = c; d.bias = bias; d.residual = residual; d.c2 = c2;
    return ds_gemm(&d, stream);
  }
  // dX[m, k] = dY[m, n] x W[k, n]^T (+ residual) (* gelu'(aux))
  int gemm_dgrad(int m, int n, int k, const void* dy, const void* wt, void* dx, int flags, const void* residual, void* aux) {
    ds_gemm_desc d;
    memset(&d, 0, sizeof(d));
    d.dtype = dtype; d.a_major = DS_K_MAJOR; d.b_major = DS_K_MAJOR;
    d.m = m; d.n = k; d.k = n; d.lda = n; d.ldb = n; d.ldc = k; d.batch = 1; d.batch_inner = 1;
    d.flags = flags; d.alpha = 1.f; d.a = dy; d.b = wt; d.c = dx; d.residual = residual; d.c2 = aux;
    return ds_gemm(&d, stream);
  }
  // dW[k, n] (fp32) += X[m, k]^T x dY[m, n]
  int gemm_wgrad(int m, int n, int k, const void* x, int64_t ldx, const void* dy, int64_t ldy, float* dw, int64_t lddw) {
    ds_gemm_desc d;
    memset(&d, 0, sizeof(d));
    d.dtype = dtype; d.a_major = DS_MN_MAJOR; d.b_major = DS_MN_MAJOR;
    d.m = k; d.n = n; d.k = m; d.lda = ldx; d.ldb = ldy; d.ldc = lddw; d.batch = 1; d.batch_inner = 1;
    d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.a = x; d.b = dy; d.c = dw;
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

  int forward(int slot, const void* in, const float* key_mask, void* out) override {
    char* sp = slotp(slot);
    const size_t act = (size_t)rows * H * esz;
    const float scale = 1.0f / sqrtf((float)D);
    const float* mask = nullptr;
    if (key_mask) {
      DS_CHECK_HIP(hipMemcpyAsync(sp + mask_off, key_mask, (size_t)B * S * 4, hipMemcpyDeviceToDevice, stream));
      mask = (const float*)(sp + mask_off);
    }
    slot_has_mask[slot] = key_mask != nullptr;
    char* x0 = L ? sp + ls[0].x : nullptr;
    if (emb) {
      DS_CHECK_HIP(hipMemcpyAsync(sp + emb_ids, in, (size_t)rows * 4, hipMemcpyDeviceToDevice, stream));
      const int32_t* tt = slot_has_tt[slot] ? (const int32_t*)(sp + emb_tt) : nullptr;
      dim3 grid((rows + 3) / 4);
      if (dtype == DS_BF16)
        hipLaunchKernelGGL(embed_fwd_kernel<bf16>, grid, dim3(256), 0, stream, rows, H, S, cfg.vocab, cfg.type_vocab,
                           (const int32_t*)(sp + emb_ids), tt, w[E_WORD], w[E_TYPE], w[E_POS], (bf16*)(sp + emb_e));
      else
        hipLaunchKernelGGL(embed_fwd_kernel<float>, grid, dim3(256), 0, stream, rows, H, S, cfg.vocab, cfg.type_vocab,
                           (const int32_t*)(sp + emb_ids), tt, w[E_WORD], w[E_TYPE], w[E_POS], (float*)(sp + emb_e));
      DS_CHECK_LAUNCH();
      DS_PROPAGATE(ds_layernorm_fwd(dtype, rows, H, sp + emb_e, w[E_LN_G], w[E_LN_B], cfg.ln_eps, L ? (void*)x0 : out,
                                    (float*)(sp + emb_st), stream));
    } else {
      DS_CHECK_HIP(hipMemcpyAsync(x0, in, act, hipMemcpyDeviceToDevice, stream));
    }
    for (int l = 0; l < L; ++l) {
      const LayerStash& t = ls[l];
      const int b = base(l);
      char* x = sp + t.x;
      char* y = (l + 1 < L) ? sp + ls[l + 1].x : (char*)out;
      // fused Q|K|V projection (modeling_slice.py:464-485)
      DS_PROPAGATE(gemm_fwd(rows, 3 * H, H, x, wqkv[l], sp + t.qkv, DS_EPI_BIAS, bqkv[l], nullptr, nullptr));
      if (fused_attn) {
        // scores, scale, mask adder, softmax and context in one kernel (:499-533)
        DS_PROPAGATE(ds_attention_fwd(dtype, B, NH, S, D, sp + t.qkv, 3 * H, mask, scale, -10000.0f, sp + t.ctx,
                                      (float*)(sp + t.lse), stream));
      } else {
      // scores = Q K^T (:499), fp32
      DS_PROPAGATE(gemm_heads(DS_K_MAJOR, DS_K_MAJOR, S, S, D, sp + t.qkv, 3 * H, (int64_t)S * 3 * H, D,
                              sp + t.qkv + (size_t)H * esz, 3 * H, (int64_t)S * 3 * H, D, ws_base + ws_fscores, S,
                              (int64_t)NH * S * S, (int64_t)S * S, DS_EPI_OUT_F32));
      // scale, mask adder, softmax (:500-518)
      DS_PROPAGATE(ds_softmax_fwd(dtype, B, NH, S, S, (const float*)(ws_base + ws_fscores), scale, mask, -10000.0f,
                                  sp + t.p, stream));
      // ctx = P V (:533), written head-interleaved as [rows, H] (:536-542)
      DS_PROPAGATE(gemm_heads(DS_K_MAJOR, DS_MN_MAJOR, S, D, S, sp + t.p, S, (int64_t)NH * S * S, (int64_t)S * S,
                              sp + t.qkv + (size_t)2 * H * esz, 3 * H, (int64_t)S * 3 * H, D, sp + t.ctx, H,
                              (int64_t)S * H, D, 0));
      }
      // attention output dense + residual (:974-978), then layer_norm (:979)
      DS_PROPAGATE(gemm_fwd(rows, H, H, sp + t.ctx, weight_T(l, W_AO), sp + t.z1, DS_EPI_BIAS | DS_EPI_RESIDUAL,
                            w[b + B_AO], x, nullptr));
      DS_PROPAGATE(ds_layernorm_fwd(dtype, rows, H, sp + t.z1, w[b + LN1_G], w[b + LN1_B], cfg.ln_eps, sp + t.a,
                                    (float*)(sp + t.st1), stream));
      // intermediate dense + gelu (:983-987)
      DS_PROPAGATE(gemm_fwd(rows, F, H, sp + t.a, weight_T(l, W_FF1), sp + t.u, DS_EPI_BIAS | DS_EPI_GELU | DS_EPI_GELU_GRAD, w[b + B_FF1],
                            nullptr, sp + t.h));
      // output dense + residual + layer_norm (:991-996)
      DS_PROPAGATE(gemm_fwd(rows, H, F, sp + t.h, weight_T(l, W_FF2), sp + t.z2, DS_EPI_BIAS | DS_EPI_RESIDUAL,
                            w[b + B_FF2], sp + t.a, nullptr));
      DS_PROPAGATE(ds_layernorm_fwd(dtype, rows, H, sp + t.z2, w[b + LN2_G], w[b + LN2_B], cfg.ln_eps, y,
                                    (float*)(sp + t.st2), stream));
    }
    return DS_OK;
  }

  int backward(int slot, const void* d_out, void* d_in) override {
    char* sp = slotp(slot);
    const float scale = 1.0f / sqrtf((float)D);
    const char* dy = (const char*)d_out;
    // With a weight-gradient stream the wgrad GEMMs and bias column sums of a layer run beside the
    // dgrad chain of the layers below it: they only feed the master gradients.
    hipStream_t ws = wgrad_stream;
    if (ws) DS_PROPAGATE(lane.ensure());
    for (int l = L - 1; l >= 0; --l) {
      const LayerStash& t = ls[l];
      const int b = base(l);
      const int par = l & 1;
      char* dz2 = ws_base + ws_dz2[par];
      char* du = ws_base + ws_du[par];
      char* da = ws_base + ws_da;
      char* dz1 = ws_base + ws_dz1[par];
      char* dctx = ws_base + ws_dctx;
      char* dqkv = ws_base + ws_dqkv[par];
      float* dp = (float*)(ws_base + ws_scores);
      char* dsm = ws_base + ws_ds;
      // the wgrads that read this parity's buffers two layers up must have run
      if (ws) DS_PROPAGATE(lane.reuse(stream, par));
      // output LayerNorm; the column sums of dz2 are the gradient of output/dense/bias
      DS_PROPAGATE(ds_layernorm_bwd(dtype, rows, H, dy, sp + t.z2, w[b + LN2_G], (const float*)(sp + t.st2), nullptr, dz2,
                                    g[b + LN2_G], g[b + LN2_B], g[b + B_FF2], stream));
      // du = (dz2 W2^T) * gelu'(u)
      DS_PROPAGATE(gemm_dgrad(rows, H, F, dz2, weight_T(l, W_FF2), du, DS_EPI_MUL, nullptr, sp + t.u));
      // da = du W1^T + dz2 (a also feeds the residual into z2)
      DS_PROPAGATE(gemm_dgrad(rows, F, H, du, weight_T(l, W_FF1), da, DS_EPI_RESIDUAL, dz2, nullptr));
      // attention-output LayerNorm; column sums of dz1 = gradient of attention/output/dense/bias
      DS_PROPAGATE(ds_layernorm_bwd(dtype, rows, H, da, sp + t.z1, w[b + LN1_G], (const float*)(sp + t.st1), nullptr, dz1,
                                    g[b + LN1_G], g[b + LN1_B], g[b + B_AO], stream));
      DS_PROPAGATE(gemm_dgrad(rows, H, H, dz1, weight_T(l, W_AO), dctx, 0, nullptr, nullptr));
      // attention backward per (batch, head)
      const char* q = sp + t.qkv;
      const char* k = q + (size_t)H * esz;
      const char* v = q + (size_t)2 * H * esz;
      const int64_t so3 = (int64_t)S * 3 * H, soH = (int64_t)S * H, soP = (int64_t)NH * S * S, siP = (int64_t)S * S;
      if (fused_attn) {
        const float* mask = slot_has_mask[slot] ? (const float*)(sp + mask_off) : nullptr;
        DS_PROPAGATE(ds_attention_bwd(dtype, B, NH, S, D, q, 3 * H, mask, scale, -10000.0f, sp + t.ctx, (const float*)(sp + t.lse),
                                      dctx, dqkv, dp, stream));
      } else {
      // dP = dctx V^T (fp32)
      DS_PROPAGATE(gemm_heads(DS_K_MAJOR, DS_K_MAJOR, S, S, D, dctx, H, soH, D, v, 3 * H, so3, D, dp, S, soP, siP,
                              DS_EPI_OUT_F32));
      // dV = P^T dctx
      DS_PROPAGATE(gemm_heads(DS_MN_MAJOR, DS_MN_MAJOR, S, D, S, sp + t.p, S, soP, siP, dctx, H, soH, D,
                              dqkv + (size_t)2 * H * esz, 3 * H, so3, D, 0));
      // dS = scale * P * (dP - rowsum(dP * P))
      DS_PROPAGATE(ds_softmax_bwd(dtype, (int64_t)B * NH * S, S, sp + t.p, dp, scale, dsm, stream));
      // dQ = dS K ; dK = dS^T Q
      DS_PROPAGATE(gemm_heads(DS_K_MAJOR, DS_MN_MAJOR, S, D, S, dsm, S, soP, siP, k, 3 * H, so3, D, dqkv, 3 * H, so3, D, 0));
      DS_PROPAGATE(gemm_heads(DS_MN_MAJOR, DS_MN_MAJOR, S, D, S, dsm, S, soP, siP, q, 3 * H, so3, D,
                              dqkv + (size_t)H * esz, 3 * H, so3, D, 0));
      }
      // ---- weight gradients of this layer (on the weight-gradient stream when there is one)
      hipStream_t chain = stream;
      if (ws) {
        DS_PROPAGATE(lane.begin(chain, ws, par));
        stream = ws;  // gemm_wgrad and the column sums below launch on `stream`
      }
      int rc = DS_OK;
      do {
        if ((rc = gemm_wgrad(rows, H, F, sp + t.h, F, dz2, H, g[b + W_FF2], H)) != DS_OK) break;
        if ((rc = ds_colsum_accum(dtype, rows, F, du, F, g[b + B_FF1], stream)) != DS_OK) break;
        if ((rc = gemm_wgrad(rows, F, H, sp + t.a, H, du, F, g[b + W_FF1], F)) != DS_OK) break;
        if ((rc = gemm_wgrad(rows, H, H, sp + t.ctx, H, dz1, H, g[b + W_AO], H)) != DS_OK) break;
        // projection gradients: three [H,H] kernels and three biases fed by the columns of dqkv
        const bool adjacent = g[b + B_K] == g[b + B_Q] + H && g[b + B_V] == g[b + B_Q] + 2 * H &&
                              g[b + W_K] == g[b + W_Q] + (size_t)H * H && g[b + W_V] == g[b + W_Q] + (size_t)2 * H * H;
        if (adjacent) {
          // q, k, v master gradients lie back to back: one column sum over [rows, 3H] and one GEMM batched
          // over the three column blocks of dqkv
          if ((rc = ds_colsum_accum(dtype, rows, 3 * H, dqkv, 3 * H, g[b + B_Q], stream)) != DS_OK) break;
          ds_gemm_desc d;
          memset(&d, 0, sizeof(d));
          d.dtype = dtype; d.a_major = DS_MN_MAJOR; d.b_major = DS_MN_MAJOR;
          d.m = H; d.n = H; d.k = rows; d.lda = H; d.ldb = 3 * H; d.ldc = H; d.batch = 3; d.batch_inner = 3;
          d.b_stride_inner = H; d.c_stride_inner = (int64_t)H * H;
          d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.a = sp + t.x; d.b = dqkv; d.c = g[b + W_Q];
          if ((rc = ds_gemm(&d, stream)) != DS_OK) break;
        } else {
          for (int j = 0; j < 3 && rc == DS_OK; ++j) {
            rc = ds_colsum_accum(dtype, rows, H, dqkv + (size_t)j * H * esz, 3 * H, g[b + B_Q + j], stream);
            if (rc == DS_OK) rc = gemm_wgrad(rows, H, H, sp + t.x, H, dqkv + (size_t)j * H * esz, 3 * H, g[b + W_Q + j], H);
          }
        }
      } while (0);
      stream = chain;
      if (rc != DS_OK) return rc;
      if (ws) DS_PROPAGATE(lane.end(ws, par));
      // dx = dqkv Wqkv^T + dz1 (x also feeds the residual into z1)
      const bool first = (l == 0);
      if (first && !emb && d_in == nullptr) break;  // a first stage takes no input gradient
      char* dx = first ? (emb ? ws_base + ws_dx[0] : (char*)d_in) : ws_base + ws_dx[l & 1];
      DS_PROPAGATE(gemm_dgrad(rows, 3 * H, H, dqkv, wqkv[l], dx, DS_EPI_RESIDUAL, dz1, nullptr));
      dy = dx;
    }
    // the stash slot and the master gradients are released to the caller in the order of `stream`
    if (ws) DS_PROPAGATE(lane.finish(stream));
    if (emb) {
      // embedding LayerNorm backward, then scatter-add into the three tables
      char* de = ws_base + ws_dz2[0];
      DS_PROPAGATE(ds_layernorm_bwd(dtype, rows, H, dy, sp + emb_e, w[E_LN_G], (const float*)(sp + emb_st), nullptr, de,
                                    g[E_LN_G], g[E_LN_B], nullptr, stream));
      const int32_t* tt = slot_has_tt[slot] ? (const int32_t*)(sp + emb_tt) : nullptr;
      dim3 grid((rows + 3) / 4);
      if (dtype == DS_BF16)
        hipLaunchKernelGGL(embed_bwd_kernel<bf16>, grid, dim3(256), 0, stream, rows, H, S, cfg.vocab, cfg.type_vocab,
                           (const int32_t*)(sp + emb_ids), tt, (const bf16*)de, g[E_WORD], g[E_TYPE], g[E_POS]);
      else
        hipLaunchKernelGGL(embed_bwd_kernel<float>, grid, dim3(256), 0, stream, rows, H, S, cfg.vocab, cfg.type_vocab,
                           (const int32_t*)(sp + emb_ids), tt, (const float*)de, g[E_WORD], g[E_TYPE], g[E_POS]);
      DS_CHECK_LAUNCH();
    }
    return DS_OK;
  }

  int set_token_types(int slot, const int32_t* tt) {
    if (!emb) { ds_set_error("ds_stage_set_token_types: stage has no embedding"); return DS_ESTATE; }
    if (tt) DS_CHECK_HIP(hipMemcpyAsync(slotp(slot) + emb_tt, tt, (size_t)rows * 4, hipMemcpyDeviceToDevice, stream));
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
