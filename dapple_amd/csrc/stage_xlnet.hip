// XLNet pipeline stage: relative-position multi-head attention layers (content stream and, optionally,
// the query stream sharing keys/values/weights), with optional memory, forward and backward.
//
// Follows xlnet/layers/rel_multihead_attn.py:71-149 of the reference (einsums of _rel_attn_core and
// call), lambda_funcs.py:85-93 (rel_shift), position_wise_feed_forward.py:92-105, layer_normalization.py:
// 69-78 (eps 1e-14), activations/gelu.py:6-11 (tanh GELU) and the layer body of
// models/slice_xlnet.py:164-180.  The reference builds the content stream with memory length 0; memory
// (keys/values from concat(mem, h), positions klen .. -qlen+1) and the query stream follow the XLNet
// formulation those layers were transcribed from.
//
// Activations are sequence-major rows (stream, i, b) of width H.  Scores are never shifted in memory:
// the position term is computed unshifted as (q + r_r) k_r^T [qlen, rlen] and the softmax kernel reads
// column j + qlen - i of it (rel_shift as index arithmetic); backward scatters with the same map.
#include <stdlib.h>
#include <string.h>

#include "group.h"
#include "stage.h"

namespace {

enum XW { X_Q = 0, X_K, X_V, X_R, X_O, X_RW, X_RR, X_RS, X_SEG, X_LN1_G, X_LN1_B, X_W1, X_B1, X_W2, X_B2, X_LN2_G, X_LN2_B, X_NW };

// qw = q + r_w, qr = q + r_r, qs = q + r_s (biases broadcast over rows)
template <typename T>
__global__ __launch_bounds__(256) void xl_bias_q_kernel(int64_t total, int H, const T* __restrict__ q, const float* __restrict__ rw,
                                                       const float* __restrict__ rr, const float* __restrict__ rs,
                                                       T* __restrict__ qw, T* __restrict__ qr, T* __restrict__ qs) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int c = (int)(i % H);
    const float v = to_f32(q[i]);
    qw[i] = from_f32<T>(v + rw[c]);
    qr[i] = from_f32<T>(v + rr[c]);
    qs[i] = from_f32<T>(v + rs[c]);
  }
}

// Kernel pack: wkv[h][0:H] = wk[h][:], wkv[h][H:2H] = wv[h][:]; other weights cast to T
template <typename T>
__global__ __launch_bounds__(256) void xl_pack_kv_kernel(int H, const float* __restrict__ wk, const float* __restrict__ wv,
                                                        T* __restrict__ wkv) {
  const int64_t total = (int64_t)H * 2 * H;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int h = (int)(i / (2 * H)), j = (int)(i % (2 * H));
    wkv[i] = from_f32<T>(j < H ? wk[(int64_t)h * H + j] : wv[(int64_t)h * H + j - H]);
  }
}

// wqkv[h][0:H] = wq[h][:], [H:2H] = wk[h][:], [2H:3H] = wv[h][:]: as a K-major operand, row h of the three kernels side by side
template <typename T>
__global__ __launch_bounds__(256) void xl_pack_qkv_kernel(int H, const float* __restrict__ wq, const float* __restrict__ wk,
                                                         const float* __restrict__ wv, T* __restrict__ wqkv) {
  const int64_t total = (int64_t)H * 3 * H;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int h = (int)(i / (3 * H)), j = (int)(i % (3 * H));
    const float* src = j < H ? wq : (j < 2 * H ? wk : wv);
    wqkv[i] = from_f32<T>(src[(int64_t)h * H + j % H]);
  }
}

// pe[r][t] = sin((klen - r) * f_t), pe[r][H/2 + t] = cos(...), f_t = 10000^(-2t/H)  (lambda_funcs.py:50-79)
template <typename T>
__global__ __launch_bounds__(256) void xl_pos_emb_kernel(int R, int H, int klen, T* __restrict__ pe) {
  const int64_t total = (int64_t)R * (H / 2);
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int r = (int)(i / (H / 2)), t = (int)(i % (H / 2));
    const double f = pow(10000.0, -2.0 * t / H);
    const double a = (double)(klen - r) * f;
    pe[(int64_t)r * H + t] = from_f32<T>((float)sin(a));
    pe[(int64_t)r * H + H / 2 + t] = from_f32<T>((float)cos(a));
  }
}

// One wave per (stacked query row i', batch b, head n); the streams' query rows are stacked, i' = stream * Q + i
// (QQ rows in all), as the q buffers and the masks hold them:
//   score[j] = (ac[i'][j] + bd[i'][j + Q - i] + ef[seg(i,j,b)]) * scale - 1e30 * mask[i'][j][b],  p = softmax_j
// with ef[s] = (q + r_s)[i',b,n,:] . seg_emb[s,n,:].  ac is [B*N][QQ][K], bd [B*N][QQ][R] (fp32).
template <typename T, int NV>
__global__ __launch_bounds__(256) void xl_softmax_fwd_kernel(int Q, int QQ, int K, int R, int B, int N, int D, const float* __restrict__ ac,
                                                            const float* __restrict__ bd, const T* __restrict__ qs,
                                                            const float* __restrict__ seg_emb, const uint8_t* __restrict__ seg_mat,
                                                            const float* __restrict__ mask, float scale, T* __restrict__ p) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // = (b*N + n)*QQ + i'
  if (w >= (int64_t)B * N * QQ) return;
  const int ii = (int)(w % QQ), i = ii % Q;
  const int bn = (int)(w / QQ), n = bn % N, b = bn / N;
  const int H = N * D;
  float e0 = 0.f, e1 = 0.f;
  if (lane < D) {
    const float qv = to_f32(qs[((int64_t)ii * B + b) * H + n * D + lane]);
    e0 = qv * seg_emb[n * D + lane];
    e1 = qv * seg_emb[H + n * D + lane];
  }
  e0 = wave_sum(e0);
  e1 = wave_sum(e1);
  const float* acr = ac + w * K;
  const float* bdr = bd + w * R + (Q - i);
  float v[NV * 4];
  float mx = -INFINITY;
#pragma unroll
  for (int t = 0; t < NV * 4; ++t) {
    const int j = lane + t * 64;
    if (j < K) {
      const float ef = (seg_mat && seg_mat[((int64_t)i * K + j) * B + b]) ? e1 : e0;
      float s = (acr[j] + bdr[j] + ef) * scale;
      if (mask) s -= 1e30f * mask[((int64_t)ii * K + j) * B + b];
      v[t] = s;
      mx = fmaxf(mx, s);
    } else {
      v[t] = -INFINITY;
    }
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < NV * 4; ++t) { v[t] = expf(v[t] - mx); sum += v[t]; }
  const float inv = 1.0f / wave_sum(sum);
  T* pr = p + w * K;
#pragma unroll
  for (int t = 0; t < NV * 4; ++t) {
    const int j = lane + t * 64;
    if (j < K) pr[j] = from_f32<T>(v[t] * inv);
  }
}

// Softmax backward of one score row (b, n, i) per wave, with everything else that needs the row while it is in
// registers: ds[j] = scale * p[j] * (dp[j] - sum_k p[k] dp[k]);
//   dbd[i][r] = ds[i][r - Q + i] when that column exists (transpose of the rel_shift index map; the other columns of
//   dbd hold zeros from the start and are never touched);
//   def[s] = sum_j [seg(i,j,b) == s] ds[i][j] (gradient of the two segment scores of the row).
template <typename T, int NV>
__global__ __launch_bounds__(256) void xl_softmax_bwd_kernel(int Q, int QQ, int K, int R, int B, int N, const T* __restrict__ p,
                                                            const float* __restrict__ dp, float scale,
                                                            const uint8_t* __restrict__ seg_mat, T* __restrict__ ds,
                                                            T* __restrict__ dbd, float* __restrict__ defs) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= (int64_t)B * N * QQ) return;
  const int i = (int)(w % QQ) % Q;
  const int b = (int)(w / QQ) / N;
  const T* pr = p + w * K;
  const float* dr = dp + w * K;
  float pv[NV][4], dv[NV][4];
  float dot = 0.f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int c = (lane + v * 64) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (c < K) { pv[v][e] = to_f32(pr[c + e]); dv[v][e] = dr[c + e]; } else { pv[v][e] = 0.f; dv[v][e] = 0.f; }
      dot += pv[v][e] * dv[v][e];
    }
  }
  dot = wave_sum(dot);
  T* out = ds + w * K;
  T* brow = dbd + w * R;
  const int shift = Q - i;  // column j of ds lands in column j + Q - i of dbd
  float d0 = 0.f, d1 = 0.f, n1 = 0.f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int c = (lane + v * 64) * 4;
    if (c < K) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const T val = from_f32<T>(scale * pv[v][e] * (dv[v][e] - dot));
        out[c + e] = val;
        brow[c + e + shift] = val;
        const float f = to_f32(val);
        if (seg_mat && seg_mat[((int64_t)i * K + c + e) * B + b]) { d1 += f; n1 += 1.f; } else d0 += f;
      }
    }
  }
  // (columns [0, shift) and [shift + K, R) of the row are zero and stay zero: the band's position depends on i alone,
  // the buffer is cleared when the stage is created and nothing else is ever written outside the band)
  d0 = wave_sum(d0);
  d1 = wave_sum(d1);
  n1 = wave_sum(n1);
  // A softmax row's score gradients sum to zero, so def[0] + def[1] = 0; what the rounded probabilities and the
  // rounded ds leave of that sum is noise, and it would be multiplied by a whole embedding row.  It is taken out of
  // the two sums in proportion to the number of keys each one covers.
  const float excess = (d0 + d1) / (float)K;
  d0 -= excess * ((float)K - n1);
  d1 -= excess * n1;
  if (lane == 0) { defs[w * 2] = d0; defs[w * 2 + 1] = d1; }
}

// One wave per (stacked query row i', b, n): writes def to deft[(n*2+s)][row] for the seg_emb gradient GEMM,
// dqs = def[0]*seg_emb[0] + def[1]*seg_emb[1], and dq = dqw + dqr + dqs.
template <typename T>
__global__ __launch_bounds__(256) void xl_seg_bwd_kernel(int QQ, int B, int N, int D, int64_t rows_total,
                                                        const float* __restrict__ defs, const float* __restrict__ seg_emb,
                                                        const T* __restrict__ dqw, const T* __restrict__ dqr, T* __restrict__ dqs,
                                                        T* __restrict__ dq, int64_t ld_dq, T* __restrict__ deft) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= (int64_t)B * N * QQ) return;
  const int ii = (int)(w % QQ);
  const int bn = (int)(w / QQ), n = bn % N, b = bn / N;
  const int H = N * D;
  const float d0 = defs[w * 2], d1 = defs[w * 2 + 1];
  const int64_t row = (int64_t)ii * B + b;
  if (lane == 0) {
    deft[(int64_t)(n * 2 + 0) * rows_total + row] = from_f32<T>(d0);
    deft[(int64_t)(n * 2 + 1) * rows_total + row] = from_f32<T>(d1);
  }
  if (lane < D) {
    const int64_t o = row * H + n * D + lane;
    const float s = d0 * seg_emb[n * D + lane] + d1 * seg_emb[H + n * D + lane];
    dqs[o] = from_f32<T>(s);
    dq[row * ld_dq + n * D + lane] = from_f32<T>(to_f32(dqw[o]) + to_f32(dqr[o]) + s);
  }
}

// (mem directly in front of x: the memory rows followed by the content stream's rows are the [klen * batch, hidden] input of
// the key / value projection, read as one matrix)
struct LayerOff { size_t mem, x, qw, qr, qs, kv, p, vec, z1, y1, u, hh, z2, st1, st2; };

struct XlnetStage : ds_stage {
  ds_xlnet_cfg xc;
  int L, H, F, N, D, B, Q, Mm, K, R, S, rowsS, rows, krows;  // rowsS = Q*B (one stream), rows = S*Q*B, krows = K*B
  int dtype;
  size_t esz;
  // compute copies
  char* wc_base = nullptr;
  std::vector<char*> wq, wkv, wqkv, wr, wo, w1, w2, kr;
  char* pe = nullptr;
  // stash
  char* stash_base = nullptr;
  size_t slot_bytes = 0, mask_off = 0, seg_off = 0, meta_off = 0, nseg_off = 0, mem_bytes = 0, layer_stride = 0;
  // scores + softmax (forward) and score gradients (backward) in one kernel each, no fp32 score matrices (attention_xl.hip)
  bool score_fused = false;
  // bf16 with xc.residual_fp32: the residual stream (the sums in front of both LayerNorms, the LayerNorm outputs that feed
  // the next sum, and the same chain of gradients in backward) stays in fp32; bf16 is only what a GEMM reads
  bool rs32 = false;
  size_t fw_xf[2] = {0, 0}, fw_y1f = 0, bw_dxf[2] = {0, 0}, bw_dz2f = 0, bw_dy1f = 0, bw_dz1f = 0;
  std::vector<LayerOff> lo;
  std::vector<char> has_mask, has_seg;
  // (the packed mask / segment bits of a slot are valid when it has either)
  // workspace
  char* ws_base = nullptr;
  // buffers the weight-gradient kernels read alternate by layer parity ([2])
  size_t ws_bytes = 0, ws_de = 0, ws_qall, ws_ac, ws_dp, ws_bd, ws_ds, ws_dbd[2], ws_def, ws_dz2[2], ws_du[2], ws_dy1, ws_dz1[2], ws_dvec, ws_dqw[2], ws_dqr[2],
         ws_dqs[2], ws_dqkv[2], ws_dkr[2], ws_deft[2], ws_dx[2];
  WgradLane lane;
  // Deferred weight gradients (xc.wgrad_group = G > 1, bf16): a backward pass leaves the operands of its weight-gradient
  // products in a ring of 2G positions per layer and its activations stay in their stash position; after every G passes
  // ONE product per weight runs over all G micro-batches (a segmented reduction: the micro-batches' rows sit one stash
  // position / one ring position apart), the products of two layers as one grouped launch.  There are then more stash
  // positions than slots (slots + G, rounded up to a multiple of G), handed out round-robin in forward order.
  int G = 1, KP = 0, NDY = 0;
  struct LayerDy { size_t dz2, du, dz1, dqkv, dqw, dqr, dqs, dbd, deft, dkr, dyn2, dyn1, rs2, rs1; };  // (deft: [heads * 2][2G * rows]; dkr: one per layer)
  std::vector<LayerDy> ld;
  char* dy_base = nullptr;
  // The query gradients and the key | value gradients of a pass share one matrix of (mem_len * batch + rows) rows and 3 H
  // columns: dq in columns [0, H) of the rows behind the memory rows, dk | dv in columns [H, 3 H) of the first klen * batch
  // rows - so the content stream's rows hold [dq | dk | dv] side by side and the input gradient
  // dx = dq Wq^T + (dk | dv) Wkv^T is ONE product over 3 H (the query stream's k | v columns are never written and stay zero).
  size_t dy_act = 0, dy_actF = 0, dy_qkv = 0, dy_bd = 0;
  struct Deferred { int xpos, dypos; };
  struct Run { int xpos, dypos, n; };
  std::vector<Deferred> deferred;
  std::vector<int> slot_pos, pos_owner;
  std::vector<char> slot_fresh, pos_deferred, x_bwd_valid, x_wg_valid, dy_wg_valid;
  std::vector<hipEvent_t> ev_x_bwd, ev_x_wg, ev_dy_wg;
  hipEvent_t ev_chain = nullptr, ev_wg_done = nullptr;
  bool wg_outstanding = false;
  int next_pos = 0;
  int64_t n_backward = 0;
  std::vector<GroupOp> wg_pending;
  hipEvent_t ev_refresh = nullptr;
  std::vector<hipEvent_t> ev_cast;   // layer l's compute copies written (refresh_weights on the weight-gradient stream)
  std::vector<char> cast_pending;

  ~XlnetStage() override {
    if (ev_refresh) (void)hipEventDestroy(ev_refresh);
    if (ev_chain) (void)hipEventDestroy(ev_chain);
    if (ev_wg_done) (void)hipEventDestroy(ev_wg_done);
    for (hipEvent_t e : ev_cast) (void)hipEventDestroy(e);
    for (hipEvent_t e : ev_x_bwd) (void)hipEventDestroy(e);
    for (hipEvent_t e : ev_x_wg) (void)hipEventDestroy(e);
    for (hipEvent_t e : ev_dy_wg) (void)hipEventDestroy(e);
    if (dy_base) (void)hipFree(dy_base);
    if (wc_base) (void)hipFree(wc_base);
    if (stash_base) (void)hipFree(stash_base);
    if (ws_base) (void)hipFree(ws_base);
  }
  int base(int l) const { return l * X_NW; }

  int init() {
    L = xc.num_layers; H = xc.hidden; F = xc.ffn; N = xc.heads; D = H / N; B = xc.batch; Q = xc.seq; Mm = xc.mem_len;
    K = Mm + Q; R = K + Q; S = xc.streams; rowsS = Q * B; rows = S * rowsS; krows = K * B;
    dtype = xc.dtype; esz = dtype == DS_BF16 ? 2 : 4;
    char name[96];
    static const char* names[X_NW] = {"q", "k", "v", "r", "o", "bias_context", "bias_relative", "bias_segment", "seg_emb",
                                      "attn_ln/gamma", "attn_ln/beta", "ff/W1", "ff/b1", "ff/W2", "ff/b2", "ff_ln/gamma", "ff_ln/beta"};
    for (int l = 0; l < L; ++l)
      for (int k = 0; k < X_NW; ++k) {
        snprintf(name, sizeof(name), "layer_%d/%s", xc.first_layer + l, names[k]);
        int64_t r = 1, c = H;
        if (k <= X_O) r = H;
        else if (k == X_SEG) r = 2;
        else if (k == X_W1) { r = H; c = F; }
        else if (k == X_B1) c = F;
        else if (k == X_W2) { r = F; c = H; }
        winfo.push_back({name, r, c});
      }
    Arena ca;
    std::vector<size_t> o_q(L), o_kv(L), o_qkv(L), o_r(L), o_o(L), o_1(L), o_2(L), o_kr(L);
    const size_t o_pe = ca.reserve((size_t)R * H * esz);
    for (int l = 0; l < L; ++l) {
      o_kv[l] = ca.reserve((size_t)H * 2 * H * esz);
      o_qkv[l] = ca.reserve((size_t)H * 3 * H * esz);
      o_kr[l] = ca.reserve((size_t)R * H * esz);
      if (dtype == DS_BF16) {
        o_q[l] = ca.reserve((size_t)H * H * esz); o_r[l] = ca.reserve((size_t)H * H * esz); o_o[l] = ca.reserve((size_t)H * H * esz);
        o_1[l] = ca.reserve((size_t)H * F * esz); o_2[l] = ca.reserve((size_t)F * H * esz);
      }
    }
    DS_CHECK_HIP(hipMalloc((void**)&wc_base, ca.used));
    pe = wc_base + o_pe;
    wq.resize(L); wkv.resize(L); wqkv.resize(L); wr.resize(L); wo.resize(L); w1.resize(L); w2.resize(L); kr.resize(L);
    for (int l = 0; l < L; ++l) {
      wkv[l] = wc_base + o_kv[l]; wqkv[l] = wc_base + o_qkv[l]; kr[l] = wc_base + o_kr[l];
      if (dtype == DS_BF16) { wq[l] = wc_base + o_q[l]; wr[l] = wc_base + o_r[l]; wo[l] = wc_base + o_o[l]; w1[l] = wc_base + o_1[l]; w2[l] = wc_base + o_2[l]; }
    }
    // stash
    Arena sa;
    const size_t act = (size_t)rows * H * esz, actF = (size_t)rows * F * esz, stats = (size_t)rows * 2 * 4;
    mask_off = sa.reserve((size_t)S * Q * K * B * 4);
    seg_off = sa.reserve((size_t)Q * K * B);
    score_fused = xc.fused_attention != DS_XL_ATTN_SEPARATE && ds_xl_scores_fit(dtype, D, Q, K, R);
    rs32 = dtype == DS_BF16 && xc.residual_fp32 != 0 && H % 8 == 0 && H <= 2048;
    if (score_fused) {
      meta_off = sa.reserve(ds_xl_meta_bytes(S * Q, K, B));
      nseg_off = sa.reserve((size_t)Q * B * 4);
    }
    lo.resize(L);
    mem_bytes = (size_t)Mm * B * H * esz;   // a multiple of 16: x stays aligned for vector loads
    size_t next_x = sa.reserve(mem_bytes + act);
    for (int l = 0; l < L; ++l) {
      LayerOff& t = lo[l];
      t.mem = next_x;
      t.x = next_x + mem_bytes;
      t.qw = sa.reserve(act); t.qr = sa.reserve(act); t.qs = sa.reserve(act);
      t.kv = sa.reserve((size_t)krows * 2 * H * esz);
      t.p = sa.reserve((size_t)S * B * N * Q * K * esz);
      t.vec = sa.reserve(act); t.z1 = sa.reserve(rs32 ? (size_t)rows * H * 4 : act); t.y1 = sa.reserve(act);
      t.u = sa.reserve(actF); t.hh = sa.reserve(actF); t.z2 = sa.reserve(rs32 ? (size_t)rows * H * 4 : act);
      t.st1 = sa.reserve(stats); t.st2 = sa.reserve(stats);
      if (l + 1 < L) next_x = sa.reserve(mem_bytes + act);
    }
    layer_stride = L > 1 ? lo[1].mem - lo[0].mem : mem_bytes + act;
    slot_bytes = sa.used;
    // deferred weight gradients need whole k-tiles per segment of every reduction (bf16: 64 rows)
    G = xc.wgrad_group > 1 && dtype == DS_BF16 && rows % 64 == 0 && krows % 64 == 0 && R % 64 == 0 && H % 8 == 0 && F % 8 == 0 ? xc.wgrad_group : 1;
    KP = G > 1 ? (xc.stash_slots + G + G - 1) / G * G : xc.stash_slots;
    NDY = 2 * G;
    DS_CHECK_HIP(hipMalloc((void**)&stash_base, slot_bytes * KP));
    slot_pos.assign(xc.stash_slots, -1);
    slot_fresh.assign(xc.stash_slots, 0);
    if (G <= 1) for (int i = 0; i < xc.stash_slots; ++i) slot_pos[i] = i;
    if (G > 1) {
      pos_owner.assign(KP, -1);
      pos_deferred.assign(KP, 0);
      Arena da;
      dy_act = act; dy_actF = actF; dy_qkv = ((size_t)Mm * B + rows) * 3 * H * esz; dy_bd = (size_t)B * N * S * Q * R * esz;
      ld.resize(L);
      for (int l = 0; l < L; ++l) {
        ld[l].dz2 = da.reserve(dy_act * NDY); ld[l].du = da.reserve(dy_actF * NDY); ld[l].dz1 = da.reserve(dy_act * NDY);
        ld[l].dqkv = da.reserve(dy_qkv * NDY); ld[l].dqw = da.reserve(dy_act * NDY); ld[l].dqr = da.reserve(dy_act * NDY);
        ld[l].dqs = da.reserve(dy_act * NDY); ld[l].dbd = da.reserve(dy_bd * NDY);
        ld[l].deft = da.reserve((size_t)N * 2 * rows * esz * NDY); ld[l].dkr = da.reserve((size_t)R * H * esz);
        if (rs32) {  // the fp32 gradients entering the two LayerNorms and two sums per row: their parameter gradients are formed per group
          ld[l].dyn2 = da.reserve((size_t)rows * H * 4 * NDY); ld[l].dyn1 = da.reserve((size_t)rows * H * 4 * NDY);
          ld[l].rs2 = da.reserve((size_t)rows * 8 * NDY); ld[l].rs1 = da.reserve((size_t)rows * 8 * NDY);
        }
      }
      DS_CHECK_HIP(hipMalloc((void**)&dy_base, da.used));
      // the un-shifted score gradients are zero outside the band the score-gradient kernel writes, in every ring position
      for (int l = 0; l < L; ++l) {
        DS_CHECK_HIP(hipMemsetAsync(dy_base + ld[l].dbd, 0, dy_bd * NDY, stream));
        DS_CHECK_HIP(hipMemsetAsync(dy_base + ld[l].dqkv, 0, dy_qkv * NDY, stream));
      }
      ev_x_bwd.assign(KP, nullptr); ev_x_wg.assign(KP, nullptr); ev_dy_wg.assign(NDY, nullptr);
      for (int i = 0; i < KP; ++i) {
        DS_CHECK_HIP(hipEventCreateWithFlags(&ev_x_bwd[i], hipEventDisableTiming));
        DS_CHECK_HIP(hipEventCreateWithFlags(&ev_x_wg[i], hipEventDisableTiming));
      }
      for (int i = 0; i < NDY; ++i) DS_CHECK_HIP(hipEventCreateWithFlags(&ev_dy_wg[i], hipEventDisableTiming));
      DS_CHECK_HIP(hipEventCreateWithFlags(&ev_chain, hipEventDisableTiming));
      DS_CHECK_HIP(hipEventCreateWithFlags(&ev_wg_done, hipEventDisableTiming));
      x_bwd_valid.assign(KP, 0); x_wg_valid.assign(KP, 0); dy_wg_valid.assign(NDY, 0);
    }
    slot_forwarded.assign(xc.stash_slots, 0);
    has_mask.assign(xc.stash_slots, 0);
    has_seg.assign(xc.stash_slots, 0);
    // workspace
    Arena w;
    ws_qall = w.reserve(act);
    if (score_fused) ws_de = w.reserve((size_t)B * N * S * Q * 4);   // forward only, like qall
    const size_t QQ = (size_t)S * Q;  // the streams' query rows stacked: one product / one softmax launch for all of them
    // fp32 scores: only the path of separate products and softmax launches has them
    ws_ac = w.reserve(score_fused ? 256 : (size_t)B * N * QQ * K * 4);
    ws_dp = w.reserve(score_fused ? 256 : (size_t)B * N * QQ * K * 4);  // backward's own score-gradient buffer: forward keeps ws_ac
    ws_bd = w.reserve(score_fused ? 256 : (size_t)B * N * QQ * R * 4);
    ws_ds = w.reserve((size_t)B * N * QQ * K * esz);
    ws_dbd[0] = w.reserve((size_t)B * N * QQ * R * esz);  // read by the weight-gradient stream too (dkr): one per layer parity
    ws_dbd[1] = w.reserve((size_t)B * N * QQ * R * esz);
    ws_def = w.reserve((size_t)B * N * QQ * 2 * 4);
    ws_dy1 = w.reserve(act); ws_dvec = w.reserve(act);
    for (int p = 0; p < 2; ++p) {
      ws_dz2[p] = w.reserve(act); ws_du[p] = w.reserve(actF); ws_dz1[p] = w.reserve(act);
      ws_dqw[p] = w.reserve(act); ws_dqr[p] = w.reserve(act); ws_dqs[p] = w.reserve(act);
      ws_dqkv[p] = w.reserve(((size_t)Mm * B + rows) * 3 * H * esz);
      ws_dkr[p] = w.reserve((size_t)R * H * esz);
      ws_deft[p] = w.reserve((size_t)N * 2 * rows * esz);
    }
    ws_dx[0] = w.reserve(act); ws_dx[1] = w.reserve(act);
    if (rs32) {
      const size_t act32 = (size_t)rows * H * 4;
      fw_xf[0] = w.reserve(act32); fw_xf[1] = w.reserve(act32); fw_y1f = w.reserve(act32);
      bw_dxf[0] = w.reserve(act32); bw_dxf[1] = w.reserve(act32);
      bw_dz2f = w.reserve(act32); bw_dy1f = w.reserve(act32); bw_dz1f = w.reserve(act32);
    }
    ws_bytes = w.used;
    DS_CHECK_HIP(hipMalloc((void**)&ws_base, ws_bytes));
    // the un-shifted score gradients: zero outside the band the softmax backward kernel writes
    // (queued on the stage's stream, ahead of every pass; creation is not something a caller captures in a graph)
    DS_CHECK_HIP(hipMemsetAsync(ws_base + ws_dbd[0], 0, (size_t)B * N * QQ * R * esz, stream));
    DS_CHECK_HIP(hipMemsetAsync(ws_base + ws_dbd[1], 0, (size_t)B * N * QQ * R * esz, stream));
    for (int p = 0; p < 2; ++p) DS_CHECK_HIP(hipMemsetAsync(ws_base + ws_dqkv[p], 0, ((size_t)Mm * B + rows) * 3 * H * esz, stream));
    return DS_OK;
  }

  size_t workspace_bytes() const override { return ws_bytes; }
  // forward writes qall / ac / bd and its stash slot, backward everything else: disjoint
  bool overlap_safe() const override { return true; }
  size_t stash_bytes(int slots) const override { return slot_bytes * (size_t)(G > 1 ? (slots + G + G - 1) / G * G : slots); }

  const void* WT(int l, int which) const {
    if (dtype == DS_BF16) {
      switch (which) { case X_Q: return wq[l]; case X_R: return wr[l]; case X_O: return wo[l]; case X_W1: return w1[l]; default: return w2[l]; }
    }
    return w[base(l) + which];
  }

  int gemm(int am, int bm, int m, int n, int k, const void* a, int64_t lda, const void* b, int64_t ldb, void* c, int64_t ldc,
           int flags = 0, const float* bias = nullptr, const void* residual = nullptr, void* c2 = nullptr) {
    ds_gemm_desc d;
    memset(&d, 0, sizeof(d));
    d.dtype = dtype; d.a_major = am; d.b_major = bm; d.m = m; d.n = n; d.k = k; d.lda = lda; d.ldb = ldb; d.ldc = ldc;
    d.batch = 1; d.batch_inner = 1; d.flags = flags; d.alpha = 1.f; d.a = a; d.b = b; d.c = c; d.bias = bias; d.residual = residual; d.c2 = c2;
    return ds_gemm(&d, stream);
  }
  // batched over (b, n): zo = b, zi = n
  ds_gemm_desc desc_bn(int am, int bm, int m, int n, int k, const void* a, int64_t lda, int64_t a_so, int64_t a_si, const void* b,
                       int64_t ldb, int64_t b_so, int64_t b_si, void* c, int64_t ldc, int64_t c_so, int64_t c_si, int flags,
                       const void* residual = nullptr, int nb = -1) const {
    ds_gemm_desc d;
    memset(&d, 0, sizeof(d));
    d.dtype = dtype; d.a_major = am; d.b_major = bm; d.m = m; d.n = n; d.k = k; d.lda = lda; d.ldb = ldb; d.ldc = ldc;
    d.batch = (nb < 0 ? B : nb) * N; d.batch_inner = N;
    d.a_stride_outer = a_so; d.a_stride_inner = a_si; d.b_stride_outer = b_so; d.b_stride_inner = b_si;
    d.c_stride_outer = c_so; d.c_stride_inner = c_si;
    d.flags = flags; d.alpha = 1.f; d.a = a; d.b = b; d.c = c; d.residual = residual;
    return d;
  }
  int gemm_bn(int am, int bm, int m, int n, int k, const void* a, int64_t lda, int64_t a_so, int64_t a_si, const void* b,
              int64_t ldb, int64_t b_so, int64_t b_si, void* c, int64_t ldc, int64_t c_so, int64_t c_si, int flags,
              const void* residual = nullptr, int nb = -1) {
    const ds_gemm_desc d = desc_bn(am, bm, m, n, k, a, lda, a_so, a_si, b, ldb, b_so, b_si, c, ldc, c_so, c_si, flags, residual, nb);
    return ds_gemm(&d, stream);
  }
  // The per-head products of a backward pass that read the score gradients do not depend on each other: with bf16 and
  // reductions of whole 64-deep k-tiles they go out as ONE launch of 128 x 64 tiles (DS_XL_GROUP_PRODUCTS=0: one each).
  bool group_products(int QQ) const {
    static const char* env = getenv("DS_XL_GROUP_PRODUCTS");
    return dtype == DS_BF16 && D == 64 && QQ % 64 == 0 && K % 64 == 0 && R % 64 == 0 && QQ > 256 && K > 256 && !(env && atoi(env) == 0);
  }
  static int g1(int64_t n) { int64_t b = (n + 255) / 256; return (int)(b > 8192 ? 8192 : (b < 1 ? 1 : b)); }

  // Layer l's compute copies (and its k_r) are only needed when the next forward pass reaches layer l: with a
  // weight-gradient stream at hand those of layers 1.. are made there, one event per layer, and the first forward
  // pass after the refresh waits for each layer's event as it gets to it.
  int refresh_weights() override {
    if (dtype == DS_BF16) hipLaunchKernelGGL(xl_pos_emb_kernel<bf16>, dim3(g1((int64_t)R * H / 2)), dim3(256), 0, stream, R, H, K, (bf16*)pe);
    else hipLaunchKernelGGL(xl_pos_emb_kernel<float>, dim3(g1((int64_t)R * H / 2)), dim3(256), 0, stream, R, H, K, (float*)pe);
    DS_CHECK_LAUNCH();
    hipStream_t side = wgrad_stream;
    if (side) {
      if (ev_cast.empty()) {
        ev_cast.resize(L);
        for (int l = 0; l < L; ++l) DS_CHECK_HIP(hipEventCreateWithFlags(&ev_cast[l], hipEventDisableTiming));
        DS_CHECK_HIP(hipEventCreateWithFlags(&ev_refresh, hipEventDisableTiming));
      }
      // everything queued before this call (the master weights' last update, the position table) precedes the copies
      DS_CHECK_HIP(hipEventRecord(ev_refresh, stream));
      DS_CHECK_HIP(hipStreamWaitEvent(side, ev_refresh, 0));
    }
    cast_pending.assign(L, 0);
    hipStream_t main_stream = stream;
    int rc = DS_OK;
    for (int l = 0; l < L && rc == DS_OK; ++l) {
      const int b = base(l);
      hipStream_t cs = (side && l > 0) ? side : main_stream;
      stream = cs;  // gemm() launches on `stream`
      do {
        if (dtype == DS_BF16) {
          hipLaunchKernelGGL(xl_pack_kv_kernel<bf16>, dim3(1024), dim3(256), 0, cs, H, w[b + X_K], w[b + X_V], (bf16*)wkv[l]);
          hipLaunchKernelGGL(xl_pack_qkv_kernel<bf16>, dim3(1024), dim3(256), 0, cs, H, w[b + X_Q], w[b + X_K], w[b + X_V], (bf16*)wqkv[l]);
          if ((rc = ds_cast_f32_to_bf16(wq[l], w[b + X_Q], (size_t)H * H, cs)) != DS_OK) break;
          if ((rc = ds_cast_f32_to_bf16(wr[l], w[b + X_R], (size_t)H * H, cs)) != DS_OK) break;
          if ((rc = ds_cast_f32_to_bf16(wo[l], w[b + X_O], (size_t)H * H, cs)) != DS_OK) break;
          if ((rc = ds_cast_f32_to_bf16(w1[l], w[b + X_W1], (size_t)H * F, cs)) != DS_OK) break;
          if ((rc = ds_cast_f32_to_bf16(w2[l], w[b + X_W2], (size_t)F * H, cs)) != DS_OK) break;
        } else {
          hipLaunchKernelGGL(xl_pack_kv_kernel<float>, dim3(1024), dim3(256), 0, cs, H, w[b + X_K], w[b + X_V], (float*)wkv[l]);
          hipLaunchKernelGGL(xl_pack_qkv_kernel<float>, dim3(1024), dim3(256), 0, cs, H, w[b + X_Q], w[b + X_K], w[b + X_V], (float*)wqkv[l]);
        }
        // k_r = pos_emb @ Wr does not depend on the micro-batch: once per refresh
        rc = gemm(DS_K_MAJOR, DS_MN_MAJOR, R, H, H, pe, H, WT(l, X_R), H, kr[l], H);
      } while (0);
      stream = main_stream;
      if (rc == DS_OK && cs != main_stream) {
        if (hipEventRecord(ev_cast[l], cs) != hipSuccess) { ds_set_error("ds_stage_refresh_weights: hipEventRecord failed"); rc = DS_EHIP; }
        cast_pending[l] = 1;
      }
    }
    if (rc == DS_OK) DS_CHECK_LAUNCH();
    return rc;
  }
  int await_cast(int l, hipStream_t s) {
    if (!cast_pending.empty() && cast_pending[l]) {
      DS_CHECK_HIP(hipStreamWaitEvent(s, ev_cast[l], 0));
      cast_pending[l] = 0;
    }
    return DS_OK;
  }

  // A stash position for the micro-batch that enters `slot` next (deferred weight gradients only): round-robin over the
  // positions no micro-batch owns; a position that deferred weight-gradient work still reads is flushed first, and
  // `s` - the stream that will write the position - waits for the kernels that last read it.
  int assign_pos(int slot, hipStream_t s) {
    for (int tries = 0; tries < KP; ++tries) {
      const int p = next_pos;
      next_pos = next_pos + 1 == KP ? 0 : next_pos + 1;
      if (pos_owner[p] >= 0) continue;
      if (pos_deferred[p]) DS_PROPAGATE(flush_deferred(false));
      if (x_bwd_valid[p]) DS_CHECK_HIP(hipStreamWaitEvent(s, ev_x_bwd[p], 0));
      if (x_wg_valid[p]) DS_CHECK_HIP(hipStreamWaitEvent(s, ev_x_wg[p], 0));
      x_bwd_valid[p] = x_wg_valid[p] = 0;
      pos_owner[p] = slot;
      slot_pos[slot] = p;
      return DS_OK;
    }
    ds_set_error("ds_stage_forward: no free stash position");
    return DS_ESTATE;
  }
  char* slot_base(int slot) const { return stash_base + (size_t)slot_pos[slot] * slot_bytes; }

  int set_aux(int slot, const float* masks, const uint8_t* seg_mat, const void* mems) {
    if (G > 1 && !slot_fresh[slot]) {  // the side inputs of a micro-batch travel with its stash position
      DS_PROPAGATE(assign_pos(slot, stream));
      slot_fresh[slot] = 1;
    }
    char* sp = slot_base(slot);
    if (masks) DS_CHECK_HIP(hipMemcpyAsync(sp + mask_off, masks, (size_t)S * Q * K * B * 4, hipMemcpyDeviceToDevice, stream));
    if (seg_mat) DS_CHECK_HIP(hipMemcpyAsync(sp + seg_off, seg_mat, (size_t)Q * K * B, hipMemcpyDeviceToDevice, stream));
    if (Mm > 0) {
      if (!mems) { ds_set_error("ds_xlnet_stage_set_inputs: mem_len is %d but mems is NULL", Mm); return DS_EINVAL; }
      DS_CHECK_HIP(hipMemcpy2DAsync(sp + lo[0].mem, layer_stride, mems, mem_bytes, mem_bytes, L, hipMemcpyDeviceToDevice, stream));
    }
    has_mask[slot] = masks != nullptr;
    has_seg[slot] = seg_mat != nullptr;
    if (score_fused && (masks || seg_mat))
      DS_PROPAGATE(ds_xl_pack_meta(Q, S * Q, K, B, masks ? (const float*)(sp + mask_off) : nullptr,
                                   seg_mat ? (const uint8_t*)(sp + seg_off) : nullptr, sp + meta_off, (float*)(sp + nseg_off), stream));
    return DS_OK;
  }

  template <typename T> int softmax_fwd_t(const float* ac, const float* bd, const T* qs, const float* seg_emb, const uint8_t* seg,
                                          const float* mask, float scale, T* p) {
    const int QQ = S * Q;
    const int64_t waves = (int64_t)B * N * QQ;
    dim3 grid((unsigned)((waves + 3) / 4));
    const int need = (K + 255) / 256;
    ds_prof_scope prof(stream, sizeof(T) == 2 ? "xl_softmax_fwd_kernel<bf16>" : "xl_softmax_fwd_kernel<float>",
                       (double)waves * K * (8 + sizeof(T) + 5), "B");
    if (need <= 1) hipLaunchKernelGGL((xl_softmax_fwd_kernel<T, 1>), grid, dim3(256), 0, stream, Q, QQ, K, R, B, N, D, ac, bd, qs, seg_emb, seg, mask, scale, p);
    else if (need <= 2) hipLaunchKernelGGL((xl_softmax_fwd_kernel<T, 2>), grid, dim3(256), 0, stream, Q, QQ, K, R, B, N, D, ac, bd, qs, seg_emb, seg, mask, scale, p);
    else if (need <= 4) hipLaunchKernelGGL((xl_softmax_fwd_kernel<T, 4>), grid, dim3(256), 0, stream, Q, QQ, K, R, B, N, D, ac, bd, qs, seg_emb, seg, mask, scale, p);
    else hipLaunchKernelGGL((xl_softmax_fwd_kernel<T, 8>), grid, dim3(256), 0, stream, Q, QQ, K, R, B, N, D, ac, bd, qs, seg_emb, seg, mask, scale, p);
    DS_CHECK_LAUNCH();
    return DS_OK;
  }

  template <typename T> int softmax_bwd_t(const T* p, const float* dp, float scale, const uint8_t* seg, T* dsm, T* dbd, float* defs) {
    const int QQ = S * Q;
    const int64_t waves = (int64_t)B * N * QQ;
    dim3 grid((unsigned)((waves + 3) / 4));
    const int need = (K + 255) / 256;
    ds_prof_scope prof(stream, sizeof(T) == 2 ? "xl_softmax_bwd_kernel<bf16>" : "xl_softmax_bwd_kernel<float>",
                       (double)waves * (K * (4 + 2 * sizeof(T)) + R * sizeof(T)), "B");
    if (need <= 1) hipLaunchKernelGGL((xl_softmax_bwd_kernel<T, 1>), grid, dim3(256), 0, stream, Q, QQ, K, R, B, N, p, dp, scale, seg, dsm, dbd, defs);
    else if (need <= 2) hipLaunchKernelGGL((xl_softmax_bwd_kernel<T, 2>), grid, dim3(256), 0, stream, Q, QQ, K, R, B, N, p, dp, scale, seg, dsm, dbd, defs);
    else if (need <= 4) hipLaunchKernelGGL((xl_softmax_bwd_kernel<T, 4>), grid, dim3(256), 0, stream, Q, QQ, K, R, B, N, p, dp, scale, seg, dsm, dbd, defs);
    else hipLaunchKernelGGL((xl_softmax_bwd_kernel<T, 8>), grid, dim3(256), 0, stream, Q, QQ, K, R, B, N, p, dp, scale, seg, dsm, dbd, defs);
    DS_CHECK_LAUNCH();
    return DS_OK;
  }

  int forward(int slot, const void* in, const float*, void* out) override {
    ds_prio_scope prio(1);
    if (G > 1) {
      if (!slot_fresh[slot]) {
        if (has_mask[slot] || has_seg[slot] || Mm > 0) {
          ds_set_error("ds_stage_forward: with wgrad_group > 1 a micro-batch's masks, segments and memories live in its own stash "
                       "position: call ds_xlnet_stage_set_inputs before every forward pass");
          return DS_ESTATE;
        }
        DS_PROPAGATE(assign_pos(slot, stream));
      }
      slot_fresh[slot] = 0;
    }
    char* sp = slot_base(slot);
    const size_t act = (size_t)rows * H * esz;
    const float scale = 1.0f / sqrtf((float)D);
    const uint8_t* seg = has_seg[slot] ? (const uint8_t*)(sp + seg_off) : nullptr;
    DS_CHECK_HIP(hipMemcpyAsync(sp + lo[0].x, in, act, hipMemcpyDeviceToDevice, stream));
    if (rs32) DS_PROPAGATE(ds_cast_bf16_to_f32(ws_base + fw_xf[0], in, (size_t)rows * H, stream));
    const int res32 = DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32 | DS_EPI_OUT_F32;
    char* qall = ws_base + ws_qall;
    float* ac = (float*)(ws_base + ws_ac);
    float* bd = (float*)(ws_base + ws_bd);
    for (int l = 0; l < L; ++l) {
      const LayerOff& t = lo[l];
      const int b = base(l);
      char* x = sp + t.x;
      char* y = (l + 1 < L) ? sp + lo[l + 1].x : (char*)out;
      DS_PROPAGATE(await_cast(l, stream));
      // q for every stream row; k|v for memory rows and for the content-stream rows
      // The two projections do not depend on each other: one grouped launch of 128 x 128 tiles (64 + 112 of them at the
      // XLNet-36 shape) instead of two launches of 64 x 64 tiles, 1 % of the step.  DS_XL_GROUP_QKV = -1: two launches; 0..5: tile shape.
      static const char* env_qkv = getenv("DS_XL_GROUP_QKV");
      const int qkv_cfg = env_qkv ? atoi(env_qkv) : 2;
      if (qkv_cfg >= 0 && dtype == DS_BF16 && H % 64 == 0 && H > 256) {
        GroupOp ops[2];
        for (GroupOp& o : ops) { o.kind = GOP_GEMM; o.cfg = qkv_cfg; o.prio = ds_launch_prio; memset(&o.gemm, 0, sizeof(o.gemm)); }
        ds_gemm_desc& dq_ = ops[1].gemm; ds_gemm_desc& dk_ = ops[0].gemm;
        dq_.dtype = dtype; dq_.a_major = DS_K_MAJOR; dq_.b_major = DS_MN_MAJOR; dq_.m = rows; dq_.n = H; dq_.k = H; dq_.lda = H; dq_.ldb = H; dq_.ldc = H;
        dq_.batch = 1; dq_.batch_inner = 1; dq_.alpha = 1.f; dq_.a = x; dq_.b = WT(l, X_Q); dq_.c = qall;
        dk_ = dq_; dk_.m = krows; dk_.n = 2 * H; dk_.ldb = 2 * H; dk_.ldc = 2 * H; dk_.a = sp + t.mem; dk_.b = wkv[l]; dk_.c = sp + t.kv;
        DS_PROPAGATE(ds_group_launch(ops, 2, stream));
      } else {
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, rows, H, H, x, H, WT(l, X_Q), H, qall, H));
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, krows, 2 * H, H, sp + t.mem, H, wkv[l], 2 * H, sp + t.kv, 2 * H));
      }
      {
        const int64_t total = (int64_t)rows * H;
        if (score_fused)
          DS_PROPAGATE(ds_xl_bias_q(S * Q, B, N, qall, w[b + X_RW], w[b + X_RR], w[b + X_RS], w[b + X_SEG], sp + t.qw, sp + t.qr, sp + t.qs,
                                    (float*)(ws_base + ws_de), stream));
        else if (dtype == DS_BF16)
          hipLaunchKernelGGL(xl_bias_q_kernel<bf16>, dim3(g1(total)), dim3(256), 0, stream, total, H, (const bf16*)qall, w[b + X_RW],
                             w[b + X_RR], w[b + X_RS], (bf16*)(sp + t.qw), (bf16*)(sp + t.qr), (bf16*)(sp + t.qs));
        else
          hipLaunchKernelGGL(xl_bias_q_kernel<float>, dim3(g1(total)), dim3(256), 0, stream, total, H, (const float*)qall, w[b + X_RW],
                             w[b + X_RR], w[b + X_RS], (float*)(sp + t.qw), (float*)(sp + t.qr), (float*)(sp + t.qs));
        DS_CHECK_LAUNCH();
      }
      if (score_fused) {
        const int QQ = S * Q;
        XlScoreArgs xa;
        memset(&xa, 0, sizeof(xa));
        xa.qw = sp + t.qw; xa.qr = sp + t.qr; xa.de = (const float*)(ws_base + ws_de); xa.ldq = (int64_t)B * H;
        xa.k = sp + t.kv; xa.ldk = (int64_t)B * 2 * H; xa.ldk_b = 2 * H;
        xa.kr = kr[l]; xa.ldkr = H;
        xa.meta = (has_mask[slot] || has_seg[slot]) ? sp + meta_off : nullptr;
        xa.p = sp + t.p;
        xa.Q = Q; xa.QQ = QQ; xa.K = K; xa.R = R; xa.B = B; xa.N = N; xa.H = H; xa.scale = scale;
        DS_PROPAGATE(ds_xl_scores_fwd(&xa, stream));
        // vec = P v
        DS_PROPAGATE(gemm_bn(DS_K_MAJOR, DS_MN_MAJOR, QQ, D, K, sp + t.p, K, (int64_t)N * QQ * K, (int64_t)QQ * K, sp + t.kv + (size_t)H * esz,
                             (int64_t)B * 2 * H, 2 * H, D, sp + t.vec, (int64_t)B * H, H, D, 0));
      } else {
        // The streams' query rows are stacked in the q buffers ([stream][i][b] = row stream*Q + i of stride B*H): every
        // product below and the softmax run once over all QQ = S*Q rows; probabilities are stashed as [B*N][QQ][K].
        const int QQ = S * Q;
        // ac = (q + r_w) k^T ; bd (unshifted) = (q + r_r) k_r^T
        DS_PROPAGATE(gemm_bn(DS_K_MAJOR, DS_K_MAJOR, QQ, K, D, sp + t.qw, (int64_t)B * H, H, D, sp + t.kv, (int64_t)B * 2 * H, 2 * H, D,
                             ac, K, (int64_t)N * QQ * K, (int64_t)QQ * K, DS_EPI_OUT_F32));
        DS_PROPAGATE(gemm_bn(DS_K_MAJOR, DS_K_MAJOR, QQ, R, D, sp + t.qr, (int64_t)B * H, H, D, kr[l], H, 0, D,
                             bd, R, (int64_t)N * QQ * R, (int64_t)QQ * R, DS_EPI_OUT_F32));
        const float* mask = has_mask[slot] ? (const float*)(sp + mask_off) : nullptr;
        char* p = sp + t.p;
        if (dtype == DS_BF16) DS_PROPAGATE(softmax_fwd_t<bf16>(ac, bd, (const bf16*)(sp + t.qs), w[b + X_SEG], seg, mask, scale, (bf16*)p));
        else DS_PROPAGATE(softmax_fwd_t<float>(ac, bd, (const float*)(sp + t.qs), w[b + X_SEG], seg, mask, scale, (float*)p));
        // vec = P v
        DS_PROPAGATE(gemm_bn(DS_K_MAJOR, DS_MN_MAJOR, QQ, D, K, p, K, (int64_t)N * QQ * K, (int64_t)QQ * K, sp + t.kv + (size_t)H * esz,
                             (int64_t)B * 2 * H, 2 * H, D, sp + t.vec, (int64_t)B * H, H, D, 0));
      }
      // attn_out = vec Wo^T (einsum ibnd,hnd->ibh) + x, LayerNorm
      if (rs32) {
        // fp32 stream: x and y1 travel as fp32 beside their bf16 copies (the GEMM operands); z1, z2 are stashed in fp32
        float* xf = (float*)(ws_base + fw_xf[l & 1]);
        float* y1f = (float*)(ws_base + fw_y1f);
        float* yf = (l + 1 < L) ? (float*)(ws_base + fw_xf[(l + 1) & 1]) : nullptr;
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, H, H, sp + t.vec, H, WT(l, X_O), H, sp + t.z1, H, res32, nullptr, xf));
        DS_PROPAGATE(ds_layernorm_fwd_mixed(rows, H, (const float*)(sp + t.z1), w[b + X_LN1_G], w[b + X_LN1_B], xc.ln_eps, sp + t.y1, y1f,
                                            (float*)(sp + t.st1), stream));
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, rows, F, H, sp + t.y1, H, WT(l, X_W1), F, sp + t.u, F,
                          DS_EPI_BIAS | DS_EPI_GELU | DS_EPI_TANH_FORM, w[b + X_B1], nullptr, sp + t.hh));
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, rows, H, F, sp + t.hh, F, WT(l, X_W2), H, sp + t.z2, H, DS_EPI_BIAS | res32,
                          w[b + X_B2], y1f));
        DS_PROPAGATE(ds_layernorm_fwd_mixed(rows, H, (const float*)(sp + t.z2), w[b + X_LN2_G], w[b + X_LN2_B], xc.ln_eps, y, yf,
                                            (float*)(sp + t.st2), stream));
        continue;
      }
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, H, H, sp + t.vec, H, WT(l, X_O), H, sp + t.z1, H, DS_EPI_RESIDUAL, nullptr, x));
      DS_PROPAGATE(ds_layernorm_fwd(dtype, rows, H, sp + t.z1, w[b + X_LN1_G], w[b + X_LN1_B], xc.ln_eps, sp + t.y1, (float*)(sp + t.st1), stream));
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, rows, F, H, sp + t.y1, H, WT(l, X_W1), F, sp + t.u, F,
                        DS_EPI_BIAS | DS_EPI_GELU | DS_EPI_TANH_FORM, w[b + X_B1], nullptr, sp + t.hh));
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, rows, H, F, sp + t.hh, F, WT(l, X_W2), H, sp + t.z2, H, DS_EPI_BIAS | DS_EPI_RESIDUAL,
                        w[b + X_B2], sp + t.y1));
      DS_PROPAGATE(ds_layernorm_fwd(dtype, rows, H, sp + t.z2, w[b + X_LN2_G], w[b + X_LN2_B], xc.ln_eps, y, (float*)(sp + t.st2), stream));
    }
    return DS_OK;
  }

  int release(int slot) override {
    if (G > 1 && slot_pos[slot] >= 0) {  // the stash position goes back to the pool; nothing was deferred for it
      const int pos = slot_pos[slot];
      pos_owner[pos] = -1;
      x_bwd_valid[pos] = 0;
    }
    return DS_OK;
  }

  // runs of micro-batches that sit in consecutive stash positions and consecutive ring positions: one product per run
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
  int launch_pending_wgrads() {
    if (wg_pending.empty()) return DS_OK;
    const int rc = ds_group_launch(wg_pending.data(), (int)wg_pending.size(), stream);
    wg_pending.clear();
    return rc;
  }
  // The deferred weight gradients of layer l for every run, on `stream`: six products per run - W2, W1, o, q, r, k|v - each
  // a segmented reduction over the run's micro-batches (activations one stash position apart, gradients one ring position
  // apart), queued for a grouped launch of 256 x 128 tiles (two layers per launch) where the reduction is long enough,
  // and the bias column sums over the run's rows.
  int layer_wgrad_runs(int l, const std::vector<Run>& runs) {
    const LayerOff& t = lo[l];
    const int b = base(l);
    ds_prio_scope prio(0);
    const int64_t sstride = (int64_t)(slot_bytes / esz);
    const bool kv_adjacent = g[b + X_V] == g[b + X_K] + (size_t)H * H;
    for (const Run& r : runs) {
      const char* sp0 = stash_base + (size_t)r.xpos * slot_bytes;
      const char* dz2 = dy_base + ld[l].dz2 + r.dypos * dy_act; const char* du = dy_base + ld[l].du + r.dypos * dy_actF;
      const char* dz1 = dy_base + ld[l].dz1 + r.dypos * dy_act;
      const char* dqkv = dy_base + ld[l].dqkv + r.dypos * dy_qkv;
      const char* dq = dqkv + (size_t)Mm * B * 3 * H * esz;   // columns [0, H) behind the memory rows
      const char* dkv = dqkv + (size_t)H * esz;                // columns [H, 3 H) from the first row
      const int64_t qkv_seg = (int64_t)(dy_qkv / esz);
      char* dkr = dy_base + ld[l].dkr;
      const int QQ = S * Q;
      // dk_r = sum over micro-batches and samples of dbd^T (q + r_r), per head: k_r is shared by the batch, so one launch per
      // batch entry, added in place (launched before the grouped products: W_r's needs it)
      for (int bb = 0; bb < B; ++bb) {
        ds_gemm_desc d = desc_bn(DS_MN_MAJOR, DS_MN_MAJOR, R, D, QQ * r.n, dy_base + ld[l].dbd + r.dypos * dy_bd + (size_t)bb * N * QQ * R * esz, R, 0,
                                 (int64_t)QQ * R, sp0 + t.qr + (size_t)bb * H * esz, (int64_t)B * H, 0, D, dkr, H, 0, D,
                                 bb > 0 ? DS_EPI_RESIDUAL : 0, dkr, 1);
        if (r.n > 1) { d.k_segment = QQ; d.a_segment_stride = (int64_t)(dy_bd / esz); d.b_segment_stride = sstride; }
        if (D == 64 && R >= 128 && d.k / 64 > 4) {  // a long reduction into 64 columns per head: 8-wave 128 x 64 tiles
          GroupOp o;
          o.kind = GOP_GEMM; o.gemm = d; o.cfg = 3; o.prio = 0;
          DS_PROPAGATE(ds_group_launch(&o, 1, stream));
        } else {
          DS_PROPAGATE(ds_gemm(&d, stream));
        }
      }
      // seg_emb[s][n][:] += sum_rows def[row][n][s] * qs[row][n][:]   (batched over heads; the run's rows are contiguous in deft)
      {
        ds_gemm_desc d;
        memset(&d, 0, sizeof(d));
        d.dtype = dtype; d.a_major = DS_K_MAJOR; d.b_major = DS_MN_MAJOR; d.m = 2; d.n = D; d.k = rows * r.n;
        d.lda = (int64_t)NDY * rows; d.ldb = H; d.ldc = H; d.batch = N; d.batch_inner = N;
        d.a_stride_inner = (int64_t)2 * NDY * rows; d.b_stride_inner = D; d.c_stride_inner = D;
        d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.a = dy_base + ld[l].deft + (size_t)r.dypos * rows * esz; d.b = sp0 + t.qs; d.c = g[b + X_SEG];
        if (r.n > 1) { d.k_segment = rows; d.b_segment_stride = sstride; }
        DS_PROPAGATE(ds_gemm(&d, stream));
      }
      ds_gemm_desc ds[7];
      int nd = 0;
      auto wg = [&](int m, int n, int kseg, const void* a, int64_t lda, int64_t aseg, const void* bb, int64_t ldb, int64_t bseg, float* c,
                    int64_t ldc) -> ds_gemm_desc& {
        ds_gemm_desc& d = ds[nd++];
        memset(&d, 0, sizeof(d));
        d.dtype = dtype; d.a_major = DS_MN_MAJOR; d.b_major = DS_MN_MAJOR; d.m = m; d.n = n; d.k = kseg * r.n; d.lda = lda; d.ldb = ldb; d.ldc = ldc;
        d.batch = 1; d.batch_inner = 1; d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.a = a; d.b = bb; d.c = c;
        if (r.n > 1) { d.k_segment = kseg; d.a_segment_stride = aseg; d.b_segment_stride = bseg; }
        return d;
      };
      wg(F, H, rows, sp0 + t.hh, F, sstride, dz2, H, (int64_t)rows * H, g[b + X_W2], H);
      wg(H, F, rows, sp0 + t.y1, H, sstride, du, F, (int64_t)rows * F, g[b + X_W1], F);
      wg(H, H, rows, dz1, H, (int64_t)rows * H, sp0 + t.vec, H, sstride, g[b + X_O], H);
      wg(H, H, rows, sp0 + t.x, H, sstride, dq, 3 * H, qkv_seg, g[b + X_Q], H);
      { ds_gemm_desc& d = wg(H, H, R, pe, H, 0, dkr, H, 0, g[b + X_R], H); d.k = R; d.k_segment = 0; }   // dk_r already holds the run's sum
      if (kv_adjacent) {  // k and v: the two column halves of dkv, batched (z = 0: k, 1: v)
        ds_gemm_desc& d = wg(H, H, krows, sp0 + t.mem, H, sstride, dkv, 3 * H, qkv_seg, g[b + X_K], H);
        d.batch = 2; d.batch_inner = 2; d.b_stride_inner = H; d.c_stride_inner = (int64_t)H * H;
      } else {
        for (int j = 0; j < 2; ++j)
          wg(H, H, krows, sp0 + t.mem, H, sstride, dkv + (size_t)j * H * esz, 3 * H, qkv_seg, g[b + X_K + j], H);
      }
      bool b1_fused = false;   // the first FFN bias gradient = column sums of du, the dY operand of W1's product
      for (int i = 0; i < nd; ++i) {
        // (one launch never carries two products into the same master gradient: runs of one layer are flushed apart)
        const bool grouped = ds[i].k / 64 > 3 && ds[i].m >= 128 && ds[i].n >= 128;
        if (grouped) {
          GroupOp o;
          o.kind = GOP_GEMM; o.gemm = ds[i]; o.cfg = ds[i].m >= 256 ? 1 : 2; o.prio = 0;
          if (i == 1 && o.cfg == 1) {
            o.colsum = g[b + X_B1];
            b1_fused = true;
          }
          wg_pending.push_back(o);
        } else {
          DS_PROPAGATE(ds_gemm(&ds[i], stream));
        }
      }
      if (runs.size() > 1 || wg_pending.size() + nd > (size_t)DS_GROUP_MAX_TASKS) DS_PROPAGATE(launch_pending_wgrads());
      if (!b1_fused) DS_PROPAGATE(ds_colsum_accum(dtype, rows * r.n, F, du, F, g[b + X_B1], stream));
      if (rs32) {
        const size_t a32 = (size_t)rows * H * 4, r8 = (size_t)rows * 8;
        const int64_t s4 = (int64_t)(slot_bytes / 4);
        DS_PROPAGATE(ds_layernorm_param_grads_exact_seg(rows * r.n, H, (const float*)(dy_base + ld[l].dyn2 + r.dypos * a32), (const float*)(sp0 + t.z2),
                                                        w[b + X_LN2_G], (const float*)(sp0 + t.st2), (const float*)(dy_base + ld[l].rs2 + r.dypos * r8),
                                                        g[b + X_LN2_G], g[b + X_LN2_B], g[b + X_B2], rows, s4, s4, stream));
        DS_PROPAGATE(ds_layernorm_param_grads_exact_seg(rows * r.n, H, (const float*)(dy_base + ld[l].dyn1 + r.dypos * a32), (const float*)(sp0 + t.z1),
                                                        w[b + X_LN1_G], (const float*)(sp0 + t.st1), (const float*)(dy_base + ld[l].rs1 + r.dypos * r8),
                                                        g[b + X_LN1_G], g[b + X_LN1_B], nullptr, rows, s4, s4, stream));
      }
      const void* const xs3[3] = {dy_base + ld[l].dqw + r.dypos * dy_act, dy_base + ld[l].dqr + r.dypos * dy_act, dy_base + ld[l].dqs + r.dypos * dy_act};
      float* const out3[3] = {g[b + X_RW], g[b + X_RR], g[b + X_RS]};
      DS_PROPAGATE(ds_colsum_accum_multi(dtype, rows * r.n, H, 3, xs3, H, out3, stream));
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

  int backward(int slot, const void* d_out, void* d_in) override {
    ds_prio_scope prio(3);  // the chain every later pass waits on
    char* sp = slot_base(slot);
    const int pos = slot_pos[slot];
    const int dypos = G > 1 ? (int)(n_backward % NDY) : 0;
    if (G > 1 && dy_wg_valid[dypos]) DS_CHECK_HIP(hipStreamWaitEvent(stream, ev_dy_wg[dypos], 0));
    // the pass that completes a group queues the group's products layer by layer as its own chain passes each layer
    const bool closing = G > 1 && (int)deferred.size() + 1 >= G;
    std::vector<Run> runs;
    if (closing) {
      std::vector<Deferred> all = deferred;
      all.push_back({pos, dypos});
      runs = make_runs(all);
    }
    const float scale = 1.0f / sqrtf((float)D);
    const uint8_t* seg = has_seg[slot] ? (const uint8_t*)(sp + seg_off) : nullptr;
    const char* dy = (const char*)d_out;
    char* dy1 = ws_base + ws_dy1; char* dvec = ws_base + ws_dvec;
    float* dp = (float*)(ws_base + ws_dp);
    char* dsm = ws_base + ws_ds;
    // with a weight-gradient stream, a layer's weight gradients run beside the dgrad chain of the layers below
    hipStream_t wgs = wgrad_stream;
    if (wgs) DS_PROPAGATE(lane.ensure());
    const int res32 = DS_EPI_RESIDUAL | DS_EPI_RESIDUAL_F32 | DS_EPI_OUT_F32;
    const float* dyf = nullptr;   // fp32 stream: the gradient that travels down the layers
    if (rs32) {
      DS_PROPAGATE(ds_cast_bf16_to_f32(ws_base + bw_dxf[L & 1], d_out, (size_t)rows * H, stream));
      dyf = (const float*)(ws_base + bw_dxf[L & 1]);
    }
    for (int l = L - 1; l >= 0; --l) {
      const LayerOff& t = lo[l];
      const int b = base(l);
      const int par = l & 1;
      // with deferred weight gradients their operands go to the layer's ring position of this pass
      auto ringp = [&](size_t off, size_t per) { return dy_base + off + (size_t)dypos * per; };
      char* dz2 = G > 1 ? ringp(ld[l].dz2, dy_act) : ws_base + ws_dz2[par];
      char* du = G > 1 ? ringp(ld[l].du, dy_actF) : ws_base + ws_du[par];
      char* dz1 = G > 1 ? ringp(ld[l].dz1, dy_act) : ws_base + ws_dz1[par];
      char* dqw = G > 1 ? ringp(ld[l].dqw, dy_act) : ws_base + ws_dqw[par];
      char* dqr = G > 1 ? ringp(ld[l].dqr, dy_act) : ws_base + ws_dqr[par];
      char* dqs = G > 1 ? ringp(ld[l].dqs, dy_act) : ws_base + ws_dqs[par];
      char* dqkv = G > 1 ? ringp(ld[l].dqkv, dy_qkv) : ws_base + ws_dqkv[par];
      char* dq = dqkv + (size_t)Mm * B * 3 * H * esz;   // [rows, H] at row stride 3 H
      char* dkv = dqkv + (size_t)H * esz;                // [klen * batch, 2 H] at row stride 3 H
      char* dkr = ws_base + ws_dkr[par];
      char* deft = G > 1 ? dy_base + ld[l].deft + (size_t)dypos * rows * esz : ws_base + ws_deft[par];
      const int64_t deft_ld = G > 1 ? (int64_t)NDY * rows : (int64_t)rows;
      char* dbd = G > 1 ? ringp(ld[l].dbd, dy_bd) : ws_base + ws_dbd[par];
      if (wgs && G <= 1) DS_PROPAGATE(lane.reuse(stream, par));
      char* x = sp + t.x;
      float* dz2f = (float*)(ws_base + bw_dz2f);
      float* dy1f = (float*)(ws_base + bw_dy1f);
      float* dz1f = (float*)(ws_base + bw_dz1f);
      if (rs32 && G > 1) {
        // rows only on the chain (no atomics); gamma / beta / bias gradients come from the fp32 copy and the row sums, per group
        const size_t a32 = (size_t)rows * H * 4, r8 = (size_t)rows * 8;
        DS_PROPAGATE(ds_layernorm_bwd_mixed_rows(rows, H, dyf, (const float*)(sp + t.z2), w[b + X_LN2_G], (const float*)(sp + t.st2), dz2, dz2f,
                                                 (float*)(dy_base + ld[l].dyn2 + dypos * a32), (float*)(dy_base + ld[l].rs2 + dypos * r8), stream));
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, F, H, dz2, H, WT(l, X_W2), H, du, F, DS_EPI_DGELU | DS_EPI_TANH_FORM, nullptr, nullptr, sp + t.u));
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, H, F, du, F, WT(l, X_W1), F, dy1f, H, res32, nullptr, dz2f));
        DS_PROPAGATE(ds_layernorm_bwd_mixed_rows(rows, H, dy1f, (const float*)(sp + t.z1), w[b + X_LN1_G], (const float*)(sp + t.st1), dz1, dz1f,
                                                 (float*)(dy_base + ld[l].dyn1 + dypos * a32), (float*)(dy_base + ld[l].rs1 + dypos * r8), stream));
      } else if (rs32) {
        DS_PROPAGATE(ds_layernorm_bwd_mixed(rows, H, dyf, (const float*)(sp + t.z2), w[b + X_LN2_G], (const float*)(sp + t.st2), dz2, dz2f,
                                            nullptr, g[b + X_LN2_G], g[b + X_LN2_B], g[b + X_B2], stream));
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, F, H, dz2, H, WT(l, X_W2), H, du, F, DS_EPI_DGELU | DS_EPI_TANH_FORM, nullptr, nullptr, sp + t.u));
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, H, F, du, F, WT(l, X_W1), F, dy1f, H, res32, nullptr, dz2f));
        DS_PROPAGATE(ds_layernorm_bwd_mixed(rows, H, dy1f, (const float*)(sp + t.z1), w[b + X_LN1_G], (const float*)(sp + t.st1), dz1, dz1f,
                                            nullptr, g[b + X_LN1_G], g[b + X_LN1_B], nullptr, stream));
      } else {
      DS_PROPAGATE(ds_layernorm_bwd(dtype, rows, H, dy, sp + t.z2, w[b + X_LN2_G], (const float*)(sp + t.st2), nullptr, dz2,
                                    g[b + X_LN2_G], g[b + X_LN2_B], g[b + X_B2], stream));
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, F, H, dz2, H, WT(l, X_W2), H, du, F, DS_EPI_DGELU | DS_EPI_TANH_FORM, nullptr, nullptr, sp + t.u));
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, H, F, du, F, WT(l, X_W1), F, dy1, H, DS_EPI_RESIDUAL, nullptr, dz2));
      DS_PROPAGATE(ds_layernorm_bwd(dtype, rows, H, dy1, sp + t.z1, w[b + X_LN1_G], (const float*)(sp + t.st1), nullptr, dz1,
                                    g[b + X_LN1_G], g[b + X_LN1_B], nullptr, stream));
      }
      // o projection: attn_out[row,h] = sum_nd vec[row,nd] Wo[h,nd]
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_MN_MAJOR, rows, H, H, dz1, H, WT(l, X_O), H, dvec, H));
      {
        // all streams' query rows at once (QQ = S*Q stacked rows, see forward): the sums over the streams that k, v and
        // k_r receive fall out of the longer reductions
        const int QQ = S * Q;
        const char* p = sp + t.p;
        // dP = dvec v^T (inside the score-gradient kernel where that one runs) ; dv = P^T dvec
        if (!score_fused)
          DS_PROPAGATE(gemm_bn(DS_K_MAJOR, DS_K_MAJOR, QQ, K, D, dvec, (int64_t)B * H, H, D, sp + t.kv + (size_t)H * esz, (int64_t)B * 2 * H,
                               2 * H, D, dp, K, (int64_t)N * QQ * K, (int64_t)QQ * K, DS_EPI_OUT_F32));
        const bool grouped = group_products(QQ);
        const ds_gemm_desc d_dv = desc_bn(DS_MN_MAJOR, DS_MN_MAJOR, K, D, QQ, p, K, (int64_t)N * QQ * K, (int64_t)QQ * K, dvec, (int64_t)B * H, H, D,
                                          dkv + (size_t)H * esz, (int64_t)B * 3 * H, 3 * H, D, 0);
        if (!grouped) DS_PROPAGATE(ds_gemm(&d_dv, stream));
        // dS, its un-shifted copy for the position term (dbd[i][r] = dS[i][r - Q + i]) and the segment sums, in one pass
        float* defs = (float*)(ws_base + ws_def);
        if (score_fused) {
          XlScoreArgs xa;
          memset(&xa, 0, sizeof(xa));
          xa.ldq = (int64_t)B * H;
          xa.v = sp + t.kv + (size_t)H * esz; xa.ldk = (int64_t)B * 2 * H; xa.ldk_b = 2 * H;
          xa.ldkr = H;
          xa.meta = (has_mask[slot] || has_seg[slot]) ? sp + meta_off : nullptr;
          xa.nseg = has_seg[slot] ? (const float*)(sp + nseg_off) : nullptr;
          xa.p = (void*)p; xa.dvec = dvec; xa.ds = dsm; xa.dbd = dbd; xa.defs = defs;
          xa.Q = Q; xa.QQ = QQ; xa.K = K; xa.R = R; xa.B = B; xa.N = N; xa.H = H; xa.scale = scale;
          DS_PROPAGATE(ds_xl_scores_bwd(&xa, stream));
        } else if (dtype == DS_BF16) DS_PROPAGATE(softmax_bwd_t<bf16>((const bf16*)p, dp, scale, seg, (bf16*)dsm, (bf16*)dbd, defs));
        else DS_PROPAGATE(softmax_bwd_t<float>((const float*)p, dp, scale, seg, (float*)dsm, (float*)dbd, defs));
        // content term: dqw = dS k ; dk = dS^T qw
        const ds_gemm_desc d_dqw = desc_bn(DS_K_MAJOR, DS_MN_MAJOR, QQ, D, K, dsm, K, (int64_t)N * QQ * K, (int64_t)QQ * K, sp + t.kv,
                                           (int64_t)B * 2 * H, 2 * H, D, dqw, (int64_t)B * H, H, D, 0);
        const ds_gemm_desc d_dk = desc_bn(DS_MN_MAJOR, DS_MN_MAJOR, K, D, QQ, dsm, K, (int64_t)N * QQ * K, (int64_t)QQ * K, sp + t.qw, (int64_t)B * H,
                                          H, D, dkv, (int64_t)B * 3 * H, 3 * H, D, 0);
        // position term through the shift
        const ds_gemm_desc d_dqr = desc_bn(DS_K_MAJOR, DS_MN_MAJOR, QQ, D, R, dbd, R, (int64_t)N * QQ * R, (int64_t)QQ * R, kr[l], H, 0, D,
                                           dqr, (int64_t)B * H, H, D, 0);
        if (grouped) {
          GroupOp ops[4];
          ops[0].gemm = d_dqr; ops[1].gemm = d_dqw; ops[2].gemm = d_dk; ops[3].gemm = d_dv;
          // 128x64 tiles with two buffers (48 KB: three workgroups per CU, or room beside the forward pass's blocks) - these
          // products stream 130 MB of score gradients for 7.5 GFLOP, so what counts is loads in flight per CU, not the
          // depth of one block's ring (measured on the XLNet-36 half-stage: 42.27 ms per step against 42.96 with four
          // buffers, 43.7 / 44.3 with 128x128 tiles of three / two buffers).  DS_XL_PRODUCTS_CFG = 2..5 forces a shape.
          static const char* env_pc = getenv("DS_XL_PRODUCTS_CFG");
          const int pcfg = env_pc ? atoi(env_pc) : 5;
          for (GroupOp& o : ops) { o.kind = GOP_GEMM; o.cfg = pcfg; o.prio = ds_launch_prio; }
          DS_PROPAGATE(ds_group_launch(ops, 4, stream));
        } else {
          DS_PROPAGATE(ds_gemm(&d_dqw, stream));
          DS_PROPAGATE(ds_gemm(&d_dk, stream));
          DS_PROPAGATE(ds_gemm(&d_dqr, stream));
        }
        // (dk_r = dbd^T qr feeds only Wr's gradient: it runs with the weight gradients below)
        // segment term + dq = dqw + dqr + dqs
        {
          const int64_t waves = (int64_t)B * N * QQ;
          dim3 grid((unsigned)((waves + 3) / 4));
          if (dtype == DS_BF16)
            hipLaunchKernelGGL(xl_seg_bwd_kernel<bf16>, grid, dim3(256), 0, stream, QQ, B, N, D, deft_ld, defs, w[b + X_SEG],
                               (const bf16*)dqw, (const bf16*)dqr, (bf16*)dqs, (bf16*)dq, (int64_t)3 * H, (bf16*)deft);
          else
            hipLaunchKernelGGL(xl_seg_bwd_kernel<float>, grid, dim3(256), 0, stream, QQ, B, N, D, deft_ld, defs, w[b + X_SEG],
                               (const float*)dqw, (const float*)dqr, (float*)dqs, (float*)dq, (int64_t)3 * H, (float*)deft);
          DS_CHECK_LAUNCH();
        }
      }
      // ---- weight gradients of this layer (on the weight-gradient stream when there is one)
      hipStream_t chain = stream;
      if (wgs && (G <= 1 || closing)) {
        DS_PROPAGATE(lane.begin(chain, wgs, par));
        stream = wgs;  // gemm() and the column sums below launch on `stream`
      }
      int rc = DS_OK;
      if (G <= 1) do {
        ds_prio_scope wprio(0);  // feeds only the master gradients
        {
        if ((rc = gemm(DS_MN_MAJOR, DS_MN_MAJOR, F, H, rows, sp + t.hh, F, dz2, H, g[b + X_W2], H, DS_EPI_ACCUM)) != DS_OK) break;
        if ((rc = ds_colsum_accum(dtype, rows, F, du, F, g[b + X_B1], stream)) != DS_OK) break;
        if ((rc = gemm(DS_MN_MAJOR, DS_MN_MAJOR, H, F, rows, sp + t.y1, H, du, F, g[b + X_W1], F, DS_EPI_ACCUM)) != DS_OK) break;
        if ((rc = gemm(DS_MN_MAJOR, DS_MN_MAJOR, H, H, rows, dz1, H, sp + t.vec, H, g[b + X_O], H, DS_EPI_ACCUM)) != DS_OK) break;
        }
        // relative biases: column sums of the three query-gradient pieces
        {
          const void* const xs3[3] = {dqw, dqr, dqs};
          float* const out3[3] = {g[b + X_RW], g[b + X_RR], g[b + X_RS]};
          if ((rc = ds_colsum_accum_multi(dtype, rows, H, 3, xs3, H, out3, stream)) != DS_OK) break;
        }
        // seg_emb[s][n][:] += sum_rows def[row][n][s] * qs[row][n][:]   (batched over heads)
        {
          ds_gemm_desc d;
          memset(&d, 0, sizeof(d));
          d.dtype = dtype; d.a_major = DS_K_MAJOR; d.b_major = DS_MN_MAJOR; d.m = 2; d.n = D; d.k = rows;
          d.lda = rows; d.ldb = H; d.ldc = H; d.batch = N; d.batch_inner = N;
          d.a_stride_inner = (int64_t)2 * rows; d.b_stride_inner = D; d.c_stride_inner = D;
          d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.a = deft; d.b = sp + t.qs; d.c = g[b + X_SEG];
          if ((rc = ds_gemm(&d, stream)) != DS_OK) break;
        }
        // projections
        if ((rc = gemm(DS_MN_MAJOR, DS_MN_MAJOR, H, H, rows, x, H, dq, 3 * H, g[b + X_Q], H, DS_EPI_ACCUM)) != DS_OK) break;
        for (int bb = 0; bb < B && rc == DS_OK; ++bb) {  // k_r is shared by the batch: one launch per batch entry, added in place
          const int a2 = bb > 0 ? DS_EPI_RESIDUAL : 0;
          rc = gemm_bn(DS_MN_MAJOR, DS_MN_MAJOR, R, D, S * Q, dbd + (size_t)bb * N * S * Q * R * esz, R, 0, (int64_t)S * Q * R,
                       sp + t.qr + (size_t)bb * H * esz, (int64_t)B * H, 0, D, dkr, H, 0, D, a2, dkr, 1);
        }
        if (rc != DS_OK) break;
        if ((rc = gemm(DS_MN_MAJOR, DS_MN_MAJOR, H, H, R, pe, H, dkr, H, g[b + X_R], H, DS_EPI_ACCUM)) != DS_OK) break;
        // Wk and Wv: the two column halves of dkv against the same rows, one batched launch (z = 0: k, 1: v) when the two
        // master gradients sit one behind the other with no gap
        if (g[b + X_V] == g[b + X_K] + (size_t)H * H) {
          ds_gemm_desc d;
          memset(&d, 0, sizeof(d));
          d.dtype = dtype; d.a_major = DS_MN_MAJOR; d.b_major = DS_MN_MAJOR; d.m = H; d.n = H; d.lda = H; d.ldb = 3 * H; d.ldc = H;
          d.batch = 2; d.batch_inner = 2; d.b_stride_inner = H; d.c_stride_inner = (int64_t)H * H;
          d.flags = DS_EPI_ACCUM; d.alpha = 1.f; d.c = g[b + X_K];
          d.k = krows; d.a = sp + t.mem; d.b = dkv;   // memory rows and content rows in one reduction
          if ((rc = ds_gemm(&d, stream)) != DS_OK) break;
        } else {
          for (int j = 0; j < 2 && rc == DS_OK; ++j)  // j = 0: k, 1: v
            rc = gemm(DS_MN_MAJOR, DS_MN_MAJOR, H, H, krows, sp + t.mem, H, dkv + (size_t)j * H * esz, 3 * H, g[b + X_K + j], H, DS_EPI_ACCUM);
        }
      } while (0);
      if (wgs && G <= 1) {
        stream = chain;
        if (rc != DS_OK) return rc;
        DS_PROPAGATE(lane.end(wgs, par));
      }
      // deferred weight gradients: nothing per pass; the pass that completes a group queues the group's work for this layer,
      // behind what the chain has just left in the ring
      if (closing) rc = layer_wgrad_runs(l, runs);
      stream = chain;
      if (rc != DS_OK) return rc;
      // dx = dq Wq^T + dz1 (residual) and, on the content stream's rows, + (dk | dv) Wkv^T: one product over [dq | dk | dv]
      const bool first = l == 0;
      if (first && d_in == nullptr) break;
      char* dx = first ? (char*)d_in : ws_base + ws_dx[l & 1];
      if (rs32) {
        float* dxf = (float*)(ws_base + bw_dxf[l & 1]);
        DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, H, 3 * H, dq, 3 * H, wqkv[l], 3 * H, dxf, H, res32, nullptr, dz1f));
        if (first) DS_PROPAGATE(ds_cast_f32_to_bf16(d_in, dxf, (size_t)rows * H, stream));  // the stage's input gradient leaves as bf16
        dyf = dxf;
        continue;
      }
      DS_PROPAGATE(gemm(DS_K_MAJOR, DS_K_MAJOR, rows, H, 3 * H, dq, 3 * H, wqkv[l], 3 * H, dx, H, DS_EPI_RESIDUAL, nullptr, dz1));
      dy = dx;
    }
    // the stash slot and the master gradients are released to the caller in the order of `stream`
    if (wgs) DS_PROPAGATE(lane.finish(stream));
    if (G > 1) {
      deferred.push_back({pos, dypos});
      pos_deferred[pos] = 1;
      pos_owner[pos] = -1;
      ++n_backward;
      if (bwd_stream) {
        DS_CHECK_HIP(hipEventRecord(ev_x_bwd[pos], stream));
        x_bwd_valid[pos] = 1;
      } else {
        x_bwd_valid[pos] = 0;
      }
      if (closing) {
        hipStream_t side = wgs ? wgs : stream;
        hipStream_t chain = stream;
        stream = side;
        const int rc = launch_pending_wgrads();
        stream = chain;
        if (rc != DS_OK) return rc;
        DS_PROPAGATE(retire_deferred(side, stream));
      }
    }
    return DS_OK;
  }
};

}  // namespace

extern "C" int ds_xlnet_stage_create(const ds_xlnet_cfg* c, void* stream, ds_stage** out) {
  DS_CHECK_ARG(c != nullptr && out != nullptr, "ds_xlnet_stage_create: null argument");
  *out = nullptr;
  DS_CHECK_ARG(c->dtype == DS_F32 || c->dtype == DS_BF16, "ds_xlnet_stage_create: dtype %d", c->dtype);
  DS_CHECK_ARG(c->num_layers > 0 && c->hidden > 0 && c->heads > 0 && c->ffn > 0 && c->batch > 0 && c->seq > 0 && c->mem_len >= 0,
               "ds_xlnet_stage_create: non-positive shape");
  DS_CHECK_ARG(c->streams == 1 || c->streams == 2, "ds_xlnet_stage_create: streams must be 1 (content) or 2 (content + query)");
  DS_CHECK_ARG(c->hidden % c->heads == 0, "ds_xlnet_stage_create: hidden %d is not a multiple of heads %d", c->hidden, c->heads);
  const int vec = c->dtype == DS_BF16 ? 8 : 4;
  const int d = c->hidden / c->heads;
  DS_CHECK_ARG(d % vec == 0 && d <= 64, "ds_xlnet_stage_create: head size %d must be a multiple of %d and at most 64", d, vec);
  DS_CHECK_ARG(c->seq % vec == 0 && c->mem_len % vec == 0 && c->hidden % vec == 0 && c->ffn % vec == 0,
               "ds_xlnet_stage_create: seq %d, mem_len %d, hidden %d, ffn %d must be multiples of %d", c->seq, c->mem_len, c->hidden, c->ffn, vec);
  DS_CHECK_ARG(c->seq + c->mem_len <= 2048, "ds_xlnet_stage_create: klen %d exceeds 2048", c->seq + c->mem_len);
  DS_CHECK_ARG(c->hidden <= 64 * vec * 8, "ds_xlnet_stage_create: hidden %d too large for the LayerNorm kernel", c->hidden);
  DS_CHECK_ARG(c->stash_slots >= 1, "ds_xlnet_stage_create: stash_slots must be >= 1");
  XlnetStage* s = new XlnetStage();
  memset(&s->cfg, 0, sizeof(s->cfg));
  s->cfg.kind = DS_STAGE_XLNET;
  s->cfg.dtype = c->dtype;
  s->cfg.stash_slots = c->stash_slots;
  s->xc = *c;
  s->stream = (hipStream_t)stream;
  const int rc = s->init();
  if (rc != DS_OK) { delete s; return rc; }
  *out = s;
  return DS_OK;
}

extern "C" int ds_xlnet_stage_set_inputs(ds_stage* h, int slot, const float* masks, const uint8_t* seg_mat, const void* mems) {
  DS_CHECK_ARG(h != nullptr, "ds_xlnet_stage_set_inputs: null handle");
  DS_CHECK_ARG(h->cfg.kind == DS_STAGE_XLNET, "ds_xlnet_stage_set_inputs: not an XLNet stage");
  DS_CHECK_ARG(slot >= 0 && slot < h->cfg.stash_slots, "ds_xlnet_stage_set_inputs: slot %d out of range", slot);
  DS_PROPAGATE(ds_stage_acquire_slot(h, slot));
  return static_cast<XlnetStage*>(h)->set_aux(slot, masks, seg_mat, mems);
}
