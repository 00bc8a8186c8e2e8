// Scores and softmax of XLNet's relative attention without the fp32 score matrices (xlnet/layers/rel_multihead_attn.py:71-115,
// the relative shift of xlnet/layers/lambda_funcs.py:85-93), bf16 with head size 64.  For a stacked query row i' (stream * Q + i),
// sample b and head n
//   score[j] = (qw[i'] . k[j] + qr[i'] . kr[j + Q - i] + ef[seg(i, j, b)]) * scale - 1e30 * mask[i'][j][b],   p = softmax_j score
// and, backward, with dp[j] = dvec[i'] . v[j]:
//   ds[j] = scale * p[j] * (dp[j] - sum_k p[k] dp[k]),  dbd[i'][j + Q - i] = ds[j],  def[s] = sum_j [seg == s] ds[j].
// A block owns 32 query rows and ALL keys of one (b, n): wave w keeps the scores of keys [128 w, 128 w + 128) in registers
// (four 32x32 MFMA accumulators, query rows down the registers, keys across the lanes), so a row's softmax needs one pass and
// the only thing written is the bf16 probability (forward) or the bf16 score gradients (backward).
// The relative shift in that orientation: the position product is computed UN-shifted for the 64 consecutive k_r rows a
// 32 x 32 tile can touch (two accumulators, the second one shared with the next key tile), and the element of row m, key
// column n is column n + 31 - m of that window - for a fixed register (fixed m) a rotation of the lanes, i.e. one
// ds_bpermute after the source lanes picked the accumulator they are asked for.
#include "common.h"
#include "stage.h"

namespace {

constexpr int HD = 64;    // head size
constexpr int NT = 4;     // key tiles (of 32 keys) per wave
constexpr int MAXW = 8;   // waves per block: up to 32 * NT * MAXW = 1024 keys
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ f32x16 mfma(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
// query row (0..31) of accumulator element e in this lane's half
__device__ __forceinline__ int acc_row(int e, int half) { return (e >> 2) * 8 + half * 4 + (e & 3); }
__device__ __forceinline__ float lane_read(float v, int src_lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, v)));
}
// reductions over the 32 lanes of a half wave (the keys of one tile row)
__device__ __forceinline__ float half_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));
  v = fmaxf(v, dpp_move<0x4E>(v));
  v = fmaxf(v, dpp_move<0x141>(v));
  v = fmaxf(v, dpp_move<0x140>(v));
  return fmaxf(v, __shfl_xor(v, 16, 64));
}
__device__ __forceinline__ float half_sum(float v) {
  v += dpp_move<0xB1>(v);
  v += dpp_move<0x4E>(v);
  v += dpp_move<0x141>(v);
  v += dpp_move<0x140>(v);
  return v + __shfl_xor(v, 16, 64);
}

// workgroups of one XCD (equal launch index mod 8) take whole heads, so a head's k, k_r and v rows stay in one L2
__device__ __forceinline__ void block_map(int& bh, int& blk) {
  const int nb = gridDim.x, nbh = gridDim.y;
  if (nbh % 8 != 0) { bh = blockIdx.y; blk = blockIdx.x; return; }
  const int id = blockIdx.x + nb * blockIdx.y;
  const int xcd = id & 7, k = id >> 3;
  bh = (k / nb) * 8 + xcd;
  blk = k % nb;
}

// meta[b][rb][kt][lane][e]: bit 0 = mask != 0, bit 1 = segment bit of query row rb*32 + acc_row(e, lane/32) and key
// kt*32 + lane%32: the 16 bytes a lane needs for one tile, in the order of its accumulator registers
__global__ __launch_bounds__(256) void xl_pack_meta_kernel(int Q, int QQ, int K, int B, const float* __restrict__ mask,
                                                          const uint8_t* __restrict__ seg, u32x4* __restrict__ meta) {
  const int KT = K >> 5, RB = QQ >> 5;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)B * RB * KT * 64) return;
  const int lane = (int)(idx & 63), half = lane >> 5, il = lane & 31;
  const int kt = (int)((idx >> 6) % KT), rb = (int)((idx >> 6) / KT % RB), b = (int)((idx >> 6) / ((int64_t)KT * RB));
  const int j = kt * 32 + il;
  u32x4 out = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int ii = rb * 32 + acc_row(e, half), i = ii % Q;
    uint32_t bits = 0;
    if (mask && mask[((int64_t)ii * K + j) * B + b] != 0.f) bits |= 1u;
    if (seg && seg[((int64_t)i * K + j) * B + b]) bits |= 2u;
    out[e >> 2] |= bits << (8 * (e & 3));
  }
  meta[idx] = out;
}

// nseg[b][i] = number of keys in the other segment (seg bit set) of query row i
__global__ __launch_bounds__(256) void xl_seg_count_kernel(int Q, int K, int B, const uint8_t* __restrict__ seg, float* __restrict__ nseg) {
  const int lane = threadIdx.x & 63;
  const int w = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (w >= Q * B) return;
  const int i = w % Q, b = w / Q;
  float n = 0.f;
  for (int j = lane; j < K; j += 64) n += seg[((int64_t)i * K + j) * B + b] ? 1.f : 0.f;
  n = wave_sum(n);
  if (lane == 0) nseg[w] = n;
}

// this lane's 16-byte MFMA operand slices of one 64-wide row (k index 16 ks + 8 half .. + 7)
__device__ __forceinline__ void load_frags(const bf16* row_ptr, bf16x8 (&f)[4]) {
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) f[ks] = *reinterpret_cast<const bf16x8*>(row_ptr + 16 * ks);
}

// grid (QQ / 32, B * N), 64 * ceil(K / 128) threads
__global__ __launch_bounds__(64 * MAXW) void xl_scores_fwd_kernel(XlScoreArgs a, int prio) {
  ds_wave_prio(prio);
  __shared__ float sm[MAXW][32], sl[MAXW][32];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, il = lane & 31;
  const int nw = blockDim.x >> 6;
  int bh, blk;
  block_map(bh, blk);
  const int b = bh / a.N, hd = bh % a.N;
  const int ii0 = blk * 32, i0 = ii0 % a.Q;
  const int KT = a.K >> 5;
  const int64_t hoff = (int64_t)b * a.H + hd * HD;
  const bf16* qw = reinterpret_cast<const bf16*>(a.qw);
  const bf16* qr = reinterpret_cast<const bf16*>(a.qr);
  const bf16* qs = reinterpret_cast<const bf16*>(a.qs);
  const bf16* kb = reinterpret_cast<const bf16*>(a.k) + (int64_t)b * a.ldk_b + hd * HD + 8 * half;
  const bf16* krb = reinterpret_cast<const bf16*>(a.kr) + hd * HD + 8 * half;
  bf16x8 qwf[4], qrf[4];
  load_frags(qw + (int64_t)(ii0 + il) * a.ldq + hoff + 8 * half, qwf);
  load_frags(qr + (int64_t)(ii0 + il) * a.ldq + hoff + 8 * half, qrf);
  // E: lanes 0..31 hold ef[0] of query row `lane`, lanes 32..63 ef[1] of row lane - 32
  float E = 0.f;
  {
    const bf16* qsp = qs + (int64_t)(ii0 + il) * a.ldq + hoff;
    const float* se = a.seg_emb + (int64_t)half * a.H + hd * HD;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const bf16x8 qv = *reinterpret_cast<const bf16x8*>(qsp + 8 * c);
#pragma unroll
      for (int j = 0; j < 8; ++j) E += (float)qv[j] * se[8 * c + j];
    }
  }
  const float c2 = a.scale * LOG2E;
  float s[NT][16];
  f32x16 raw0;
  const int kt0 = wave * NT;
  {
    // the un-shifted position products of the window's first 32 rows: k_r rows kt0*32 + Q - i0 - 31 + lane
    int r = kt0 * 32 + a.Q - i0 - 31 + il;
    r = r < a.R ? r : a.R - 1;
    bf16x8 krf[4];
    load_frags(krb + (int64_t)r * a.ldkr, krf);
#pragma unroll
    for (int e = 0; e < 16; ++e) raw0[e] = 0.f;
    if (kt0 < KT) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) raw0 = mfma(qrf[ks], krf[ks], raw0);
    }
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int kt = kt0 + t;
    if (kt < KT) {
      const int j0 = kt * 32;
      bf16x8 kf[4], krf[4];
      load_frags(kb + (int64_t)(j0 + il) * a.ldk, kf);
      int r = j0 + a.Q - i0 + 1 + il;   // second half of the window
      r = r < a.R ? r : a.R - 1;
      load_frags(krb + (int64_t)r * a.ldkr, krf);
      u32x4 mw = {0u, 0u, 0u, 0u};
      if (a.meta) mw = reinterpret_cast<const u32x4*>(a.meta)[(((int64_t)b * (a.QQ >> 5) + blk) * KT + kt) * 64 + lane];
      f32x16 ac, raw1;
#pragma unroll
      for (int e = 0; e < 16; ++e) { ac[e] = 0.f; raw1[e] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        ac = mfma(qwf[ks], kf[ks], ac);
        raw1 = mfma(qrf[ks], krf[ks], raw1);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = acc_row(e, half);
        // column u = n + 31 - m of the window is wanted by lane n: lanes u >= 31 - m serve it from the first accumulator
        const float y = il >= 31 - m ? raw0[e] : raw1[e];
        const float bd = lane_read(y, half * 32 + ((il + 31 - m) & 31));
        const uint32_t bits = (mw[e >> 2] >> (8 * (e & 3))) & 3u;
        const float ef = lane_read(E, (int)(bits >> 1) * 32 + m);
        s[t][e] = (ac[e] + bd + ef) * c2 - ((bits & 1u) ? 1e30f : 0.f);
      }
      raw0 = raw1;
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[t][e] = -INFINITY;
    }
  }
  // the wave's own maxima and sums per row, then the block's
  float mx[16], l[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    float v = s[0][e];
#pragma unroll
    for (int t = 1; t < NT; ++t) v = fmaxf(v, s[t][e]);
    mx[e] = half_max(v);
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    float v = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      s[t][e] = kt0 + t < KT ? __builtin_amdgcn_exp2f(s[t][e] - mx[e]) : 0.f;
      v += s[t][e];
    }
    l[e] = half_sum(v);
  }
  if (il == 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      sm[wave][acc_row(e, half)] = mx[e];
      sl[wave][acc_row(e, half)] = l[e];
    }
  }
  __syncthreads();
  if (kt0 >= KT) return;
  float f;
  {
    float M = sm[0][il];
    for (int w = 1; w < nw; ++w) M = fmaxf(M, sm[w][il]);
    float L = 0.f;
    for (int w = 0; w < nw; ++w) L += sl[w][il] * __builtin_amdgcn_exp2f(sm[w][il] - M);
    f = __builtin_amdgcn_exp2f(sm[wave][il] - M) / L;
  }
  bf16* p = reinterpret_cast<bf16*>(a.p) + ((int64_t)bh * a.QQ + ii0) * a.K + il;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int m = acc_row(e, half);
    const float fr = lane_read(f, m);
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (kt0 + t < KT) p[(int64_t)m * a.K + (kt0 + t) * 32] = (bf16)(s[t][e] * fr);
  }
}

// Backward of the same rows: dp = dvec v^T per tile, the row's sum_k p[k] dp[k] over all waves, then ds, its un-shifted
// copy and the two segment sums.  grid and block as the forward kernel.
__global__ __launch_bounds__(64 * MAXW) void xl_scores_bwd_kernel(XlScoreArgs a, int prio) {
  ds_wave_prio(prio);
  __shared__ float sd[MAXW][32], st[MAXW][32], s1[MAXW][32];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, il = lane & 31;
  const int nw = blockDim.x >> 6;
  int bh, blk;
  block_map(bh, blk);
  const int b = bh / a.N, hd = bh % a.N;
  const int ii0 = blk * 32, i0 = ii0 % a.Q;
  const int KT = a.K >> 5;
  const int kt0 = wave * NT;
  const int64_t hoff = (int64_t)b * a.H + hd * HD;
  const bf16* vb = reinterpret_cast<const bf16*>(a.v) + (int64_t)b * a.ldk_b + hd * HD + 8 * half;
  const bf16* p = reinterpret_cast<const bf16*>(a.p) + ((int64_t)bh * a.QQ + ii0) * a.K + il;
  bf16x8 dvf[4];
  load_frags(reinterpret_cast<const bf16*>(a.dvec) + (int64_t)(ii0 + il) * a.ldq + hoff + 8 * half, dvf);
  float dp[NT][16], pp[NT][16], dot[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) dot[e] = 0.f;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int kt = kt0 + t;
    if (kt < KT) {
      bf16x8 vf[4];
      load_frags(vb + (int64_t)(kt * 32 + il) * a.ldk, vf);
#pragma unroll
      for (int e = 0; e < 16; ++e) pp[t][e] = (float)p[(int64_t)acc_row(e, half) * a.K + kt * 32];
      f32x16 acc;
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[e] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) acc = mfma(dvf[ks], vf[ks], acc);
#pragma unroll
      for (int e = 0; e < 16; ++e) { dp[t][e] = acc[e]; dot[e] += pp[t][e] * acc[e]; }
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e) { dp[t][e] = 0.f; pp[t][e] = 0.f; }
    }
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) dot[e] = half_sum(dot[e]);
  if (il == 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) sd[wave][acc_row(e, half)] = dot[e];
  }
  __syncthreads();
  float D = 0.f;
  for (int w = 0; w < nw; ++w) D += sd[w][il];
  float tot[16], d1[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) { dot[e] = lane_read(D, acc_row(e, half)); tot[e] = 0.f; d1[e] = 0.f; }
  bf16* ds = reinterpret_cast<bf16*>(a.ds) + ((int64_t)bh * a.QQ + ii0) * a.K + il;
  // column j of row i lands in column j + Q - i of the un-shifted copy
  bf16* dbd = reinterpret_cast<bf16*>(a.dbd) + ((int64_t)bh * a.QQ + ii0) * a.R + il + a.Q - i0;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int kt = kt0 + t;
    if (kt < KT) {
      u32x4 mw = {0u, 0u, 0u, 0u};
      if (a.meta) mw = reinterpret_cast<const u32x4*>(a.meta)[(((int64_t)b * (a.QQ >> 5) + blk) * KT + kt) * 64 + lane];
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = acc_row(e, half);
        const bf16 val = (bf16)(a.scale * pp[t][e] * (dp[t][e] - dot[e]));
        ds[(int64_t)m * a.K + kt * 32] = val;
        dbd[(int64_t)m * a.R - m + kt * 32] = val;
        const float f = (float)val;
        tot[e] += f;
        if ((mw[e >> 2] >> (8 * (e & 3))) & 2u) d1[e] += f;
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) { tot[e] = half_sum(tot[e]); d1[e] = half_sum(d1[e]); }
  if (il == 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) { st[wave][acc_row(e, half)] = tot[e]; s1[wave][acc_row(e, half)] = d1[e]; }
  }
  __syncthreads();
  if (wave == 0 && half == 0) {
    float T = 0.f, S1 = 0.f;
    for (int w = 0; w < nw; ++w) { T += st[w][il]; S1 += s1[w][il]; }
    // A softmax row's score gradients sum to zero; what the rounded probabilities and the rounded ds leave of that sum is
    // noise that would be multiplied by a whole embedding row: it is taken out of the two segment sums in proportion to the
    // number of keys each one covers.
    const float n1 = a.nseg ? a.nseg[b * a.Q + i0 + il] : 0.f;
    const float excess = T / (float)a.K;
    const float o0 = (T - S1) - excess * ((float)a.K - n1);
    const float o1 = S1 - excess * n1;
    *reinterpret_cast<f32x2*>(a.defs + ((int64_t)bh * a.QQ + ii0 + il) * 2) = f32x2{o0, o1};
  }
}


}  // namespace

bool ds_xl_scores_fit(int dtype, int head_dim, int Q, int K, int R) {
  return dtype == DS_BF16 && head_dim == HD && Q > 0 && Q % 32 == 0 && K >= 32 && K % 32 == 0 && K <= 32 * NT * MAXW && R == K + Q;
}

size_t ds_xl_meta_bytes(int QQ, int K, int B) { return (size_t)B * QQ * K; }

int ds_xl_pack_meta(int Q, int QQ, int K, int B, const float* mask, const uint8_t* seg, void* meta, float* nseg, hipStream_t s) {
  DS_CHECK_ARG(Q > 0 && QQ % Q == 0 && Q % 32 == 0 && K % 32 == 0 && B > 0 && meta && ds_aligned16(meta), "ds_xl_pack_meta: bad shape or pointer");
  const int64_t n = (int64_t)B * (QQ / 32) * (K / 32) * 64;
  hipLaunchKernelGGL(xl_pack_meta_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, Q, QQ, K, B, mask, seg, (u32x4*)meta);
  if (nseg && seg) hipLaunchKernelGGL(xl_seg_count_kernel, dim3((unsigned)((Q * B + 3) / 4)), dim3(256), 0, s, Q, K, B, seg, nseg);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

static int xl_scores_check(const char* who, const XlScoreArgs* a) {
  DS_CHECK_ARG(a && a->N > 0 && a->H == a->N * HD && ds_xl_scores_fit(DS_BF16, HD, a->Q, a->K, a->R) && a->QQ % a->Q == 0 && a->B > 0,
               "%s: shape outside the kernel (Q %d, QQ %d, K %d, R %d, H %d, N %d)", who, a ? a->Q : 0, a ? a->QQ : 0, a ? a->K : 0,
               a ? a->R : 0, a ? a->H : 0, a ? a->N : 0);
  DS_CHECK_ARG((int64_t)a->B * a->N <= 65535, "%s: batch * heads exceeds 65535", who);
  DS_CHECK_ARG(a->ldq % 8 == 0 && a->ldk % 8 == 0 && a->ldk_b % 8 == 0 && a->ldkr % 8 == 0, "%s: strides must be multiples of 8", who);
  return DS_OK;
}

int ds_xl_scores_fwd(const XlScoreArgs* a, hipStream_t s) {
  DS_PROPAGATE(xl_scores_check("ds_xl_scores_fwd", a));
  DS_CHECK_ARG(a->qw && a->qr && a->qs && a->k && a->kr && a->seg_emb && a->p, "ds_xl_scores_fwd: null pointer");
  DS_CHECK_ARG(ds_aligned16(a->qw) && ds_aligned16(a->qr) && ds_aligned16(a->qs) && ds_aligned16(a->k) && ds_aligned16(a->kr) &&
               ds_aligned16(a->meta), "ds_xl_scores_fwd: operands must be 16-byte aligned");
  const int nw = (a->K / 32 + NT - 1) / NT;
  // q k^T once, q k_r^T over 5 window tiles per 4 key tiles
  ds_prof_scope prof(s, "xl_scores_fwd_kernel", 2.0 * (1.0 + 1.25) * a->B * a->N * (double)a->QQ * a->K * HD, "FLOP");
  hipLaunchKernelGGL(xl_scores_fwd_kernel, dim3(a->QQ / 32, a->B * a->N), dim3(64 * nw), 0, s, *a, ds_launch_prio);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

int ds_xl_scores_bwd(const XlScoreArgs* a, hipStream_t s) {
  DS_PROPAGATE(xl_scores_check("ds_xl_scores_bwd", a));
  DS_CHECK_ARG(a->dvec && a->v && a->p && a->ds && a->dbd && a->defs, "ds_xl_scores_bwd: null pointer");
  DS_CHECK_ARG(ds_aligned16(a->dvec) && ds_aligned16(a->v) && ds_aligned16(a->meta) && (reinterpret_cast<uintptr_t>(a->defs) & 7) == 0,
               "ds_xl_scores_bwd: operands must be 16-byte aligned");
  const int nw = (a->K / 32 + NT - 1) / NT;
  ds_prof_scope prof(s, "xl_scores_bwd_kernel", (double)a->B * a->N * a->QQ * (3.0 * a->K * 2 + 0.0), "B");
  hipLaunchKernelGGL(xl_scores_bwd_kernel, dim3(a->QQ / 32, a->B * a->N), dim3(64 * nw), 0, s, *a, ds_launch_prio);
  DS_CHECK_LAUNCH();
  return DS_OK;
}
