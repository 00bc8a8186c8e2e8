// Scores and softmax of XLNet's relative attention without the fp32 score matrices (xlnet/layers/rel_multihead_attn.py:71-115,
// the relative shift of xlnet/layers/lambda_funcs.py:85-93), bf16 with head size 64.  For a stacked query row i' (stream * Q + i),
// sample b and head n
//   score[j] = (qw[i'] . k[j] + qr[i'] . kr[j + Q - i] + ef[seg(i, j, b)]) * scale - 1e30 * mask[i'][j][b],   p = softmax_j score
// and, backward, with dp[j] = dvec[i'] . v[j]:
//   ds[j] = scale * p[j] * (dp[j] - sum_k p[k] dp[k]),  dbd[i'][j + Q - i] = ds[j],  def[s] = sum_j [seg == s] ds[j].
// A block owns 16 query rows and ALL keys of one (b, n): wave w keeps the scores of keys [128 w, 128 w + 128) in registers
// (eight 16x16 MFMA accumulators: keys across the 16 lanes of a lane group, four query rows per lane group down the
// registers), so a row's softmax needs one pass and the only thing written is the bf16 probability (forward) or the bf16
// score gradients (backward).  At about 110 registers a wave, four waves share a SIMD and two blocks a CU.
// The relative shift in that orientation: the position product is computed UN-shifted for the 32 consecutive k_r rows a
// 16 x 16 tile can touch (two accumulators, the second one shared with the next key tile), and the element of row m, key
// column n is column n + 15 - m of that window - for a fixed register (fixed m within the lane group) a rotation of the
// group's lanes, i.e. one ds_bpermute after the source lanes picked the accumulator they are asked for.
// Key, position and value rows reach the MFMA operand registers through LDS: a lane-per-row load straight into operand order
// is one 16-byte request per lane to the vector cache (64 per instruction, four times what contiguous lanes cost), which made
// the cache's request rate the limit of both kernels.  Every wave stages its own 16-row tiles (LDS DMA, eight lanes per row,
// chunks XOR-swizzled by the row, two stages) and reads them back in operand order; no barrier is involved.
// Of the two segment scores only their difference matters (a softmax row ignores a constant), and the mask / segment bits
// of a lane's 32 scores are two 32-bit words, turned into addends with a bit-field extract and an AND each.
#include <string.h>

#include "common.h"
#include "stage.h"

namespace {

constexpr int HD = 64;    // head size
constexpr int RB = 16;    // query rows per block
constexpr int NT = 8;     // key tiles (of 16 keys) per wave
constexpr int MAXW = 8;   // waves per block: up to 16 * NT * MAXW = 1024 keys
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
__device__ __forceinline__ float lane_read(float v, int byte_addr) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(byte_addr, __builtin_bit_cast(int, v)));
}
// x where bit `idx` of `bits` is set, else 0
__device__ __forceinline__ float bit_select(uint32_t bits, int idx, float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_sbfe((int)bits, idx, 1) & __builtin_bit_cast(int, x));
}
// reductions over the 16 lanes of a lane group (the keys of one tile row): DPP moves only
__device__ __forceinline__ float group_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));
  v = fmaxf(v, dpp_move<0x4E>(v));
  v = fmaxf(v, dpp_move<0x141>(v));
  return fmaxf(v, dpp_move<0x140>(v));
}
__device__ __forceinline__ float group_sum(float v) {
  v += dpp_move<0xB1>(v);
  v += dpp_move<0x4E>(v);
  v += dpp_move<0x141>(v);
  return v + dpp_move<0x140>(v);
}

// Two accumulator registers of a lane (rows m and m + 1 of its key column n) against one bf16 pair per lane: even lanes hold
// row m, keys (n, n + 1), odd lanes row m + 1, keys (n - 1, n) - so that a 32-bit access per lane covers what two 16-bit
// accesses would.  The lanes of a pair swap one value through a DPP move.
__device__ __forceinline__ uint32_t pair_pack(float a, float b, bool odd) {
  const float recv = dpp_move<0xB1>(odd ? a : b);
  const bf16x2 v = {(bf16)(odd ? recv : a), (bf16)(odd ? b : recv)};
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ void pair_unpack(uint32_t w, bool odd, float& a, float& b) {
  const float lo = __builtin_bit_cast(float, w << 16), hi = __builtin_bit_cast(float, w & 0xffff0000u);
  const float recv = dpp_move<0xB1>(odd ? lo : hi);
  a = odd ? recv : lo;
  b = odd ? hi : recv;
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

// meta[b][rb][w][lane] = (mask bits, segment bits) of the 32 scores that lane `lane` of wave w holds for row block rb:
// bit 4 t + v belongs to query row rb*16 + 4 (lane/16) + v and key w*128 + t*16 + lane%16
__global__ __launch_bounds__(256) void xl_pack_meta_kernel(int Q, int QQ, int K, int B, const float* __restrict__ mask,
                                                          const uint8_t* __restrict__ seg, uint2* __restrict__ meta) {
  const int NW = (K + 127) >> 7, NRB = QQ / RB;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)B * NRB * NW * 64) return;
  const int lane = (int)(idx & 63), g = lane >> 4, n = lane & 15;
  const int w = (int)((idx >> 6) % NW), rb = (int)((idx >> 6) / NW % NRB), b = (int)((idx >> 6) / ((int64_t)NW * NRB));
  uint32_t mb = 0, sb = 0;
  for (int t = 0; t < NT; ++t) {
    const int j = w * 128 + t * 16 + n;
    if (j >= K) break;
    for (int v = 0; v < 4; ++v) {
      const int ii = rb * RB + 4 * g + v, i = ii % Q;
      if (mask && mask[((int64_t)ii * K + j) * B + b] != 0.f) mb |= 1u << (4 * t + v);
      if (seg && seg[((int64_t)i * K + j) * B + b]) sb |= 1u << (4 * t + v);
    }
  }
  meta[idx] = make_uint2(mb, sb);
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

typedef __attribute__((address_space(3))) void* lds_vptr;
typedef __attribute__((address_space(1))) void* glb_vptr;
constexpr int TILE_BYTES = 16 * HD * 2;   // 16 rows of 64 bf16
// vmcnt(n): at most n of this wave's vector-memory operations still in flight
__device__ __forceinline__ void wait_vm4() { __builtin_amdgcn_s_waitcnt((4 & 15) | (7 << 4) | (15 << 8)); }
__device__ __forceinline__ void wait_vm0() { __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8)); }
// Before a stage is handed to the DMA again every LDS read of it must have RETURNED: LDS DMA writes do not queue behind the
// wave's ds_read instructions, and the compiler, which orders the two only by issue, otherwise moves the next request above
// the wait that completes the previous tile's last read.
__device__ __forceinline__ void stage_free() {
  __builtin_amdgcn_s_waitcnt(15 | (3 << 14) | (7 << 4) | (0 << 8));   // lgkmcnt(0)
  __builtin_amdgcn_sched_barrier(0);
}
// LDS tile: [16 rows][8 chunks of 16 bytes], chunk index XOR-swizzled by the row so that the 16 lanes reading one chunk
// column of 16 rows spread over the banks (64 banks: a 256-byte line is two rows)
__device__ __forceinline__ int tile_swz(int row) {
  const int t = (row >> 1) & 7;
  return ((t & 1) << 2) | (t >> 1);
}
// rows row0 .. row0 + 15 (clamped to last_row) of a row-major matrix, 64 columns from `base` -> one LDS tile; two instructions,
// eight lanes per row
__device__ __forceinline__ void tile16_fill(char* lds, const bf16* base, int64_t ld, int row0, int last_row, int lane) {
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int r = c * 8 + (lane >> 3), pc = lane & 7;
    int gr = row0 + r;
    gr = gr < last_row ? gr : last_row;
    const bf16* src = base + (int64_t)gr * ld + (pc ^ tile_swz(r)) * 8;
    __builtin_amdgcn_global_load_lds((glb_vptr)src, (lds_vptr)(lds + c * 1024), 16, 0, 0);
  }
}
// MFMA operand slices of lane (g, n) from a tile: row n, k index 32 ks + 8 g .. + 7
__device__ __forceinline__ void tile16_frags(const char* lds, int g, int n, bf16x8 (&f)[2]) {
  const char* row = lds + n * (HD * 2);
  const int z = tile_swz(n);
  f[0] = *reinterpret_cast<const bf16x8*>(row + ((g ^ z) << 4));
  f[1] = *reinterpret_cast<const bf16x8*>(row + (((g + 4) ^ z) << 4));
}

// qw, qr, qs = q + r_w, q + r_r, q + r_s (bf16) for one row [H] per wave, and de[b][n][i'] = qs . (seg_emb[1] - seg_emb[0]) over
// head n's 64 columns: the difference of the row's two segment scores, from the ROUNDED qs like every other use of it.
// A lane owns 8 consecutive columns, so a head is 8 lanes.
__global__ __launch_bounds__(256) void xl_bias_q_de_kernel(int rows, int B, int N, int QQ, const bf16* __restrict__ q,
                                                          const float* __restrict__ rw, const float* __restrict__ rr,
                                                          const float* __restrict__ rs, const float* __restrict__ seg_emb,
                                                          bf16* __restrict__ qw, bf16* __restrict__ qr, bf16* __restrict__ qs,
                                                          float* __restrict__ de) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);   // row ii * B + b
  if (r >= rows) return;
  const int ii = r / B, b = r % B, H = N * HD;
  for (int c0 = lane * 8; c0 < H; c0 += 512) {
    const bf16x8 x = *reinterpret_cast<const bf16x8*>(q + (int64_t)r * H + c0);
    bf16x8 ow, orr, os;
    float d = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const f32x4 bw = *reinterpret_cast<const f32x4*>(rw + c0 + 4 * h), br = *reinterpret_cast<const f32x4*>(rr + c0 + 4 * h);
      const f32x4 bs = *reinterpret_cast<const f32x4*>(rs + c0 + 4 * h);
      const f32x4 s0 = *reinterpret_cast<const f32x4*>(seg_emb + c0 + 4 * h), s1 = *reinterpret_cast<const f32x4*>(seg_emb + H + c0 + 4 * h);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float v = (float)x[4 * h + j];
        ow[4 * h + j] = (bf16)(v + bw[j]);
        orr[4 * h + j] = (bf16)(v + br[j]);
        os[4 * h + j] = (bf16)(v + bs[j]);
        d += (float)os[4 * h + j] * (s1[j] - s0[j]);
      }
    }
    *reinterpret_cast<bf16x8*>(qw + (int64_t)r * H + c0) = ow;
    *reinterpret_cast<bf16x8*>(qr + (int64_t)r * H + c0) = orr;
    *reinterpret_cast<bf16x8*>(qs + (int64_t)r * H + c0) = os;
    d += dpp_move<0xB1>(d);    // lane ^ 1
    d += dpp_move<0x4E>(d);    // lane ^ 2
    d += dpp_move<0x141>(d);   // mirror within 8 lanes: the other quad
    if ((lane & 7) == 0) de[((int64_t)b * N + c0 / HD) * QQ + ii] = d;
  }
}

// this lane's two 16-byte MFMA operand slices of one 64-wide row (k index 32 ks + 8 (lane / 16) .. + 7; row_ptr includes 8 (lane / 16))
__device__ __forceinline__ void load_frags(const bf16* row_ptr, bf16x8 (&f)[2]) {
  f[0] = *reinterpret_cast<const bf16x8*>(row_ptr);
  f[1] = *reinterpret_cast<const bf16x8*>(row_ptr + 32);
}

// grid (QQ / 16, B * N), 64 * ceil(K / 128) threads.  FULL: K is a multiple of 128, so every wave has all its tiles; META: mask /
// segment bits exist.
template <bool FULL, bool META>
__global__ __launch_bounds__(64 * MAXW) void xl_scores_fwd_kernel(XlScoreArgs a, int prio) {
  ds_wave_prio(prio);
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), g = lane >> 4, n = lane & 15;
  const int nw = blockDim.x >> 6;
  int bh, blk;
  block_map(bh, blk);
  const int b = bh / a.N, hd = bh % a.N;
  const int ii0 = blk * RB, i0 = ii0 % a.Q;
  const int KT = a.K >> 4;
  const int kt0 = wave * NT;
  const int64_t qoff = (int64_t)(ii0 + n) * a.ldq + (int64_t)b * a.H + hd * HD;
  const bf16* kb = reinterpret_cast<const bf16*>(a.k) + (int64_t)b * a.ldk_b + hd * HD;
  const bf16* krb = reinterpret_cast<const bf16*>(a.kr) + hd * HD;
  // the per-wave maxima and sums meet in the first 128 bytes of every wave's own stage area, once its tiles are done with:
  // the block then needs exactly 8 KB per wave, and two blocks of 7 waves leave room for a 48 KB GEMM block on the CU
  auto sm = [&](int w) { return reinterpret_cast<float*>(lds + w * 4 * TILE_BYTES); };
  auto sl = [&](int w) { return reinterpret_cast<float*>(lds + w * 4 * TILE_BYTES) + RB; };
  char* stage = lds + wave * 4 * TILE_BYTES;   // two stages of (key tile, position tile)
  // The tile loop has no branches: tiles past the last key stage clamped rows and their scores are replaced below.  The
  // next tile's rows are requested before the current tile is worked on.
  auto request = [&](int t) {
    char* st = stage + (t & 1) * 2 * TILE_BYTES;
    tile16_fill(st, kb, a.ldk, (kt0 + t) * 16, a.K - 1, lane);
    tile16_fill(st + TILE_BYTES, krb, a.ldkr, (kt0 + t) * 16 + a.Q - i0 + 1, a.R - 1, lane);   // second half of the window
  };
  bf16x8 qwf[2], qrf[2], f0[2];
  load_frags(reinterpret_cast<const bf16*>(a.qr) + qoff + 8 * g, qrf);
  {
    int r = kt0 * 16 + a.Q - i0 - 15 + n;   // first half of the first window
    if (!FULL) r = r < a.R ? r : a.R - 1;
    load_frags(krb + (int64_t)r * a.ldkr + 8 * g, f0);
  }
  load_frags(reinterpret_cast<const bf16*>(a.qw) + qoff + 8 * g, qwf);
  request(0);
  // de[v]: ef[1] - ef[0] of this lane's query row 4 g + v (a row's softmax ignores ef[0]), from ds_xl_bias_q
  float de[4] = {0.f, 0.f, 0.f, 0.f};
  uint32_t mbits = 0, sbits = 0;
  if (META) {
    const uint2 mw = reinterpret_cast<const uint2*>(a.meta)[(((int64_t)b * (a.QQ / RB) + blk) * nw + wave) * 64 + lane];
    mbits = mw.x; sbits = mw.y;
    const f32x4 dv = *reinterpret_cast<const f32x4*>(a.de + ((int64_t)b * a.N + hd) * a.QQ + ii0 + 4 * g);
#pragma unroll
    for (int v = 0; v < 4; ++v) de[v] = dv[v];
  }
  // column u = n + 15 - m of a tile's window is wanted by lane n of the group: the lane holding it is 16 g + (u & 15), and
  // that lane serves it from the window's first accumulator when its own column is >= 15 - m
  int rot[4];
  bool first[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int m = 4 * g + v;
    rot[v] = (16 * g + ((n + 15 - m) & 15)) << 2;
    asm volatile("" : "+v"(rot[v]));   // computed once, not once per tile
    first[v] = n >= 15 - m;
  }
  const float c2 = a.scale * LOG2E;
  float s[NT][4];
  f32x4 raw0 = {0.f, 0.f, 0.f, 0.f};
  raw0 = mfma16(qrf[0], f0[0], raw0);
  raw0 = mfma16(qrf[1], f0[1], raw0);
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    stage_free();
    if (t + 1 < NT) { request(t + 1); wait_vm4(); } else wait_vm0();   // tile t has landed; only tile t + 1 may be in flight
    const char* st = stage + (t & 1) * 2 * TILE_BYTES;
    bf16x8 kf[2], krf[2];
    tile16_frags(st, g, n, kf);
    tile16_frags(st + TILE_BYTES, g, n, krf);
    f32x4 ac = {0.f, 0.f, 0.f, 0.f}, raw1 = {0.f, 0.f, 0.f, 0.f};
    ac = mfma16(qwf[0], kf[0], ac);
    raw1 = mfma16(qrf[0], krf[0], raw1);
    ac = mfma16(qwf[1], kf[1], ac);
    raw1 = mfma16(qrf[1], krf[1], raw1);
    float bd[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) bd[v] = lane_read(first[v] ? raw0[v] : raw1[v], rot[v]);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float x = ac[v] + bd[v];
      if (META) {
        x += bit_select(sbits, 4 * t + v, de[v]);
        s[t][v] = fmaf(x, c2, bit_select(mbits, 4 * t + v, -1e30f));
      } else {
        s[t][v] = x * c2;
      }
    }
    raw0 = raw1;
  }
  // the wave's own maxima and sums per row, then the block's
  const float dead = -INFINITY;   // tiles past the last key
  float mx[4], l[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    float x = s[0][v];
#pragma unroll
    for (int t = 1; t < NT; ++t) x = fmaxf(x, FULL || kt0 + t < KT ? s[t][v] : dead);
    mx[v] = group_max(x);
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    float x = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      s[t][v] = FULL || kt0 + t < KT ? __builtin_amdgcn_exp2f(s[t][v] - mx[v]) : 0.f;
      x += s[t][v];
    }
    l[v] = group_sum(x);
  }
  // (a wave of a block always has its first tile: the block has ceil(K / 128) waves)
  if (n == 0) {
#pragma unroll
    for (int v = 0; v < 4; ++v) { sm(wave)[4 * g + v] = mx[v]; sl(wave)[4 * g + v] = l[v]; }
  }
  __syncthreads();
  float f;
  {
    float M = sm(0)[n];
    for (int w = 1; w < nw; ++w) M = fmaxf(M, sm(w)[n]);
    float L = 0.f;
    for (int w = 0; w < nw; ++w) L += sl(w)[n] * __builtin_amdgcn_exp2f(sm(w)[n] - M);
    f = __builtin_amdgcn_exp2f(sm(wave)[n] - M) / L;
  }
  const bool odd = n & 1;
  bf16* p = reinterpret_cast<bf16*>(a.p) + ((int64_t)bh * a.QQ + ii0 + 4 * g + (odd ? 1 : 0)) * a.K + (n & ~1);
#pragma unroll
  for (int v = 0; v < 4; v += 2) {
    const float f0s = lane_read(f, (4 * g + v) << 2), f1s = lane_read(f, (4 * g + v + 1) << 2);
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (FULL || kt0 + t < KT)
        *reinterpret_cast<uint32_t*>(p + (int64_t)v * a.K + (kt0 + t) * 16) = pair_pack(s[t][v] * f0s, s[t][v + 1] * f1s, odd);
  }
}

// Backward of the same rows: dp = dvec v^T per tile, the row's sum_k p[k] dp[k] over all waves, then ds, its un-shifted
// copy and the two segment sums.  grid and block as the forward kernel.
__global__ __launch_bounds__(64 * MAXW) void xl_scores_bwd_kernel(XlScoreArgs a, int prio) {
  ds_wave_prio(prio);
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), g = lane >> 4, n = lane & 15;
  const int nw = blockDim.x >> 6;
  int bh, blk;
  block_map(bh, blk);
  const int b = bh / a.N, hd = bh % a.N;
  const int ii0 = blk * RB, i0 = ii0 % a.Q;
  const int KT = a.K >> 4;
  const int kt0 = wave * NT;
  const bool odd = n & 1;
  const bf16* vb = reinterpret_cast<const bf16*>(a.v) + (int64_t)b * a.ldk_b + hd * HD;
  float (*sd)[RB] = reinterpret_cast<float (*)[RB]>(lds + nw * 2 * TILE_BYTES);
  float (*st)[RB] = sd + MAXW;
  float (*s1)[RB] = st + MAXW;
  char* stage = lds + wave * 2 * TILE_BYTES;   // two stages of a value tile
  const bf16* p = reinterpret_cast<const bf16*>(a.p) + ((int64_t)bh * a.QQ + ii0 + 4 * g + (odd ? 1 : 0)) * a.K + (n & ~1);
  bf16x8 dvf[2];
  load_frags(reinterpret_cast<const bf16*>(a.dvec) + (int64_t)(ii0 + n) * a.ldq + (int64_t)b * a.H + hd * HD + 8 * g, dvf);
  uint32_t sbits = 0;
  if (a.meta) sbits = reinterpret_cast<const uint2*>(a.meta)[(((int64_t)b * (a.QQ / RB) + blk) * nw + wave) * 64 + lane].y;
  float dp[NT][4], pp[NT][4], dot[4] = {0.f, 0.f, 0.f, 0.f};
  uint32_t pw[2][2];
  // (no branches in the tile loop: tiles past the last key read the last tile again and count as zeros)
  auto request = [&](int t) {
    const int kt = kt0 + t < KT ? kt0 + t : KT - 1;
    tile16_fill(stage + (t & 1) * TILE_BYTES, vb, a.ldk, kt * 16, a.K - 1, lane);
    pw[t & 1][0] = *reinterpret_cast<const uint32_t*>(p + kt * 16);
    pw[t & 1][1] = *reinterpret_cast<const uint32_t*>(p + 2 * (int64_t)a.K + kt * 16);
  };
  request(0);
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    {
      stage_free();
      if (t + 1 < NT) { request(t + 1); wait_vm4(); } else wait_vm0();   // tile t (two tile loads, two probability loads) has landed
      bf16x8 vf[2];
      tile16_frags(stage + (t & 1) * TILE_BYTES, g, n, vf);
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      acc = mfma16(dvf[0], vf[0], acc);
      acc = mfma16(dvf[1], vf[1], acc);
      pair_unpack(pw[t & 1][0], odd, pp[t][0], pp[t][1]);
      pair_unpack(pw[t & 1][1], odd, pp[t][2], pp[t][3]);
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        if (kt0 + t >= KT) pp[t][v] = 0.f;
        dp[t][v] = acc[v];
        dot[v] = fmaf(pp[t][v], acc[v], dot[v]);
      }
    }
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) dot[v] = group_sum(dot[v]);
  if (n == 0) {
#pragma unroll
    for (int v = 0; v < 4; ++v) sd[wave][4 * g + v] = dot[v];
  }
  __syncthreads();
  float D = 0.f;
  for (int w = 0; w < nw; ++w) D += sd[w][n];
  float tot[4], d1[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) { dot[v] = lane_read(D, (4 * g + v) << 2); tot[v] = 0.f; d1[v] = 0.f; }
  bf16* ds = reinterpret_cast<bf16*>(a.ds) + ((int64_t)bh * a.QQ + ii0 + 4 * g + (odd ? 1 : 0)) * a.K + (n & ~1);
  // column j of row i lands in column j + Q - i of the un-shifted copy
  bf16* dbd = reinterpret_cast<bf16*>(a.dbd) + ((int64_t)bh * a.QQ + ii0 + 4 * g) * a.R + n + a.Q - i0 - 4 * g;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (kt0 + t < KT) {
      const int kt = kt0 + t;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const bf16 val = (bf16)(a.scale * pp[t][v] * (dp[t][v] - dot[v]));
        dbd[(int64_t)v * a.R - v + kt * 16] = val;
        const float f = (float)val;
        pp[t][v] = f;
        tot[v] += f;
        d1[v] += bit_select(sbits, 4 * t + v, f);
      }
      *reinterpret_cast<uint32_t*>(ds + kt * 16) = pair_pack(pp[t][0], pp[t][1], odd);
      *reinterpret_cast<uint32_t*>(ds + 2 * (int64_t)a.K + kt * 16) = pair_pack(pp[t][2], pp[t][3], odd);
    }
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) { tot[v] = group_sum(tot[v]); d1[v] = group_sum(d1[v]); }
  if (n == 0) {
#pragma unroll
    for (int v = 0; v < 4; ++v) { st[wave][4 * g + v] = tot[v]; s1[wave][4 * g + v] = d1[v]; }
  }
  __syncthreads();
  if (wave == 0 && g == 0) {
    float T = 0.f, S1 = 0.f;
    for (int w = 0; w < nw; ++w) { T += st[w][n]; S1 += s1[w][n]; }
    // A softmax row's score gradients sum to zero; what the rounded probabilities and the rounded ds leave of that sum is
    // noise that would be multiplied by a whole embedding row: it is taken out of the two segment sums in proportion to the
    // number of keys each one covers.
    const float n1 = a.nseg ? a.nseg[b * a.Q + i0 + n] : 0.f;
    const float excess = T / (float)a.K;
    const float o0 = (T - S1) - excess * ((float)a.K - n1);
    const float o1 = S1 - excess * n1;
    *reinterpret_cast<f32x2*>(a.defs + ((int64_t)bh * a.QQ + ii0 + n) * 2) = f32x2{o0, o1};
  }
}

}  // namespace

bool ds_xl_scores_fit(int dtype, int head_dim, int Q, int K, int R) {
  return dtype == DS_BF16 && head_dim == HD && Q > 0 && Q % RB == 0 && K >= 16 && K % 16 == 0 && K <= 16 * NT * MAXW && R == K + Q;
}

size_t ds_xl_meta_bytes(int QQ, int K, int B) { return (size_t)B * (QQ / RB) * ((K + 127) / 128) * 64 * sizeof(uint2); }

int ds_xl_pack_meta(int Q, int QQ, int K, int B, const float* mask, const uint8_t* seg, void* meta, float* nseg, hipStream_t s) {
  DS_CHECK_ARG(Q > 0 && QQ % Q == 0 && Q % RB == 0 && K % 16 == 0 && B > 0 && meta && ds_aligned16(meta), "ds_xl_pack_meta: bad shape or pointer");
  const int64_t n = (int64_t)B * (QQ / RB) * ((K + 127) / 128) * 64;
  hipLaunchKernelGGL(xl_pack_meta_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, Q, QQ, K, B, mask, seg, (uint2*)meta);
  if (nseg && seg) hipLaunchKernelGGL(xl_seg_count_kernel, dim3((unsigned)((Q * B + 3) / 4)), dim3(256), 0, s, Q, K, B, seg, nseg);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

int ds_xl_bias_q(int rows, int B, int N, const void* q, const float* rw, const float* rr, const float* rs, const float* seg_emb,
                 void* qw, void* qr, void* qs, float* de, hipStream_t s) {
  DS_CHECK_ARG(rows > 0 && B > 0 && N > 0 && q && rw && rr && rs && seg_emb && qw && qr && qs && de, "ds_xl_bias_q: bad argument");
  DS_CHECK_ARG(ds_aligned16(q) && ds_aligned16(rw) && ds_aligned16(rr) && ds_aligned16(rs) && ds_aligned16(seg_emb) && ds_aligned16(qw) &&
               ds_aligned16(qr) && ds_aligned16(qs), "ds_xl_bias_q: operands must be 16-byte aligned");
  hipLaunchKernelGGL(xl_bias_q_de_kernel, dim3((unsigned)((rows * B + 3) / 4)), dim3(256), 0, s, rows * B, B, N, rows, (const bf16*)q, rw, rr, rs,
                     seg_emb, (bf16*)qw, (bf16*)qr, (bf16*)qs, de);
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
  DS_CHECK_ARG(a->qw && a->qr && a->k && a->kr && a->p && (a->de || !a->meta), "ds_xl_scores_fwd: null pointer");
  DS_CHECK_ARG(ds_aligned16(a->qw) && ds_aligned16(a->qr) && ds_aligned16(a->de) && ds_aligned16(a->k) && ds_aligned16(a->kr) &&
               ds_aligned16(a->meta), "ds_xl_scores_fwd: operands must be 16-byte aligned");
  const int nw = (a->K + 127) / 128;
  // q k^T once, q k_r^T over 9 window tiles per 8 key tiles
  ds_prof_scope prof(s, "xl_scores_fwd_kernel", 2.0 * (1.0 + 1.125) * a->B * a->N * (double)a->QQ * a->K * HD, "FLOP");
  const dim3 grid(a->QQ / RB, a->B * a->N), block(64 * nw);
  const bool full = a->K % 128 == 0;
  const size_t lds = (size_t)nw * 4 * TILE_BYTES;
  static std::atomic<bool> attr(false);  // two threads may both set the (idempotent) attribute; neither launches before it is set
  if (!attr) {
    const int most = MAXW * 4 * TILE_BYTES;
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)xl_scores_fwd_kernel<true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, most));
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)xl_scores_fwd_kernel<true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, most));
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)xl_scores_fwd_kernel<false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, most));
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)xl_scores_fwd_kernel<false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, most));
    attr = true;
  }
  if (full && a->meta) hipLaunchKernelGGL((xl_scores_fwd_kernel<true, true>), grid, block, lds, s, *a, ds_launch_prio);
  else if (full) hipLaunchKernelGGL((xl_scores_fwd_kernel<true, false>), grid, block, lds, s, *a, ds_launch_prio);
  else if (a->meta) hipLaunchKernelGGL((xl_scores_fwd_kernel<false, true>), grid, block, lds, s, *a, ds_launch_prio);
  else hipLaunchKernelGGL((xl_scores_fwd_kernel<false, false>), grid, block, lds, s, *a, ds_launch_prio);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

int ds_xl_scores_bwd(const XlScoreArgs* a, hipStream_t s) {
  DS_PROPAGATE(xl_scores_check("ds_xl_scores_bwd", a));
  DS_CHECK_ARG(a->dvec && a->v && a->p && a->ds && a->dbd && a->defs, "ds_xl_scores_bwd: null pointer");
  DS_CHECK_ARG(ds_aligned16(a->dvec) && ds_aligned16(a->v) && ds_aligned16(a->meta) && (reinterpret_cast<uintptr_t>(a->defs) & 7) == 0,
               "ds_xl_scores_bwd: operands must be 16-byte aligned");
  const int nw = (a->K + 127) / 128;
  ds_prof_scope prof(s, "xl_scores_bwd_kernel", (double)a->B * a->N * a->QQ * (3.0 * a->K * 2 + 0.0), "B");
  hipLaunchKernelGGL(xl_scores_bwd_kernel, dim3(a->QQ / RB, a->B * a->N), dim3(64 * nw), (size_t)nw * 2 * TILE_BYTES + 3 * MAXW * RB * sizeof(float), s,
                     *a, ds_launch_prio);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

// ---- the same kernels as operators of the C ABI (dense layouts: q rows [QQ][B][H], kv rows [K][B][2H], kr rows [R][H])
static void xl_dense_args(XlScoreArgs& a, int seq, int rows, int klen, int batch, int heads, float scale) {
  memset(&a, 0, sizeof(a));
  const int H = heads * HD;
  a.ldq = (int64_t)batch * H; a.ldk = (int64_t)batch * 2 * H; a.ldk_b = 2 * H; a.ldkr = H;
  a.Q = seq; a.QQ = rows; a.K = klen; a.R = klen + seq; a.B = batch; a.N = heads; a.H = H; a.scale = scale;
}

extern "C" size_t ds_xlnet_scores_meta_bytes(int rows, int klen, int batch) {
  return rows > 0 && klen > 0 && batch > 0 ? ds_xl_meta_bytes(rows, klen, batch) : 0;
}

extern "C" int ds_xlnet_scores_pack(int seq, int rows, int klen, int batch, const float* masks, const uint8_t* seg_mat, void* meta,
                                    float* nseg, void* stream) {
  DS_CHECK_ARG(ds_xl_scores_fit(DS_BF16, HD, seq, klen, klen + seq), "ds_xlnet_scores_pack: seq %d / klen %d outside the kernels", seq, klen);
  return ds_xl_pack_meta(seq, rows, klen, batch, masks, seg_mat, meta, nseg, (hipStream_t)stream);
}

extern "C" int ds_xlnet_bias_q(int rows, int batch, int heads, const void* q, const float* bias_context, const float* bias_relative,
                               const float* bias_segment, const float* seg_emb, void* qw, void* qr, void* qs, float* de, void* stream) {
  return ds_xl_bias_q(rows, batch, heads, q, bias_context, bias_relative, bias_segment, seg_emb, qw, qr, qs, de, (hipStream_t)stream);
}

extern "C" int ds_xlnet_scores_fwd(int seq, int rows, int klen, int batch, int heads, const void* qw, const void* qr, const float* de,
                                   const void* kv, const void* kr, const void* meta, float scale, void* p, void* stream) {
  DS_CHECK_ARG(heads > 0 && batch > 0, "ds_xlnet_scores_fwd: non-positive shape");
  XlScoreArgs a;
  xl_dense_args(a, seq, rows, klen, batch, heads, scale);
  a.qw = qw; a.qr = qr; a.de = de; a.k = kv; a.kr = kr; a.meta = meta; a.p = p;
  return ds_xl_scores_fwd(&a, (hipStream_t)stream);
}

extern "C" int ds_xlnet_scores_bwd(int seq, int rows, int klen, int batch, int heads, const void* kv, const void* p, const void* dvec,
                                   const void* meta, const float* nseg, float scale, void* ds, void* dbd, float* defs, void* stream) {
  DS_CHECK_ARG(heads > 0 && batch > 0 && kv, "ds_xlnet_scores_bwd: bad argument");
  XlScoreArgs a;
  xl_dense_args(a, seq, rows, klen, batch, heads, scale);
  a.v = (const char*)kv + (size_t)a.H * sizeof(bf16); a.p = (void*)p; a.dvec = dvec; a.meta = meta; a.nseg = nseg;
  a.ds = ds; a.dbd = dbd; a.defs = defs;
  return ds_xl_scores_bwd(&a, (hipStream_t)stream);
}
