// The fused attention kernels of attention.hip as device functions (a workgroup of 512 threads, its dynamic LDS and
// its index among the problem's workgroups), shared by the kernels of their own and the grouped launches of group.hip.
#pragma once
#include "common.h"

namespace dsattn {


typedef __attribute__((address_space(3))) void* lds_vptr;
typedef __attribute__((address_space(1))) void* glb_vptr;
#define VMCNT0 ((0 & 15) | ((0 >> 4) << 14) | (7 << 4) | (15 << 8))

constexpr int HD = 64;        // head size
constexpr int ROWB = 128;     // bytes per tile row (64 bf16)
constexpr int CHUNK = 256;    // rows of K/V (or Q/dO) resident in LDS at a time (XLNet kernel: one buffer of this size)
constexpr int CH = 128;       // BERT kernels: the same 64 KB as two buffers of 128 rows per tensor; chunk c+2 is loaded while
                              // chunk c+1 is multiplied, and a chunk is exactly one 32-row step for each of the SPLIT waves
// A block owns 64 rows of the parallel axis (two groups of 32) and splits the walked axis SPLIT ways:
// wave w works for group (w & 1) on every SPLIT-th 32-row step starting at (w >> 1).  2*SPLIT waves
// give every SIMD two waves, so one wave's softmax arithmetic runs under the other's MFMAs.  The
// partial results are combined through LDS at the end.
constexpr int SPLIT = 4;
constexpr int NWAVES = 2 * SPLIT;
constexpr int NTHREADS = 64 * NWAVES;

// LDS tile layout: row-major [row][64 bf16], the 16-byte chunk index XOR-swizzled by the row.  The
// LDS has 64 banks (a 256-byte line = two tile rows).  The swizzle serves both read patterns:
//   frag_rows: 16 lanes read one chunk column of 16 consecutive rows -> the 8 rows of equal parity
//              need 8 different chunks: any bijection of t = (row >> 1) & 7;
//   frag_cols: 32 lanes read 4 consecutive rows x 4 adjacent chunks -> rows r and r+2 (same half
//              line, t differs in bit 0) must land in different 64-byte quarters: bit 0 of t is
//              moved to bit 2 of the chunk index.
__device__ __forceinline__ int tile_swz(int row) {
  const int t = (row >> 1) & 7;
  return ((t & 1) << 2) | (t >> 1);
}
__device__ __forceinline__ int tile_off(int row, int byte) {
  return row * ROWB + ((((byte >> 4) ^ tile_swz(row))) << 4) + (byte & 15);
}

// Fills `rows` tile rows (multiple of 16) from global rows of stride ld (elements); all waves of the block.
__device__ __forceinline__ void tile_fill(char* lds, const bf16* src, int64_t ld, int rows, int wave, int lane) {
  for (int c = wave; c < rows / 8; c += NWAVES) {  // each call: one wave writes 64 consecutive 16-byte slots = 8 rows
    const int p = c * 64 + lane;
    const int r = p >> 3, pc = p & 7;
    const bf16* s = src + (int64_t)r * ld + (pc ^ tile_swz(r)) * 8;
    __builtin_amdgcn_global_load_lds((glb_vptr)s, (lds_vptr)(lds + c * 1024), 16, 0, 0);
  }
}

// The kernels below never issue another vector-memory load between their prologue and their last chunk, so vmcnt counts
// tile loads only: a thread issues rows / 64 loads per tensor and chunk.  Waits until only the next chunk's loads (two
// tensors of next_rows rows) may still be in flight.
__device__ __forceinline__ void wait_chunk(int next_rows) {
  const int n = next_rows / 32;  // 2 tensors x next_rows / 64
  if (n >= 4) __builtin_amdgcn_s_waitcnt((4 & 15) | (7 << 4) | (15 << 8));
  else if (n >= 2) __builtin_amdgcn_s_waitcnt((2 & 15) | (7 << 4) | (15 << 8));
  else __builtin_amdgcn_s_waitcnt(VMCNT0);
}

// The mask adders of the 16 accumulator rows of a 32-row step (rows (e/4)*8 + 4*half + e%4): four 16-byte LDS reads, or
// zeros without a mask - one uniform branch per step instead of one per element.
__device__ __forceinline__ void step_adders(const float* adder, bool masked, int row0, int half, float (&ad)[16]) {
  if (masked) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(adder + row0 + g * 8 + half * 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) ad[4 * g + j] = v[j];
    }
  } else {
#pragma unroll
    for (int e = 0; e < 16; ++e) ad[e] = 0.f;
  }
}

// A operand, rows = tile rows (row0 + lane%32), k = 8 consecutive columns starting at 16*ks + 8*half
__device__ __forceinline__ bf16x8 frag_rows(const char* lds, int row0, int ks, int lane) {
  return *reinterpret_cast<const bf16x8*>(lds + tile_off(row0 + (lane & 31), (2 * ks + (lane >> 5)) * 16));
}
// A operand of the transposed use: rows = tile columns (col0 + lane%32), k = tile rows in the order the
// accumulator layout hands them over: elements 0-3 -> rows r0 + 4*half + 0..3, elements 4-7 -> r0 + 8 + 4*half + 0..3
__device__ __forceinline__ bf16x8 frag_cols(const char* lds, int r0, int col0, int lane) {
  const int h = lane >> 5, s = lane & 15;
  const int col = col0 + (((lane >> 4) & 1) << 4) + ((s & 3) << 2);
  typedef __attribute__((address_space(3))) s16x4* lp;
  union { s16x4 v[2]; bf16x8 f; } u;
  u.v[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lp)(lds + tile_off(r0 + 4 * h + (s >> 2), col * 2)));
  u.v[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lp)(lds + tile_off(r0 + 8 + 4 * h + (s >> 2), col * 2)));
  return u.f;
}
__device__ __forceinline__ bf16x8 pack8(const float* p) {
  bf16x8 r;
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = (bf16)p[j];
  return r;
}
constexpr float LOG2E = 1.4426950408889634f, LN2 = 0.6931471805599453f;
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ f32x16 mfma(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
// index along the softmax axis of accumulator element e for this lane's half: (e/4)*8 + 4*half + e%4
__device__ __forceinline__ int acc_row(int e, int half) { return (e >> 2) * 8 + half * 4 + (e & 3); }

struct AttnArgs {
  const bf16* qkv; int64_t ld;   // q at column 0, k at H, v at 2H
  const float* key_mask;         // [B, S] 0/1 or null
  bf16* ctx;                     // [B*S, H]
  float* lse;                    // [B, N, S]
  const bf16* dctx;              // backward
  bf16* dqkv;
  float* delta;                  // [B, N, S]
  int B, N, S, H;
  float scale, mask_value;
  int prio;                      // wave priority (0..3)
  const float* kbar;             // backward, nullable: [B, H] mean key of every sample and head (see attn_bwd_dq_body)
};

// Which (batch, head) pair and which 64-row block of the parallel axis a workgroup takes.  Workgroups go to the 8 XCDs
// round-robin in launch order (grid x fastest), and the XCDs' L2s are private: with the plain mapping the S/64 blocks of one
// head land on 8 different XCDs and every one of them fetches that head's K and V (or Q and dO) from memory.  Here the
// workgroups of one XCD (equal launch index mod 8) take whole heads, one after the other, so a head's tiles are fetched
// into one L2 once and its other blocks hit there.
// `id` is the workgroup's index in launch order among the nb * nbh workgroups of the problem (nb = S / 64 blocks of the
// parallel axis, nbh = B * N pairs); the first of them must sit at a launch index that is a multiple of 8.
__device__ __forceinline__ void attn_block_map(int id, int nb, int nbh, int& bh, int& blk) {
  if (nbh % 8 != 0) { bh = id / nb; blk = id % nb; return; }
  const int xcd = id & 7, k = id >> 3;
  bh = (k / nb) * 8 + xcd;
  blk = k % nb;
}

// store a transposed 64 x 32 accumulator pair (rows d, columns = this lane's row index) as out[row][d]
__device__ __forceinline__ void store_t(bf16* out_row, const f32x16 (&acc)[2], float mul, int half) {
#pragma unroll
  for (int dt = 0; dt < 2; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      bf16x4 v;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = (bf16)(acc[dt][g * 4 + j] * mul);
      *reinterpret_cast<bf16x4*>(out_row + dt * 32 + g * 8 + half * 4) = v;
    }
}

// Partial accumulators of one wave parked in LDS: piece (i, g) of lane l at ((i*4+g)*64 + l)*16, then
// two floats per lane.  PART_BYTES covers two accumulators; the (SPLIT-1)*2 slots overlay the K/V tiles.
constexpr int PART_XY = 2 * 4 * 64 * 16;
constexpr int PART_BYTES = PART_XY + 64 * 16;
static_assert((SPLIT - 1) * 2 * PART_BYTES <= 2 * CHUNK * ROWB, "merge slots must fit in the tile region");
template <int NACC>
__device__ __forceinline__ void part_store(char* slot, const f32x16 (&acc)[NACC], int lane) {
#pragma unroll
  for (int i = 0; i < NACC; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f32x4 v = {acc[i][4 * g], acc[i][4 * g + 1], acc[i][4 * g + 2], acc[i][4 * g + 3]};
      *reinterpret_cast<f32x4*>(slot + ((i * 4 + g) * 64 + lane) * 16) = v;
    }
}
__device__ __forceinline__ void part_store_xy(char* slot, float x, float y, int lane) {
  float* xy = reinterpret_cast<float*>(slot + PART_XY) + lane * 2;
  xy[0] = x; xy[1] = y;
}
// acc = acc * wa + parked * wb
template <int NACC>
__device__ __forceinline__ void part_merge(const char* slot, f32x16 (&acc)[NACC], float wa, float wb, int lane) {
#pragma unroll
  for (int i = 0; i < NACC; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(slot + ((i * 4 + g) * 64 + lane) * 16);
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][4 * g + j] = acc[i][4 * g + j] * wa + v[j] * wb;
    }
}
__device__ __forceinline__ void part_xy(const char* slot, float& x, float& y, int lane) {
  const float* xy = reinterpret_cast<const float*>(slot + PART_XY) + lane * 2;
  x = xy[0]; y = xy[1];
}

// ----------------------------------------------------------------------------------- forward
// grid (S/64, B*N): each wave owns 32 queries and every SPLIT-th 32-key step.
__device__ __forceinline__ void attn_fwd_body(const AttnArgs& a, char* lds, int wg) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5;
  const int grp = wave & 1, part = wave >> 1;
  int bh, blk;
  attn_block_map(wg, a.S / 64, a.B * a.N, bh, blk);
  const int b = bh / a.N, hd = bh % a.N;
  const int q = blk * 64 + grp * 32 + (lane & 31);
  const bf16* base = a.qkv + (int64_t)b * a.S * a.ld + hd * HD;
  auto sk = [&](int c) { return lds + (c & 1) * (2 * CH * ROWB); };              // two buffers of CH rows per tensor
  auto sv = [&](int c) { return lds + (c & 1) * (2 * CH * ROWB) + CH * ROWB; };
  float* adder = reinterpret_cast<float*>(lds + 4 * CH * ROWB);
  const int nch = (a.S + CH - 1) / CH;
  auto rows_of = [&](int c) { return a.S - c * CH < CH ? a.S - c * CH : CH; };
  auto fill = [&](int c) {
    tile_fill(sk(c), base + a.H + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, lane);
    tile_fill(sv(c), base + 2 * a.H + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, lane);
  };
  // the first two K / V chunks are requested before anything else: the loads below queue behind them and the whole prologue
  // costs one trip to memory (a mask row staged through LDS would otherwise be waited for before the tiles are asked for)
  fill(0);
  if (nch > 1) fill(1);
  const bool masked = a.key_mask != nullptr;
  if (masked)
    for (int j = threadIdx.x; j < a.S; j += NTHREADS) adder[j] = (1.0f - a.key_mask[(int64_t)b * a.S + j]) * a.mask_value * LOG2E;
  bf16x8 qf[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(base + (int64_t)q * a.ld + 16 * ks + 8 * half);
  f32x16 o[2];
#pragma unroll
  for (int e = 0; e < 16; ++e) { o[0][e] = 0.f; o[1][e] = 0.f; }
  // running maximum and sum in the base-2 domain: p = exp2(s * scale * log2(e) + adder * log2(e) - m)
  float m = -INFINITY, l = 0.f;
  const float c2 = a.scale * LOG2E;
  __builtin_amdgcn_s_waitcnt(VMCNT0);  // q fragments (and the first two chunks): from here on only tile loads are in flight
  for (int c = 0; c < nch; ++c) {
    const int rows = rows_of(c);
    wait_chunk(c + 1 < nch ? rows_of(c + 1) : 0);
    __syncthreads();
    const char* ck = sk(c);
    const char* cv = sv(c);
    const int kt = part * 32;
    if (kt < rows) {
      f32x16 s;
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) s = mfma(frag_rows(ck, kt, ks, lane), qf[ks], s);
      float p[16], ad[16];
      step_adders(adder, masked, c * CH + kt, half, ad);
      float mt = -INFINITY;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        p[e] = s[e] * c2 + ad[e];
        mt = fmaxf(mt, p[e]);
      }
      mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
      const float mn = fmaxf(m, mt);
      const float alpha = exp2_fast(m - mn);
      m = mn;
      float rs = 0.f;
#pragma unroll
      for (int e = 0; e < 16; ++e) { p[e] = exp2_fast(p[e] - mn); rs += p[e]; }
      l = l * alpha + rs;
#pragma unroll
      for (int e = 0; e < 16; ++e) { o[0][e] *= alpha; o[1][e] *= alpha; }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const bf16x8 pf = pack8(p + 8 * s2);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) o[dt] = mfma(frag_cols(cv, kt + 16 * s2, dt * 32, lane), pf, o[dt]);
      }
    }
    if (c + 2 < nch) {
      __syncthreads();  // every wave is done with this buffer
      fill(c + 2);
    }
  }
  // combine the SPLIT partial softmaxes of each query group (part 0 always saw key step 0: m is finite)
  __syncthreads();
  if (part > 0) {
    part_store<2>(lds + ((part - 1) * 2 + grp) * PART_BYTES, o, lane);
    part_store_xy(lds + ((part - 1) * 2 + grp) * PART_BYTES, m, l, lane);
  }
  __syncthreads();
  if (part > 0) return;
#pragma unroll
  for (int pp = 1; pp < SPLIT; ++pp) {
    const char* slot = lds + ((pp - 1) * 2 + grp) * PART_BYTES;
    float mp, lp;
    part_xy(slot, mp, lp, lane);
    const float mn = fmaxf(m, mp);
    const float wa = exp2_fast(m - mn), wb = exp2_fast(mp - mn);
    part_merge<2>(slot, o, wa, wb, lane);
    l = l * wa + lp * wb;
    m = mn;
  }
  l += __shfl_xor(l, 32, 64);
  store_t(a.ctx + ((int64_t)b * a.S + q) * a.H + hd * HD, o, 1.0f / l, half);
  if (half == 0) a.lse[((int64_t)b * a.N + hd) * a.S + q] = (m + __log2f(l)) * LN2;   // natural-log lse, as backward expects
}

// ----------------------------------------------------------------------------------- backward: dQ
// grid (S/64, B*N): each wave owns 32 queries and every SPLIT-th 32-key step.  Also writes
// delta[q] = sum_d dO[q,d] O[q,d].
__device__ __forceinline__ void attn_bwd_dq_body(const AttnArgs& a, char* lds, int wg) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5;
  const int grp = wave & 1, part = wave >> 1;
  int bh, blk;
  attn_block_map(wg, a.S / 64, a.B * a.N, bh, blk);
  const int b = bh / a.N, hd = bh % a.N;
  const int q = blk * 64 + grp * 32 + (lane & 31);
  const bf16* base = a.qkv + (int64_t)b * a.S * a.ld + hd * HD;
  auto sk = [&](int c) { return lds + (c & 1) * (2 * CH * ROWB); };              // two buffers of CH rows per tensor
  auto sv = [&](int c) { return lds + (c & 1) * (2 * CH * ROWB) + CH * ROWB; };
  float* adder = reinterpret_cast<float*>(lds + 4 * CH * ROWB);
  const int nch = (a.S + CH - 1) / CH;
  auto rows_of = [&](int c) { return a.S - c * CH < CH ? a.S - c * CH : CH; };
  auto fill = [&](int c) {
    tile_fill(sk(c), base + a.H + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, lane);
    tile_fill(sv(c), base + 2 * a.H + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, lane);
  };
  // the first two K / V chunks are requested first: delta below needs its operands in registers, and waiting for them
  // before asking for the tiles would cost a second trip to memory
  fill(0);
  if (nch > 1) fill(1);
  const bool masked = a.key_mask != nullptr;
  if (masked)
    for (int j = threadIdx.x; j < a.S; j += NTHREADS) adder[j] = (1.0f - a.key_mask[(int64_t)b * a.S + j]) * a.mask_value * LOG2E;
  bf16x8 qf[4], dof[4];
  float delta = 0.f;
  const int64_t orow = ((int64_t)b * a.S + q) * a.H + hd * HD;
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    qf[ks] = *reinterpret_cast<const bf16x8*>(base + (int64_t)q * a.ld + 16 * ks + 8 * half);
    dof[ks] = *reinterpret_cast<const bf16x8*>(a.dctx + orow + 16 * ks + 8 * half);
    const bf16x8 of = *reinterpret_cast<const bf16x8*>(a.ctx + orow + 16 * ks + 8 * half);
#pragma unroll
    for (int j = 0; j < 8; ++j) delta += (float)dof[ks][j] * (float)of[j];
  }
  delta += __shfl_xor(delta, 32, 64);
  const float lse2 = a.lse[((int64_t)b * a.N + hd) * a.S + q] * LOG2E;
  if (a.delta != nullptr && half == 0 && part == 0) a.delta[((int64_t)b * a.N + hd) * a.S + q] = delta;  // null: the caller has it
  f32x16 dq[2];
#pragma unroll
  for (int e = 0; e < 16; ++e) { dq[0][e] = 0.f; dq[1][e] = 0.f; }
  // row sums of the bf16 dS that enter the dQ products, by the matrix pipe (it has time to spare; the vector ALU does not):
  // ones[32 x 16] dS^T[16 x 32] puts the sum over a step's keys for query `lane % 32` into every register of rs
  f32x16 rs;
  bf16x8 ones;
#pragma unroll
  for (int e = 0; e < 16; ++e) rs[e] = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) ones[j] = (bf16)1.0f;
  const float c2 = a.scale * LOG2E;
  __builtin_amdgcn_s_waitcnt(VMCNT0);  // the loads and the store above: from here on only tile loads are in flight
  for (int c = 0; c < nch; ++c) {
    const int rows = rows_of(c);
    wait_chunk(c + 1 < nch ? rows_of(c + 1) : 0);
    __syncthreads();
    const char* ck = sk(c);
    const char* cv = sv(c);
    const int kt = part * 32;
    if (kt < rows) {
      f32x16 s, dp;
#pragma unroll
      for (int e = 0; e < 16; ++e) { s[e] = 0.f; dp[e] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        s = mfma(frag_rows(ck, kt, ks, lane), qf[ks], s);     // S^T[key][q]
        dp = mfma(frag_rows(cv, kt, ks, lane), dof[ks], dp);  // dP^T[key][q] = V dO^T
      }
      float ds[16], ad[16];
      step_adders(adder, masked, c * CH + kt, half, ad);
#pragma unroll
      for (int e = 0; e < 16; ++e)
        ds[e] = exp2_fast(s[e] * c2 + (ad[e] - lse2)) * (dp[e] - delta);   // the factor `scale` is applied once, to the sums
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const bf16x8 df = pack8(ds + 8 * s2);
        if (a.kbar != nullptr) rs = mfma(ones, df, rs);   // every row: what the rounded rows of dS sum to (exactly 0 before rounding)
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) dq[dt] = mfma(frag_cols(ck, kt + 16 * s2, dt * 32, lane), df, dq[dt]);  // dQ^T += K^T dS^T
      }
    }
    if (c + 2 < nch) {
      __syncthreads();  // every wave is done with this buffer
      fill(c + 2);
    }
  }
  // the mean key of this head, asked for now so that the trip to memory runs under the merge
  f32x4 kv[2][4];
  if (a.kbar != nullptr && part == 0) {
    const float* kb = a.kbar + (int64_t)b * a.H + hd * HD;
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) kv[dt][g] = *reinterpret_cast<const f32x4*>(kb + dt * 32 + g * 8 + half * 4);
  }
  __syncthreads();
  if (part > 0) {
    part_store<2>(lds + ((part - 1) * 2 + grp) * PART_BYTES, dq, lane);
    part_store_xy(lds + ((part - 1) * 2 + grp) * PART_BYTES, rs[0], 0.f, lane);
  }
  __syncthreads();
  if (part > 0) return;
  float rsum = rs[0];
#pragma unroll
  for (int pp = 1; pp < SPLIT; ++pp) {
    const char* slot = lds + ((pp - 1) * 2 + grp) * PART_BYTES;
    part_merge<2>(slot, dq, 1.f, 1.f, lane);
    float r1, unused;
    part_xy(slot, r1, unused, lane);
    rsum += r1;
  }
  if (a.kbar != nullptr) {
    // Every row of dS sums to zero, so dQ = dS K = dS (K - 1 kbar^T) for any vector kbar.  The dS that entered the
    // products above were rounded to bf16 and sum to rsum instead: against keys that share a large common part (token
    // vectors that have grown alike over the layers) rsum * kbar is the bulk of dQ's rounding error, and it is known.
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) dq[dt][g * 4 + j] -= rsum * kv[dt][g][j];
  }
  store_t(a.dqkv + ((int64_t)b * a.S + q) * a.ld + hd * HD, dq, a.scale, half);
}

// ----------------------------------------------------------------------------------- backward: dK, dV
// grid (S/64, B*N): each wave owns 32 keys and every SPLIT-th 32-query step (Q and dO tiles in LDS).
__device__ __forceinline__ void attn_bwd_dkv_body(const AttnArgs& a, char* lds, int wg) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5;
  const int grp = wave & 1, part = wave >> 1;
  int bh, blk;
  attn_block_map(wg, a.S / 64, a.B * a.N, bh, blk);
  const int b = bh / a.N, hd = bh % a.N;
  const int key = blk * 64 + grp * 32 + (lane & 31);
  const bf16* base = a.qkv + (int64_t)b * a.S * a.ld + hd * HD;
  const bf16* dobase = a.dctx + (int64_t)b * a.S * a.H + hd * HD;
  auto sq = [&](int c) { return lds + (c & 1) * (2 * CH * ROWB); };              // two buffers of CH rows per tensor
  auto sdo = [&](int c) { return lds + (c & 1) * (2 * CH * ROWB) + CH * ROWB; };
  float* slse = reinterpret_cast<float*>(lds + 4 * CH * ROWB);
  float* sdelta = slse + a.S;
  const int nch = (a.S + CH - 1) / CH;
  auto rows_of = [&](int c) { return a.S - c * CH < CH ? a.S - c * CH : CH; };
  auto fill = [&](int c) {
    tile_fill(sq(c), base + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, lane);
    tile_fill(sdo(c), dobase + (int64_t)c * CH * a.H, a.H, rows_of(c), wave, lane);
  };
  // the first two Q / dO chunks are requested first: lse and delta go through registers into LDS, and waiting for them
  // before asking for the tiles would cost a second trip to memory
  fill(0);
  if (nch > 1) fill(1);
  for (int j = threadIdx.x; j < a.S; j += NTHREADS) {
    slse[j] = a.lse[((int64_t)b * a.N + hd) * a.S + j] * LOG2E;
    sdelta[j] = a.delta[((int64_t)b * a.N + hd) * a.S + j];
  }
  const float adder = a.key_mask ? (1.0f - a.key_mask[(int64_t)b * a.S + key]) * a.mask_value * LOG2E : 0.f;
  bf16x8 kf[4], vf[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    kf[ks] = *reinterpret_cast<const bf16x8*>(base + a.H + (int64_t)key * a.ld + 16 * ks + 8 * half);
    vf[ks] = *reinterpret_cast<const bf16x8*>(base + 2 * a.H + (int64_t)key * a.ld + 16 * ks + 8 * half);
  }
  f32x16 dk[2], dv[2];
#pragma unroll
  for (int e = 0; e < 16; ++e) { dk[0][e] = 0.f; dk[1][e] = 0.f; dv[0][e] = 0.f; dv[1][e] = 0.f; }
  const float c2 = a.scale * LOG2E;
  __builtin_amdgcn_s_waitcnt(VMCNT0);  // the loads above: from here on only tile loads are in flight
  for (int c = 0; c < nch; ++c) {
    const int rows = rows_of(c);
    wait_chunk(c + 1 < nch ? rows_of(c + 1) : 0);
    __syncthreads();
    const char* cq = sq(c);
    const char* cdo = sdo(c);
    const int qt = part * 32;
    if (qt < rows) {
      f32x16 s, dp;
#pragma unroll
      for (int e = 0; e < 16; ++e) { s[e] = 0.f; dp[e] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        s = mfma(frag_rows(cq, qt, ks, lane), kf[ks], s);      // S[q][key]
        dp = mfma(frag_rows(cdo, qt, ks, lane), vf[ks], dp);   // dP[q][key] = dO V^T
      }
      float p[16], ds[16], ls[16], dl[16];
      step_adders(slse, true, c * CH + qt, half, ls);     // this step's 16 query rows: log-sum-exp and delta
      step_adders(sdelta, true, c * CH + qt, half, dl);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        p[e] = exp2_fast(s[e] * c2 + (adder - ls[e]));
        ds[e] = p[e] * (dp[e] - dl[e]);   // the factor `scale` is applied once, to dK
      }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const bf16x8 pf = pack8(p + 8 * s2), df = pack8(ds + 8 * s2);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
          dv[dt] = mfma(frag_cols(cdo, qt + 16 * s2, dt * 32, lane), pf, dv[dt]);  // dV^T += dO^T P
          dk[dt] = mfma(frag_cols(cq, qt + 16 * s2, dt * 32, lane), df, dk[dt]);   // dK^T += Q^T dS
        }
      }
    }
    if (c + 2 < nch) {
      __syncthreads();  // every wave is done with this buffer
      fill(c + 2);
    }
  }
  // two merge rounds through the same slots: dK, then dV
  char* slot = lds + ((part - 1) * 2 + grp) * PART_BYTES;
  __syncthreads();
  if (part > 0) part_store<2>(slot, dk, lane);
  __syncthreads();
  if (part == 0) {
#pragma unroll
    for (int pp = 1; pp < SPLIT; ++pp) part_merge<2>(lds + ((pp - 1) * 2 + grp) * PART_BYTES, dk, 1.f, 1.f, lane);
  }
  __syncthreads();
  if (part > 0) part_store<2>(slot, dv, lane);
  __syncthreads();
  if (part > 0) return;
#pragma unroll
  for (int pp = 1; pp < SPLIT; ++pp) part_merge<2>(lds + ((pp - 1) * 2 + grp) * PART_BYTES, dv, 1.f, 1.f, lane);
  bf16* orow = a.dqkv + ((int64_t)b * a.S + key) * a.ld + hd * HD;
  store_t(orow + a.H, dk, a.scale, half);
  store_t(orow + 2 * a.H, dv, 1.0f, half);
}

// K / V (or Q / dO) tiles, two buffers each, plus `vectors` per-position fp32 arrays (mask adders; log-sum-exp and delta).
// Every 4 KB counts: at 64 KB two 48 KB GEMM blocks of other streams fit on the CU beside an attention block, at 68 KB one.
inline size_t lds_bytes(int S, int vectors) { return (size_t)4 * CH * ROWB + (size_t)vectors * S * sizeof(float); }

}  // namespace dsattn
