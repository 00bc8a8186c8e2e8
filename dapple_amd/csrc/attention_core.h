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

// Fills `rows` tile rows (a multiple of 64) from global rows of stride ld (elements); all waves of the block.  One load
// moves 64 consecutive 16-byte slots = 8 tile rows; wave w takes rows 8w .. 8w+7 of every 64.  A lane's offset from the first
// of those 64 rows (fill_voff) is the same for every load of a tensor - the swizzle repeats every 16 rows - so a load is a
// scalar base, that offset and the LDS address in m0: no vector arithmetic in the loop.
__device__ __forceinline__ uint32_t fill_voff(int64_t ld, int wave, int lane) {
  const int r = wave * 8 + (lane >> 3), pc = lane & 7;
  return (uint32_t)(((int64_t)r * ld + (pc ^ tile_swz(r)) * 8) * (int64_t)sizeof(bf16));
}
__device__ __forceinline__ uint64_t uniform64(uint64_t v) {   // the same in every lane: to scalar registers, for an asm "s" operand
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const char*)p);
}
__device__ __forceinline__ void tile_fill(char* lds, const bf16* src, int64_t ld, int rows, int wave, uint32_t voff) {
  uint32_t slot = __builtin_amdgcn_readfirstlane(lds_addr(lds) + (uint32_t)wave * 1024u);
  uint64_t from = uniform64((uint64_t)(uintptr_t)src);
  const uint64_t step = uniform64((uint64_t)(64 * ld * (int64_t)sizeof(bf16)));
  for (int i = 0; i < rows / 64; ++i) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(slot), "v"(voff), "s"(from) : "memory", "m0");
    slot += 8 * 1024u;
    from += step;
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

// LDS reads inside the chunk loops are inline asm with explicit waits: left to the compiler, its wait-count pass puts a full
// `s_waitcnt vmcnt(0)` in front of the first LDS read that follows an LDS-DMA load - i.e. every step would first wait for the
// NEXT chunks' tiles, which are requested one to two steps ahead precisely so that nobody waits for them.  A read's
// registers are named as in/out operands of the wait that covers it, so nothing that uses them can move above that wait;
// LDS reads complete in order, so `lgkmcnt(N)` means: everything but the newest N reads has arrived.
__device__ __forceinline__ void lds_read16(bf16x8& f, uint32_t a) { asm volatile("ds_read_b128 %0, %1" : "=v"(f) : "v"(a)); }
__device__ __forceinline__ void lds_read16(f32x4& f, uint32_t a) { asm volatile("ds_read_b128 %0, %1" : "=v"(f) : "v"(a)); }
__device__ __forceinline__ void lds_read_tr(s16x4& f, uint32_t a) { asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(f) : "v"(a)); }
template <int N> __device__ __forceinline__ void lds_wait(bf16x8& f) { asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(f) : "n"(N)); }
struct ColFrag { s16x4 lo, hi; };   // the two halves of a transposed operand, as the reads deliver them
template <int N> __device__ __forceinline__ void lds_wait(ColFrag& a, ColFrag& b) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait(ColFrag& a, ColFrag& b, ColFrag& c, ColFrag& d) {
  asm volatile("s_waitcnt lgkmcnt(%8)"
               : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi), "+v"(c.lo), "+v"(c.hi), "+v"(d.lo), "+v"(d.hi) : "n"(N));
}
__device__ __forceinline__ void lds_wait_all(f32x4 (&v)[4]) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
}
__device__ __forceinline__ bf16x8 operand(const ColFrag& f) {
  union { s16x4 v[2]; bf16x8 f; } u;
  u.v[0] = f.lo; u.v[1] = f.hi;
  return u.f;
}

// Per-position values (mask adders, log-sum-exp, delta) of the 16 accumulator rows of a 32-row step (rows (e/4)*8 + 4*half +
// e%4): four 16-byte LDS reads, requested here and valid after lds_wait_all().
__device__ __forceinline__ void step_vector_issue(const float* vec, int row0, int half, f32x4 (&v)[4]) {
#pragma unroll
  for (int g = 0; g < 4; ++g) lds_read16(v[g], lds_addr(vec + row0 + g * 8 + half * 4));
}

// A operand, rows = tile rows (row0 + lane%32), k = 8 consecutive columns starting at 16*ks + 8*half
__device__ __forceinline__ void frag_rows_issue(const char* lds, int row0, int ks, int lane, bf16x8& f) {
  lds_read16(f, lds_addr(lds + tile_off(row0 + (lane & 31), (2 * ks + (lane >> 5)) * 16)));
}
// A operand of the transposed use: rows = tile columns (col0 + lane%32), k = tile rows in the order the
// accumulator layout hands them over: elements 0-3 -> rows r0 + 4*half + 0..3, elements 4-7 -> r0 + 8 + 4*half + 0..3
__device__ __forceinline__ void frag_cols_issue(const char* lds, int r0, int col0, int lane, ColFrag& f) {
  const int h = lane >> 5, s = lane & 15;
  const int col = col0 + (((lane >> 4) & 1) << 4) + ((s & 3) << 2);
  lds_read_tr(f.lo, lds_addr(lds + tile_off(r0 + 4 * h + (s >> 2), col * 2)));
  lds_read_tr(f.hi, lds_addr(lds + tile_off(r0 + 8 + 4 * h + (s >> 2), col * 2)));
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
// GENERAL = false (no key mask, scale > 0) is the short form of the step: the maximum is taken over the raw scores (one
// v_max3 per two of them), each probability is one fused multiply-add and one exponential, and the running maximum only
// moves - and the 32 output accumulators are only rescaled, a wave-uniform branch - when a step's maximum exceeds it by
// more than 2^LAZY_LOG2: probabilities then reach 2^LAZY_LOG2 at most, which costs bf16 and the fp32 sums nothing.
constexpr float LAZY_LOG2 = 8.f;
template <bool GENERAL>
__device__ __forceinline__ void attn_fwd_body_t(const AttnArgs& a, char* lds, int wg) {
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
  const uint32_t voff = fill_voff(a.ld, wave, lane);
  auto fill = [&](int c) {
    tile_fill(sk(c), base + a.H + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, voff);
    tile_fill(sv(c), base + 2 * a.H + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, voff);
  };
  // the first K / V chunk is requested before anything else, the second right behind the prologue's own loads: the whole
  // prologue costs one trip to memory (a mask row staged through LDS would otherwise be waited for before the tiles are
  // asked for), and the first step needs only what was asked for before the second chunk
  fill(0);
  const bool masked = GENERAL && a.key_mask != nullptr;
  if (masked)
    for (int j = threadIdx.x; j < a.S; j += NTHREADS) adder[j] = (1.0f - a.key_mask[(int64_t)b * a.S + j]) * a.mask_value * LOG2E;
  bf16x8 qf[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(base + (int64_t)q * a.ld + 16 * ks + 8 * half);
  if (nch > 1) fill(1);
  f32x16 o[2];
#pragma unroll
  for (int e = 0; e < 16; ++e) { o[0][e] = 0.f; o[1][e] = 0.f; }
  // running maximum and sum in the base-2 domain: p = exp2(s * scale * log2(e) + adder * log2(e) - m)
  float m = -INFINITY, l = 0.f;
  bool seen = false;   // short form: this wave has taken its first step (wave-uniform)
  const float c2 = a.scale * LOG2E;
  // no wait here: the loop's first wait leaves at most the second chunk's loads in flight, and the mask and query loads are
  // older than those (should the compiler move one behind them, its own wait for the loaded value is a full one)
  for (int c = 0; c < nch; ++c) {
    const int rows = rows_of(c);
    wait_chunk(c + 1 < nch ? rows_of(c + 1) : 0);
    __syncthreads();
    const char* ck = sk(c);
    const char* cv = sv(c);
    const int kt = part * 32;
    if (kt < rows) {
      f32x4 adv[4];
      if (GENERAL && masked) step_vector_issue(adder, c * CH + kt, half, adv);
      bf16x8 kf[4];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) frag_rows_issue(ck, kt, ks, lane, kf[ks]);
      f32x16 s;
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = 0.f;
      lds_wait<3>(kf[0]); s = mfma(kf[0], qf[0], s);
      lds_wait<2>(kf[1]); s = mfma(kf[1], qf[1], s);
      lds_wait<1>(kf[2]); s = mfma(kf[2], qf[2], s);
      lds_wait<0>(kf[3]); s = mfma(kf[3], qf[3], s);
      if (GENERAL && masked) lds_wait_all(adv);   // older than the fragments: arrived, this only ties the registers
      // V^T of the step's first 16 keys is requested under the softmax arithmetic, the second half behind it
      ColFrag vf[2][2];
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) frag_cols_issue(cv, kt, dt * 32, lane, vf[0][dt]);
      float p[16];
      if constexpr (GENERAL) {
        float ad[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) ad[e] = masked ? adv[e >> 2][e & 3] : 0.f;
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
      } else {
        float mr = s[0];
#pragma unroll
        for (int e = 1; e < 16; ++e) mr = fmaxf(mr, s[e]);
        mr = fmaxf(mr, __shfl_xor(mr, 32, 64));
        const float mt = mr * c2;   // c2 > 0: the maximum of the scaled scores
        if (!seen) {
          m = mt;
          seen = true;
        } else {
          const bool move = mt > m + LAZY_LOG2;
          if (__builtin_amdgcn_ballot_w64(move) != 0) {   // some query of the wave needs a new reference point
            const float mn = move ? mt : m;
            const float alpha = exp2_fast(m - mn);        // 1 for the lanes that stay
            m = mn;
            l *= alpha;
#pragma unroll
            for (int e = 0; e < 16; ++e) { o[0][e] *= alpha; o[1][e] *= alpha; }
          }
        }
        const float nm = -m;
        float rs = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) { p[e] = exp2_fast(__builtin_fmaf(s[e], c2, nm)); rs += p[e]; }
        l += rs;
      }
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) frag_cols_issue(cv, kt + 16, dt * 32, lane, vf[1][dt]);
      lds_wait<4>(vf[0][0], vf[0][1]);
      bf16x8 pf = pack8(p);
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) o[dt] = mfma(operand(vf[0][dt]), pf, o[dt]);
      lds_wait<0>(vf[1][0], vf[1][1]);
      pf = pack8(p + 8);
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) o[dt] = mfma(operand(vf[1][dt]), pf, o[dt]);
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
  // one common reference point for the four partial softmaxes, then one multiply-add per element and part
  float mp[SPLIT], lp[SPLIT];
  float mn = m;
#pragma unroll
  for (int pp = 1; pp < SPLIT; ++pp) {
    part_xy(lds + ((pp - 1) * 2 + grp) * PART_BYTES, mp[pp], lp[pp], lane);
    mn = fmaxf(mn, mp[pp]);
  }
  const float w0 = exp2_fast(m - mn);
  l *= w0;
#pragma unroll
  for (int e = 0; e < 16; ++e) { o[0][e] *= w0; o[1][e] *= w0; }
#pragma unroll
  for (int pp = 1; pp < SPLIT; ++pp) {
    const float wb = exp2_fast(mp[pp] - mn);   // 0 for a part that saw no key (its maximum is -inf)
    part_merge<2>(lds + ((pp - 1) * 2 + grp) * PART_BYTES, o, 1.f, wb, lane);
    l += lp[pp] * wb;
  }
  m = mn;
  l += __shfl_xor(l, 32, 64);
  store_t(a.ctx + ((int64_t)b * a.S + q) * a.H + hd * HD, o, 1.0f / l, half);
  if (half == 0) a.lse[((int64_t)b * a.N + hd) * a.S + q] = (m + __log2f(l)) * LN2;   // natural-log lse, as backward expects
}

// the short forms below need no mask and a positive scale (the maximum of the scaled scores = scale x the maximum)
__device__ __forceinline__ bool attn_general(const AttnArgs& a) { return a.key_mask != nullptr || !(a.scale > 0.f); }
__device__ __forceinline__ void attn_fwd_body(const AttnArgs& a, char* lds, int wg) {
  if (attn_general(a)) attn_fwd_body_t<true>(a, lds, wg);
  else attn_fwd_body_t<false>(a, lds, wg);
}

// ----------------------------------------------------------------------------------- backward: dQ
// grid (S/64, B*N): each wave owns 32 queries and every SPLIT-th 32-key step.  Also writes
// delta[q] = sum_d dO[q,d] O[q,d].  GENERAL = false: no mask adders in the loop.
template <bool GENERAL>
__device__ __forceinline__ void attn_bwd_dq_body_t(const AttnArgs& a, char* lds, int wg) {
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
  const uint32_t voff = fill_voff(a.ld, wave, lane);
  auto fill = [&](int c) {
    tile_fill(sk(c), base + a.H + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, voff);
    tile_fill(sv(c), base + 2 * a.H + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, voff);
  };
  // the first two K / V chunks are requested first: delta below needs its operands in registers, and waiting for them
  // before asking for the tiles would cost a second trip to memory
  fill(0);
  if (nch > 1) fill(1);
  const bool masked = GENERAL && a.key_mask != nullptr;
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
      f32x4 adv[4];
      if (GENERAL && masked) step_vector_issue(adder, c * CH + kt, half, adv);
      bf16x8 kr[4], vr[4];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        frag_rows_issue(ck, kt, ks, lane, kr[ks]);
        frag_rows_issue(cv, kt, ks, lane, vr[ks]);
      }
      f32x16 s, dp;
#pragma unroll
      for (int e = 0; e < 16; ++e) { s[e] = 0.f; dp[e] = 0.f; }
      // S^T[key][q] = K Q^T and dP^T[key][q] = V dO^T
      lds_wait<7>(kr[0]); s = mfma(kr[0], qf[0], s);
      lds_wait<6>(vr[0]); dp = mfma(vr[0], dof[0], dp);
      lds_wait<5>(kr[1]); s = mfma(kr[1], qf[1], s);
      lds_wait<4>(vr[1]); dp = mfma(vr[1], dof[1], dp);
      lds_wait<3>(kr[2]); s = mfma(kr[2], qf[2], s);
      lds_wait<2>(vr[2]); dp = mfma(vr[2], dof[2], dp);
      lds_wait<1>(kr[3]); s = mfma(kr[3], qf[3], s);
      lds_wait<0>(vr[3]); dp = mfma(vr[3], dof[3], dp);
      if (GENERAL && masked) lds_wait_all(adv);   // older than the fragments: arrived, this only ties the registers
      // K^T of the step's first 16 keys is requested under the arithmetic, the second half behind it
      ColFrag kc[2][2];
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) frag_cols_issue(ck, kt, dt * 32, lane, kc[0][dt]);
      float ds[16];
      if constexpr (GENERAL) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const float ad = masked ? adv[e >> 2][e & 3] : 0.f;
          ds[e] = exp2_fast(s[e] * c2 + (ad - lse2)) * (dp[e] - delta);   // the factor `scale` is applied once, to the sums
        }
      } else {
        const float nl = -lse2;
#pragma unroll
        for (int e = 0; e < 16; ++e) ds[e] = exp2_fast(__builtin_fmaf(s[e], c2, nl)) * (dp[e] - delta);
      }
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) frag_cols_issue(ck, kt + 16, dt * 32, lane, kc[1][dt]);
      lds_wait<4>(kc[0][0], kc[0][1]);
      bf16x8 df = pack8(ds);
      if (a.kbar != nullptr) rs = mfma(ones, df, rs);   // every row: what the rounded rows of dS sum to (exactly 0 before rounding)
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) dq[dt] = mfma(operand(kc[0][dt]), df, dq[dt]);  // dQ^T += K^T dS^T
      lds_wait<0>(kc[1][0], kc[1][1]);
      df = pack8(ds + 8);
      if (a.kbar != nullptr) rs = mfma(ones, df, rs);
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) dq[dt] = mfma(operand(kc[1][dt]), df, dq[dt]);
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

__device__ __forceinline__ void attn_bwd_dq_body(const AttnArgs& a, char* lds, int wg) {
  if (attn_general(a)) attn_bwd_dq_body_t<true>(a, lds, wg);
  else attn_bwd_dq_body_t<false>(a, lds, wg);
}

// ----------------------------------------------------------------------------------- backward: dK, dV
// grid (S/64, B*N): each wave owns 32 keys and every SPLIT-th 32-query step (Q and dO tiles in LDS).  The log-sum-exp
// values are staged negated, so that a probability is exp2(score * c + (adder + -lse)): without a mask one fused
// multiply-add and the exponential.
template <bool GENERAL>
__device__ __forceinline__ void attn_bwd_dkv_body_t(const AttnArgs& a, char* lds, int wg) {
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
  const uint32_t voff = fill_voff(a.ld, wave, lane), voff_do = fill_voff(a.H, wave, lane);
  auto fill = [&](int c) {
    tile_fill(sq(c), base + (int64_t)c * CH * a.ld, a.ld, rows_of(c), wave, voff);
    tile_fill(sdo(c), dobase + (int64_t)c * CH * a.H, a.H, rows_of(c), wave, voff_do);
  };
  // the first two Q / dO chunks are requested first: lse and delta go through registers into LDS, and waiting for them
  // before asking for the tiles would cost a second trip to memory
  fill(0);
  if (nch > 1) fill(1);
  for (int j = threadIdx.x; j < a.S; j += NTHREADS) {
    slse[j] = -a.lse[((int64_t)b * a.N + hd) * a.S + j] * LOG2E;
    sdelta[j] = a.delta[((int64_t)b * a.N + hd) * a.S + j];
  }
  const float adder = GENERAL && a.key_mask ? (1.0f - a.key_mask[(int64_t)b * a.S + key]) * a.mask_value * LOG2E : 0.f;
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
      f32x4 lsv[4], dlv[4];
      step_vector_issue(slse, c * CH + qt, half, lsv);     // this step's 16 query rows: minus log-sum-exp, and delta
      step_vector_issue(sdelta, c * CH + qt, half, dlv);
      bf16x8 qr[4], dor[4];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        frag_rows_issue(cq, qt, ks, lane, qr[ks]);
        frag_rows_issue(cdo, qt, ks, lane, dor[ks]);
      }
      f32x16 s, dp;
#pragma unroll
      for (int e = 0; e < 16; ++e) { s[e] = 0.f; dp[e] = 0.f; }
      // S[q][key] = Q K^T and dP[q][key] = dO V^T
      lds_wait<7>(qr[0]); s = mfma(qr[0], kf[0], s);
      lds_wait<6>(dor[0]); dp = mfma(dor[0], vf[0], dp);
      lds_wait<5>(qr[1]); s = mfma(qr[1], kf[1], s);
      lds_wait<4>(dor[1]); dp = mfma(dor[1], vf[1], dp);
      lds_wait<3>(qr[2]); s = mfma(qr[2], kf[2], s);
      lds_wait<2>(dor[2]); dp = mfma(dor[2], vf[2], dp);
      lds_wait<1>(qr[3]); s = mfma(qr[3], kf[3], s);
      lds_wait<0>(dor[3]); dp = mfma(dor[3], vf[3], dp);
      lds_wait_all(lsv);   // older than the fragments: arrived, these only tie the registers
      lds_wait_all(dlv);
      // dO^T and Q^T of the step's first 16 queries are requested under the arithmetic, the second half behind it
      ColFrag doc[2][2], qc[2][2];
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) {
        frag_cols_issue(cdo, qt, dt * 32, lane, doc[0][dt]);
        frag_cols_issue(cq, qt, dt * 32, lane, qc[0][dt]);
      }
      float p[16], ds[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float ls = lsv[e >> 2][e & 3];
        p[e] = GENERAL ? exp2_fast(s[e] * c2 + (adder + ls)) : exp2_fast(__builtin_fmaf(s[e], c2, ls));
        ds[e] = p[e] * (dp[e] - dlv[e >> 2][e & 3]);   // the factor `scale` is applied once, to dK
      }
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) {
        frag_cols_issue(cdo, qt + 16, dt * 32, lane, doc[1][dt]);
        frag_cols_issue(cq, qt + 16, dt * 32, lane, qc[1][dt]);
      }
      lds_wait<8>(doc[0][0], qc[0][0], doc[0][1], qc[0][1]);
      bf16x8 pf = pack8(p), df = pack8(ds);
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) {
        dv[dt] = mfma(operand(doc[0][dt]), pf, dv[dt]);  // dV^T += dO^T P
        dk[dt] = mfma(operand(qc[0][dt]), df, dk[dt]);   // dK^T += Q^T dS
      }
      lds_wait<0>(doc[1][0], qc[1][0], doc[1][1], qc[1][1]);
      pf = pack8(p + 8); df = pack8(ds + 8);
#pragma unroll
      for (int dt = 0; dt < 2; ++dt) {
        dv[dt] = mfma(operand(doc[1][dt]), pf, dv[dt]);
        dk[dt] = mfma(operand(qc[1][dt]), df, dk[dt]);
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

__device__ __forceinline__ void attn_bwd_dkv_body(const AttnArgs& a, char* lds, int wg) {
  if (attn_general(a)) attn_bwd_dkv_body_t<true>(a, lds, wg);
  else attn_bwd_dkv_body_t<false>(a, lds, wg);
}

// K / V (or Q / dO) tiles, two buffers each, plus `vectors` per-position fp32 arrays (mask adders; log-sum-exp and delta).
// Every 4 KB counts: at 64 KB two 48 KB GEMM blocks of other streams fit on the CU beside an attention block, at 68 KB one.
inline size_t lds_bytes(int S, int vectors) { return (size_t)4 * CH * ROWB + (size_t)vectors * S * sizeof(float); }

}  // namespace dsattn
