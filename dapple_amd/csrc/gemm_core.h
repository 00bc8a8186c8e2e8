// Device building blocks shared by the MFMA GEMM kernels of gemm.hip (4-wave blocks) and gemm8.hip (8-wave blocks):
// MFMA wrappers, the launch arguments, the LDS layouts, the LDS-DMA loader and the fragment readers.
#pragma once
#include <type_traits>
#include "common.h"

namespace dsgemm {

template <typename T> struct Mma;
template <> struct Mma<bf16> {
  typedef bf16x8 Frag;
  static constexpr int KT = 64;
  static __device__ __forceinline__ void mma(f32x16& acc, const Frag& a, const Frag& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
  }
};
template <> struct Mma<float> {
  typedef f32x4 Frag;
  static constexpr int KT = 32;
  static __device__ __forceinline__ void mma(f32x16& acc, const Frag& a, const Frag& b) {
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[j], acc, 0, 0, 0);
  }
};


struct GemmArgs {
  const char* a;
  const char* b;
  char* c;
  const float* bias;
  const char* residual;
  char* c2;
  int m, n, k;
  int64_t lda, ldb, ldc;
  int batch_inner;
  int64_t a_so, a_si, b_so, b_si, c_so, c_si;
  int flags;
  float alpha;
  int splitk;
  int ktiles_per_split;
  int grid_m, grid_n;
  int xcd_rm, xcd_cn;  // tiles per XCD as an xcd_rm x xcd_cn block of the tile grid (0: contiguous runs)
  int vec_epi;
  int conv_h, conv_w, conv_c;  // implicit 3x3 'same' convolution: extent of the gathered NHWC tensor
  int prio;                    // wave priority (0..3)
  float* ws_part;              // split-K by workspace (8-wave kernels): fp32 partial tiles [tile][slice][BM * BN]
  unsigned* ws_count;          // and one arrival counter per tile (zero between launches)
  size_t ws_bytes;             // bytes behind ws_part (host side: the launcher checks them against the grid it is about to start)
  // Segmented reduction (MN-major operands): k runs over segments of seg_ktiles k-tiles; segment s of A / B starts
  // a_seg / b_seg elements behind segment s - 1 (0 for both = every segment reads the same rows).  seg_ktiles = 0: one run.
  int seg_ktiles;
  int64_t a_seg, b_seg;
  float* rowdot;               // DS_EPI_ROWDOT (grouped launches only): see gemm_epilogue_vec8
  int rowdot_seq;
  // Column sums of the B operand beside the product (grouped launches, 256x128 tiles): colsum[zi * colsum_si + col] +=
  // sum_k B(col, k) - with B = dY of a weight gradient X^T dY that is the gradient of the layer's bias.  null: none.
  float* colsum;
  int64_t colsum_si;
};

// Internal epilogue flag: besides C, write for every row and every block of 64 columns the dot product of the bf16 values
// stored to C with the bf16 tensor c2 (layout of C):
//   rowdot[((row / rowdot_seq) * (n / 64) + col / 64) * rowdot_seq + row % rowdot_seq]
// With C = d ctx and c2 = ctx of an attention layer (rows = samples x positions, 64 columns per head) that is the
// delta[b][head][position] = sum_d dO O of the softmax backward.  Needs n % 64 == 0 and no other use of c2.
#define DS_EPI_ROWDOT 4096


// LDS has 64 banks of 4 bytes: one bank line is 256 bytes = two 128-byte K-major rows.
// K-major: a 16-lane phase of a 16-byte fragment read covers 16 consecutive rows of one chunk
// column; rows of equal parity share a half line, so the chunk is rotated by (row >> 1).
__device__ __forceinline__ int kmajor_swz(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int kmajor_off(int row, int chunk) { return row * 128 + ((chunk ^ kmajor_swz(row)) << 4); }
// MN-major: a transposing read touches 4 consecutive rows x two 32-byte granules per 32 lanes.
// Rows of 256 bytes or more start on a bank line: rotate the granule pair by (r & 3).  Rows of 128
// bytes alternate between the halves of a line: only rows r and r+2 collide, rotate by bit 1 of r.
template <int ROW_BYTES> __device__ __forceinline__ int mnmajor_swz(int r) {
  constexpr int NG = ROW_BYTES / 32;
  return ROW_BYTES >= 256 ? (((r & 3) << 1) & (NG - 1)) : (((r >> 1) & 1) << 1);
}
template <int ROW_BYTES> __device__ __forceinline__ int mnmajor_off(int r, int cbyte) {
  const int g = (cbyte >> 5) ^ mnmajor_swz<ROW_BYTES>(r);
  return r * ROW_BYTES + (g << 5) + (cbyte & 31);
}


// XCD-aware tile order: consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its
// own L2.  Every XCD gets a compact xcd_rm x xcd_cn block of the tile grid (chosen on the host to
// minimise the operand bytes the 8 L2s fetch between them), walked M-fastest; when the grid does not
// split that way, a contiguous run of M-fastest tile ids instead.
__device__ __forceinline__ void xcd_tile(const GemmArgs& p, int w, int& tile_m, int& tile_n) {
  const int xcd = w & 7, local = w >> 3;
  if (p.xcd_rm) {
    const int nbx = p.grid_m / p.xcd_rm;
    tile_m = (xcd % nbx) * p.xcd_rm + local % p.xcd_rm;
    tile_n = (xcd / nbx) * p.xcd_cn + local / p.xcd_rm;
  } else {
    const int tiles = p.grid_m * p.grid_n;
    const int per = (tiles + 7) >> 3, tall = (tiles & 7) ? (tiles & 7) : 8;
    const int tile_id = xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
    tile_m = tile_id % p.grid_m;
    tile_n = tile_id / p.grid_m;
  }
}


// LDS fragment reads as inline asm: the compiler's wait-count pass would otherwise put a full
// vmcnt(0) in front of LDS reads that follow an LDS-DMA load, which serialises the pipeline.
// lds_wait() is the matching s_waitcnt; it names the fragment registers as in/out operands so
// that no MFMA using them can be scheduled above it.
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const char*)p);
}
__device__ __forceinline__ void lds_read(bf16x8& f, uint32_t a) { asm volatile("ds_read_b128 %0, %1" : "=v"(f) : "v"(a)); }
__device__ __forceinline__ void lds_read(f32x4& f, uint32_t a) { asm volatile("ds_read_b128 %0, %1" : "=v"(f) : "v"(a)); }
__device__ __forceinline__ void lds_read_tr(s16x4& f, uint32_t a) { asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(f) : "v"(a)); }
__device__ __forceinline__ void lds_read_b32(float& f, uint32_t a) { asm volatile("ds_read_b32 %0, %1" : "=v"(f) : "v"(a)); }
template <typename F> __device__ __forceinline__ void lds_wait1(F& a) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a)); }

// Registers an LDS read lands in, kept apart from the MFMA operand until lds_wait() has run: any
// register copy the compiler makes to assemble the operand then happens after the data arrived.
template <typename T, int MAJOR> struct RawFrag { typename Mma<T>::Frag v; };
template <> struct RawFrag<bf16, DS_MN_MAJOR> { s16x4 lo, hi; };
template <> struct RawFrag<float, DS_MN_MAJOR> { float e0, e1, e2, e3; };

template <typename T> __device__ __forceinline__ void lds_wait(RawFrag<T, DS_K_MAJOR>& r) { lds_wait1(r.v); }
// Waits until at most N LDS reads are outstanding (they complete in order: everything but the newest N has
// arrived) and names the fragment registers as in/out operands so that nothing using them moves above it.
template <int N, typename T> __device__ __forceinline__ void lds_wait_n(RawFrag<T, DS_K_MAJOR>& r) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r.v) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait_n(RawFrag<bf16, DS_MN_MAJOR>& r) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(r.lo), "+v"(r.hi) : "n"(N));
}
template <int N> __device__ __forceinline__ void lds_wait_n(RawFrag<float, DS_MN_MAJOR>& r) {
  asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(r.e0), "+v"(r.e1), "+v"(r.e2), "+v"(r.e3) : "n"(N));
}
__device__ __forceinline__ void lds_wait(RawFrag<bf16, DS_MN_MAJOR>& r) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r.lo), "+v"(r.hi));
}
__device__ __forceinline__ void lds_wait(RawFrag<float, DS_MN_MAJOR>& r) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r.e0), "+v"(r.e1), "+v"(r.e2), "+v"(r.e3));
}
template <typename T> __device__ __forceinline__ typename Mma<T>::Frag to_frag(const RawFrag<T, DS_K_MAJOR>& r) { return r.v; }
__device__ __forceinline__ bf16x8 to_frag(const RawFrag<bf16, DS_MN_MAJOR>& r) {
  union { s16x4 v[2]; bf16x8 f; } u;
  u.v[0] = r.lo; u.v[1] = r.hi;
  return u.f;
}
__device__ __forceinline__ f32x4 to_frag(const RawFrag<float, DS_MN_MAJOR>& r) {
  f32x4 f = {r.e0, r.e1, r.e2, r.e3};
  return f;
}


// Per-lane byte offsets (inside one operand tile) of the MFMA fragments a wave reads.
template <typename T, int W, int MAJOR, int NF> struct FragReader {
  static constexpr int ROW_BYTES = W * (int)sizeof(T);
  // LDS read instructions per fragment
  static constexpr int READS = MAJOR == DS_K_MAJOR ? 1 : (sizeof(T) == 2 ? 2 : 4);
  typedef RawFrag<T, MAJOR> Raw;
  uint32_t off[MAJOR == DS_K_MAJOR ? 4 : NF];

  // ks_base: the k-step that read(.., ks = 0) addresses (a wave that multiplies only the upper k-steps of a k-tile)
  __device__ __forceinline__ void init(int ft0, int lane, int ks_base = 0) {
    const int h = lane >> 5;
    if (MAJOR == DS_K_MAJOR) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) off[ks] = kmajor_off(ft0 + (lane & 31), (2 * (ks + ks_base) + h) & 7);
    } else if (sizeof(T) == 2) {
      const int s = lane & 15;
#pragma unroll
      for (int i = 0; i < NF; ++i) {
        const int col = ft0 + i * 32 + (((lane >> 4) & 1) << 4) + ((s & 3) << 2);
        off[i] = mnmajor_off<ROW_BYTES>(8 * h + (s >> 2), col * 2) + 16 * ks_base * ROW_BYTES;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NF; ++i) off[i] = mnmajor_off<ROW_BYTES>(4 * h, (ft0 + i * 32 + (lane & 31)) * 4);
    }
  }
  // issues the reads of fragment i, k-step ks from the tile at LDS byte address `tile`
  __device__ __forceinline__ void read(RawFrag<T, DS_K_MAJOR>& f, uint32_t tile, int i, int ks) const {
    lds_read(f.v, tile + off[ks] + i * (32 * 128));
  }
  __device__ __forceinline__ void read(RawFrag<bf16, DS_MN_MAJOR>& f, uint32_t tile, int i, int ks) const {
    // rows r and r+4 (and r+16) share (r & 3), so the swizzle term is the same: constant byte offsets
    lds_read_tr(f.lo, tile + off[i] + (16 * ks) * ROW_BYTES);
    lds_read_tr(f.hi, tile + off[i] + (16 * ks + 4) * ROW_BYTES);
  }
  __device__ __forceinline__ void read(RawFrag<float, DS_MN_MAJOR>& f, uint32_t tile, int i, int ks) const {
    // rows 4h..4h+3 differ in (r & 3): redo the granule swizzle per row (off[i] is row 4h, unswizzled)
    constexpr int NG = ROW_BYTES / 32;
    const uint32_t base = off[i];
    const uint32_t g = (base % ROW_BYTES) >> 5, within = base & 31, row0 = base / ROW_BYTES;
    lds_read_b32(f.e0, tile + (row0 + 8 * ks + 0) * ROW_BYTES + ((g ^ mnmajor_swz<ROW_BYTES>(0)) << 5) + within);
    lds_read_b32(f.e1, tile + (row0 + 8 * ks + 1) * ROW_BYTES + ((g ^ mnmajor_swz<ROW_BYTES>(1)) << 5) + within);
    lds_read_b32(f.e2, tile + (row0 + 8 * ks + 2) * ROW_BYTES + ((g ^ mnmajor_swz<ROW_BYTES>(2)) << 5) + within);
    lds_read_b32(f.e3, tile + (row0 + 8 * ks + 3) * ROW_BYTES + ((g ^ mnmajor_swz<ROW_BYTES>(3)) << 5) + within);
  }
};

typedef __attribute__((address_space(3))) void* lds_vptr;
typedef __attribute__((address_space(1))) void* glb_vptr;
__device__ __forceinline__ lds_vptr lds_at(uint32_t a) { return (lds_vptr)(uintptr_t)a; }


// Operand tiles global -> LDS without VGPR staging; a wave's load writes 64 consecutive 16-byte LDS slots, so the
// swizzle is applied to the global address a lane fetches.  Out-of-range free indices are clamped to the last valid
// row / vector (they only feed accumulators the epilogue never stores).  Loads are inline asm in the scalar-base form
//   global_load_lds_dwordx4 v_offset, s[base:base+1]     (M0 = LDS address of the wave's 1 KiB slot)
// A lane's 32-bit byte offset inside the operand tile never changes; the tile base is a uniform pointer
// advanced once per k-tile with scalar adds, so a load costs no vector ALU work at all.  The compiler does
// not know these are memory operations: every wait on them is an explicit s_waitcnt in the kernel.
template <typename T, int W, int MAJOR, int NW = 4> struct AsmDma {
  static constexpr int VEC = Vec16<T>::N;
  static constexpr int KT = Mma<T>::KT;
  static constexpr int NV = W / (8 * NW);  // 16-byte vectors per thread and k-tile
  static constexpr int ROW_BYTES = W * (int)sizeof(T);
  static constexpr int CPR = ROW_BYTES / 16;
  uint32_t voff[NV];
  uint64_t tile;      // uniform: address of the current k-tile of this block's operand panel
  int64_t step;       // bytes from one k-tile to the next
  int64_t seg_jump;   // segmented reduction: what to add on top of `step` when a segment ends
  int seg_tiles, seg_left;  // k-tiles per segment (0: no segments), k-tiles left in the current one

  // a value that is the same in every lane, moved to scalar registers so that it can be an asm "s" operand
  static __device__ __forceinline__ uint64_t uniform64(uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
  }

  __device__ __forceinline__ void init(const GemmArgs& p, const T* base, int64_t ld, int f0, int F, int kt0, int wave, int lane,
                                       int64_t seg_stride = 0) {
    const int64_t k0 = (int64_t)kt0 * KT;
    seg_tiles = 0; seg_left = 0; seg_jump = 0;
    if (MAJOR == DS_K_MAJOR) {
      tile = uniform64((uint64_t)(uintptr_t)(base + (int64_t)f0 * ld + k0));
      step = (int64_t)uniform64((uint64_t)((int64_t)KT * sizeof(T)));
    } else if (p.seg_ktiles > 0) {
      // k-tile kt0 is tile `within` of segment `seg`; a segment's rows are contiguous (stride ld)
      const int seg = kt0 / p.seg_ktiles, within = kt0 - seg * p.seg_ktiles;
      tile = uniform64((uint64_t)(uintptr_t)(base + (int64_t)seg * seg_stride + (int64_t)within * KT * ld + f0));
      step = (int64_t)uniform64((uint64_t)((int64_t)KT * ld * sizeof(T)));
      seg_tiles = __builtin_amdgcn_readfirstlane(p.seg_ktiles);
      seg_left = __builtin_amdgcn_readfirstlane(p.seg_ktiles - within);
      seg_jump = (int64_t)uniform64((uint64_t)((seg_stride - (int64_t)p.seg_ktiles * KT * ld) * (int64_t)sizeof(T)));
    } else {
      tile = uniform64((uint64_t)(uintptr_t)(base + k0 * ld + f0));
      step = (int64_t)uniform64((uint64_t)((int64_t)KT * ld * sizeof(T)));
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int p = (i * NW + wave) * 64 + lane;
      if (MAJOR == DS_K_MAJOR) {
        const int row = p >> 3, c = (p & 7) ^ kmajor_swz(row);
        int f = f0 + row;
        if (f > F - 1) f = F - 1;
        voff[i] = (uint32_t)(((int64_t)(f - f0) * ld + c * VEC) * (int64_t)sizeof(T));
      } else {
        const int r = p / CPR, pc = p % CPR;
        const int g = (pc >> 1) ^ mnmajor_swz<ROW_BYTES>(r);
        int f = f0 + (g * 2 + (pc & 1)) * VEC;
        if (f > F - VEC) f = F - VEC;
        voff[i] = (uint32_t)(((int64_t)r * ld + (f - f0)) * (int64_t)sizeof(T));
      }
    }
  }
  // load i of the current k-tile into the wave's slot of the tile buffer at LDS address `lds_tile`
  __device__ __forceinline__ void issue_one(uint32_t lds_tile, int wave_s, int i) {
    const uint32_t m0v = lds_tile + (uint32_t)(i * NW + wave_s) * 1024u;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(voff[i]), "s"(tile) : "memory", "m0");
  }
  __device__ __forceinline__ void advance() {
    tile += (uint64_t)step;
    if (MAJOR != DS_K_MAJOR && seg_tiles > 0 && --seg_left == 0) {  // uniform: scalar compare and add
      tile += (uint64_t)seg_jump;
      seg_left = seg_tiles;
    }
  }
  __device__ __forceinline__ void issue(uint32_t lds_tile, int wave_s) {
#pragma unroll
    for (int i = 0; i < NV; ++i) issue_one(lds_tile, wave_s, i);
    advance();
  }
};


// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14])
#define DS_VMCNT(n) (((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))

// The rest of an epilogue for 8 consecutive columns of one row of C: x[] holds alpha * acc + bias; idx is the element
// offset of the first column inside the (batch-offset) C matrix.  Residual / auxiliary reads and every store are
// 16-byte vectors.
template <typename T>
__device__ __forceinline__ void gemm_epilogue_vec8(const GemmArgs& p, int64_t c_off, int64_t idx, float (&x)[8]) {
  const int flags = p.flags;
  const bool tanh_form = (flags & DS_EPI_TANH_FORM) != 0;
  const bool out_f32 = (flags & (DS_EPI_OUT_F32 | DS_EPI_ACCUM)) != 0 || sizeof(T) == 4;
  float* Cf = reinterpret_cast<float*>(p.c) + c_off;
  const T* R = reinterpret_cast<const T*>(p.residual) + c_off;
  T* C2 = reinterpret_cast<T*>(p.c2) + c_off;
  if (flags & DS_EPI_RESIDUAL) {
    if (sizeof(T) == 2 && !(flags & DS_EPI_RESIDUAL_F32)) {
      const bf16x8 r = *reinterpret_cast<const bf16x8*>(R + idx);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] += (float)r[e];
    } else {
      const float* Rf = reinterpret_cast<const float*>(p.residual) + c_off;
      const f32x4 r0 = *reinterpret_cast<const f32x4*>(Rf + idx), r1 = *reinterpret_cast<const f32x4*>(Rf + idx + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[e] += r0[e]; x[4 + e] += r1[e]; }
    }
  }
  if (flags & DS_EPI_DGELU) {
    if (sizeof(T) == 2) {
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(C2 + idx);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] *= gelu_any_grad((float)a[e], tanh_form);
    } else {
      const f32x4 a0 = *reinterpret_cast<const f32x4*>(C2 + idx), a1 = *reinterpret_cast<const f32x4*>(C2 + idx + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[e] *= gelu_any_grad(a0[e], tanh_form); x[4 + e] *= gelu_any_grad(a1[e], tanh_form); }
    }
  }
  if (flags & DS_EPI_MUL) {
    if (sizeof(T) == 2) {
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(C2 + idx);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] *= (float)a[e];
    } else {
      const f32x4 a0 = *reinterpret_cast<const f32x4*>(C2 + idx), a1 = *reinterpret_cast<const f32x4*>(C2 + idx + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[e] *= a0[e]; x[4 + e] *= a1[e]; }
    }
  }
  if (flags & DS_EPI_RELU) {
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = fmaxf(x[e], 0.f);
  }
  // GELU outputs first (they need the pre-activation), then what is kept for backward
  float act[8];
  if (flags & DS_EPI_GELU) {
#pragma unroll
    for (int e = 0; e < 8; ++e) act[e] = gelu_any(x[e], tanh_form);
    if (flags & DS_EPI_GELU_GRAD) {
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = gelu_any_grad(x[e], tanh_form);
    }
  }
  if (flags & DS_EPI_MASK) {
    if (sizeof(T) == 2) {
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(C2 + idx);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = (float)a[e] > 0.f ? x[e] : 0.f;
    } else {
      const f32x4 a0 = *reinterpret_cast<const f32x4*>(C2 + idx), a1 = *reinterpret_cast<const f32x4*>(C2 + idx + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[e] = a0[e] > 0.f ? x[e] : 0.f; x[4 + e] = a1[e] > 0.f ? x[4 + e] : 0.f; }
    }
  }
  if (flags & DS_EPI_ACCUM) {
    if (p.splitk > 1) {
#pragma unroll
      for (int e = 0; e < 8; ++e) atomicAdd(Cf + idx + e, x[e]);
    } else {
      f32x4 c0 = *reinterpret_cast<f32x4*>(Cf + idx), c1 = *reinterpret_cast<f32x4*>(Cf + idx + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { c0[e] += x[e]; c1[e] += x[4 + e]; }
      *reinterpret_cast<f32x4*>(Cf + idx) = c0;
      *reinterpret_cast<f32x4*>(Cf + idx + 4) = c1;
    }
  } else if (out_f32) {
    f32x4 c0, c1;
#pragma unroll
    for (int e = 0; e < 4; ++e) { c0[e] = x[e]; c1[e] = x[4 + e]; }
    *reinterpret_cast<f32x4*>(Cf + idx) = c0;
    *reinterpret_cast<f32x4*>(Cf + idx + 4) = c1;
  } else {
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (bf16)x[e];
    *reinterpret_cast<bf16x8*>(reinterpret_cast<bf16*>(p.c) + c_off + idx) = o;
    if (sizeof(T) == 2 && (flags & DS_EPI_ROWDOT)) {
      // 8 neighbouring lanes hold the 64 columns of one head of this row (the vector index runs along the row first)
      const bf16x8 a = *reinterpret_cast<const bf16x8*>(C2 + idx);
      float d = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) d += (float)o[e] * (float)a[e];
      d += __shfl_xor(d, 1, 64);
      d += __shfl_xor(d, 2, 64);
      d += __shfl_xor(d, 4, 64);
      const int64_t row = idx / p.ldc, col = idx % p.ldc;
      if ((col & 63) == 0)
        p.rowdot[((row / p.rowdot_seq) * (p.n >> 6) + (col >> 6)) * p.rowdot_seq + row % p.rowdot_seq] = d;
    }
  }
  if (flags & DS_EPI_GELU) {
    if (sizeof(T) == 2) {
      bf16x8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (bf16)act[e];
      *reinterpret_cast<bf16x8*>(reinterpret_cast<bf16*>(p.c2) + c_off + idx) = o;
    } else {
      f32x4 c0, c1;
#pragma unroll
      for (int e = 0; e < 4; ++e) { c0[e] = act[e]; c1[e] = act[4 + e]; }
      *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.c2) + c_off + idx) = c0;
      *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.c2) + c_off + idx + 4) = c1;
    }
  }
}

// Splits the tile grid into 8 equal rm x cn blocks, one per XCD.  An XCD's L2 fetches the A rows of
// its rm row tiles and the B columns of its cn column tiles once: total operand traffic is
// proportional to m * (grid_n / cn) + n * (grid_m / rm).
inline void choose_xcd_block(GemmArgs& a) {
  a.xcd_rm = a.xcd_cn = 0;
  const int tiles = a.grid_m * a.grid_n;
  if (tiles % 8) return;
  const int per = tiles / 8;
  double best = 1e300;
  for (int rm = 1; rm <= a.grid_m; ++rm) {
    if (a.grid_m % rm || per % rm) continue;
    const int cn = per / rm;
    if (cn > a.grid_n || a.grid_n % cn) continue;
    const double cost = (double)a.m * (a.grid_n / cn) + (double)a.n * (a.grid_m / rm);
    if (cost < best) { best = cost; a.xcd_rm = rm; a.xcd_cn = cn; }
  }
}

}  // namespace dsgemm

// 8-wave bf16 kernels (gemm8.hip).  cfg: 0 = 256x256 block, 1 = 256x128, 2 = 128x128; needs k % 64 == 0 and the
// vector epilogue (GemmArgs::vec_epi).  splitk, ktiles_per_split, flags as for the 4-wave kernels.
// every k-slice must hold more than ds_gemm8_stages(cfg) k-tiles (the depth of the tile ring), all slices equal.
int ds_gemm8_stages(int cfg);
// Checks a ds_gemm descriptor and fills the launch arguments that follow from it alone (operands, shapes, strides,
// epilogue, vec_epi, wave priority); tiling, slicing and workspace fields are the caller's.
int ds_gemm_make_args(const ds_gemm_desc* d, dsgemm::GemmArgs* out, int* batch_out);
int ds_gemm8_launch(const dsgemm::GemmArgs& a, int cfg, int a_major, int b_major, int batch, hipStream_t stream);
// The 64x64 block whose four waves split the k-steps of every k-tile (gemm8.hip): bf16, vector epilogue, no k-slices, an
// even number (at least 4) of 64-deep k-tiles.
int ds_gemm_ks4_launch(const dsgemm::GemmArgs& a, int a_major, int b_major, int batch, hipStream_t stream);
