// MFMA GEMM for gfx950: C[m][n] (+)= alpha * sum_k A(m,k) * B(n,k), bf16 or fp32 operands,
// fp32 accumulation, either operand K-major or MN-major, optional two-level batch strides.
//
// Tiling: a 256-thread block (4 waves as 2x2) owns a BM x BN tile of C; each wave owns
// (BM/2) x (BN/2) as 32x32 MFMA tiles.  The reduction runs in k-tiles of 128 bytes per row
// (64 bf16 / 32 fp32).  Global -> registers -> LDS with two LDS stages and one barrier per
// k-tile; the next k-tile's global loads are in flight while the current one is multiplied.
//
// LDS layouts (both XOR-swizzled so that fragment reads and tile stores are conflict free):
//   K-major operand : [free row][128 B of k]; 16-byte chunk c of row r lives at chunk c ^ ((r >> 1) & 7).
//                     A lane reads its MFMA fragment as one 16-byte load.
//   MN-major operand: [k row][free index contiguous]; 32-byte granule g of row r lives at
//                     g ^ (((r & 3) << 1) & (granules-1)).  bf16 fragments come from
//                     ds_read_b64_tr_b16 (a 4x16 transpose per 16 lanes), fp32 from 4-byte loads.
#include <stdlib.h>
#include <type_traits>
#include <string.h>

#include "gemm_core.h"

using namespace dsgemm;


namespace {


// One operand tile: W free indices x KT reduction elements = W*128 bytes, moved as W/32 16-byte
// vectors per thread.
template <typename T, int W, int MAJOR> struct OperandTile {
  static constexpr int VEC = Vec16<T>::N;
  static constexpr int KT = Mma<T>::KT;
  static constexpr int NV = W / 32;
  static constexpr int ROW_BYTES = W * (int)sizeof(T);  // MN-major row
  static constexpr int CPR = ROW_BYTES / 16;            // MN-major 16-byte chunks per row
  typedef typename Vec16<T>::type V;

  // f0: first free index of the tile, F: extent of the free index, k0: first reduction index
  static __device__ __forceinline__ void load(V (&regs)[NV], const T* base, int64_t ld, int f0, int F, int k0,
                                              int K, int tid) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = tid + i * 256;
      V val = {};
      if (MAJOR == DS_K_MAJOR) {
        const int row = v >> 3, chunk = v & 7;
        const int f = f0 + row, kk = k0 + chunk * VEC;
        if (f < F && kk < K) val = *reinterpret_cast<const V*>(base + (int64_t)f * ld + kk);
      } else {
        const int r = v / CPR, chunk = v % CPR;
        const int kk = k0 + r, f = f0 + chunk * VEC;
        if (kk < K && f < F) val = *reinterpret_cast<const V*>(base + (int64_t)kk * ld + f);
      }
      regs[i] = val;
    }
  }
  static __device__ __forceinline__ void store(const V (&regs)[NV], char* lds, int tid) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = tid + i * 256;
      int off;
      if (MAJOR == DS_K_MAJOR) {
        off = kmajor_off(v >> 3, v & 7);
      } else {
        off = mnmajor_off<ROW_BYTES>(v / CPR, (v % CPR) * 16);
      }
      *reinterpret_cast<V*>(lds + off) = regs[i];
    }
  }
  // fragment of the 32 free indices starting at tile-local index ft0, k-step ks
  static __device__ __forceinline__ typename Mma<T>::Frag frag(const char* lds, int ft0, int ks, int lane) {
    const int h = lane >> 5;
    if (MAJOR == DS_K_MAJOR) {
      return *reinterpret_cast<const typename Mma<T>::Frag*>(lds + kmajor_off(ft0 + (lane & 31), 2 * ks + h));
    } else {
      return frag_mn(lds, ft0, ks, lane, (T*)nullptr);
    }
  }
  static __device__ __forceinline__ bf16x8 frag_mn(const char* lds, int ft0, int ks, int lane, bf16*) {
    const int h = lane >> 5, s = lane & 15;
    const int col = ft0 + (((lane >> 4) & 1) << 4) + ((s & 3) << 2);
    typedef __attribute__((address_space(3))) s16x4* lds_ptr;
    union { s16x4 v[2]; bf16x8 f; } u;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int r = 16 * ks + 8 * h + 4 * t + (s >> 2);
      u.v[t] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(lds + mnmajor_off<ROW_BYTES>(r, col * 2)));
    }
    return u.f;
  }
  static __device__ __forceinline__ f32x4 frag_mn(const char* lds, int ft0, int ks, int lane, float*) {
    const int h = lane >> 5;
    const int col = ft0 + (lane & 31);
    f32x4 f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = 8 * ks + 4 * h + j;
      f[j] = *reinterpret_cast<const float*>(lds + mnmajor_off<ROW_BYTES>(r, col * 4));
    }
    return f;
  }
};

template <typename T, int BM, int BN>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& p, f32x16 (&acc)[BM / 64][BN / 64], int m0, int n0, int wm,
                                              int wn, int lane, int64_t c_off) {
  constexpr int TM = BM / 64, TN = BN / 64;
  // epilogue: lane holds column (lane & 31), rows (e/4)*8 + (lane>>5)*4 + (e&3) of each 32x32 tile
  const int flags = p.flags;
  const bool tanh_form = (flags & DS_EPI_TANH_FORM) != 0;
  const bool out_f32 = (flags & (DS_EPI_OUT_F32 | DS_EPI_ACCUM)) != 0 || sizeof(T) == 4;
  float* Cf = reinterpret_cast<float*>(p.c) + c_off;
  T* Ct = reinterpret_cast<T*>(p.c) + c_off;
  const T* R = reinterpret_cast<const T*>(p.residual) + c_off;
  T* C2 = reinterpret_cast<T*>(p.c2) + c_off;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wn * (BN / 2) + j * 32 + (lane & 31);
      if (col >= p.n) continue;
      const float bias = (flags & DS_EPI_BIAS) ? p.bias[col] : 0.f;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm * (BM / 2) + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (row >= p.m) continue;
        const int64_t idx = (int64_t)row * p.ldc + col;
        float v = acc[i][j][e] * p.alpha + bias;
        if (flags & DS_EPI_RESIDUAL)
          v += (flags & DS_EPI_RESIDUAL_F32) ? (reinterpret_cast<const float*>(p.residual) + c_off)[idx] : to_f32(R[idx]);
        if (flags & DS_EPI_DGELU) v *= gelu_any_grad(to_f32(C2[idx]), tanh_form);
        if (flags & DS_EPI_MUL) v *= to_f32(C2[idx]);
        if (flags & DS_EPI_RELU) v = fmaxf(v, 0.f);
        if (flags & DS_EPI_MASK) v = to_f32(C2[idx]) > 0.f ? v : 0.f;
        if (flags & DS_EPI_ACCUM) {
          if (p.splitk > 1) atomicAdd(Cf + idx, v); else Cf[idx] += v;
        } else {
          // with DS_EPI_GELU_GRAD the tensor kept for backward is gelu'(v) instead of the pre-activation v
          const float keep = (flags & DS_EPI_GELU_GRAD) ? gelu_any_grad(v, tanh_form) : v;
          if (out_f32) Cf[idx] = keep;
          else Ct[idx] = from_f32<T>(keep);
        }
        if (flags & DS_EPI_GELU) C2[idx] = from_f32<T>(gelu_any(v, tanh_form));
      }
    }
}


// Epilogue through LDS: accumulators (scaled, biased) are parked as fp32 rows in LDS, then every
// thread handles 8 consecutive columns of one row, so residual / aux reads and C writes are
// 16-byte vectors that cover whole rows of the tile.  Needs n, ldc and the C-side batch strides
// to be multiples of 8 and 16-byte aligned bases (checked on the host: GemmArgs::vec_epi).
template <typename T, int BM, int BN>
__device__ __forceinline__ void gemm_epilogue_staged(const GemmArgs& p, f32x16 (&acc)[BM / 64][BN / 64], int m0, int n0,
                                                     int wm, int wn, int lane, int tid, int64_t c_off, char* lds) {
  constexpr int TM = BM / 64, TN = BN / 64;
  constexpr int LDW = BN + 4;
  constexpr int VPR = BN / 8;             // 8-column vectors per tile row
  constexpr int ITER = BM * VPR / 256;    // vectors per thread
  float* sc = reinterpret_cast<float*>(lds);
  const int flags = p.flags;
  float* Cf = reinterpret_cast<float*>(p.c) + c_off;
  // C += acc with nothing else in the epilogue: fetch this thread's share of C now, in one batch, so
  // that the round trip to memory runs under the LDS staging below instead of once per vector afterwards
  const bool preload = (flags & DS_EPI_ACCUM) && p.splitk == 1 &&
                       (flags & ~(DS_EPI_ACCUM | DS_EPI_BIAS | DS_EPI_OUT_F32)) == 0;
  f32x4 cpre[ITER][2];
  if (preload) {
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int v = tid + it * 256;
      const int row = m0 + v / VPR, col = n0 + (v % VPR) * 8;
      if (row < p.m && col < p.n) {
        const float* src = Cf + (int64_t)row * p.ldc + col;
        cpre[it][0] = *reinterpret_cast<const f32x4*>(src);
        cpre[it][1] = *reinterpret_cast<const f32x4*>(src + 4);
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int cl = wn * (BN / 2) + j * 32 + (lane & 31);
      const int col = n0 + cl;
      const float bias = ((flags & DS_EPI_BIAS) && col < p.n) ? p.bias[col] : 0.f;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int rl = wm * (BM / 2) + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        sc[rl * LDW + cl] = acc[i][j][e] * p.alpha + bias;
      }
    }
  __syncthreads();
  if (preload) {
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int v = tid + it * 256;
      const int rl = v / VPR, cl = (v % VPR) * 8;
      const int row = m0 + rl, col = n0 + cl;
      if (row >= p.m || col >= p.n) continue;
      const f32x4 lo = *reinterpret_cast<const f32x4*>(sc + rl * LDW + cl);
      const f32x4 hi = *reinterpret_cast<const f32x4*>(sc + rl * LDW + cl + 4);
      float* dst = Cf + (int64_t)row * p.ldc + col;
      *reinterpret_cast<f32x4*>(dst) = cpre[it][0] + lo;
      *reinterpret_cast<f32x4*>(dst + 4) = cpre[it][1] + hi;
    }
    return;
  }
#pragma unroll 2
  for (int v = tid; v < BM * VPR; v += 256) {
    const int rl = v / VPR, cl = (v % VPR) * 8;
    const int row = m0 + rl, col = n0 + cl;
    if (row >= p.m || col >= p.n) continue;
    const int64_t idx = (int64_t)row * p.ldc + col;
    float x[8];
    {
      const f32x4 lo = *reinterpret_cast<const f32x4*>(sc + rl * LDW + cl);
      const f32x4 hi = *reinterpret_cast<const f32x4*>(sc + rl * LDW + cl + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[e] = lo[e]; x[4 + e] = hi[e]; }
    }
    gemm_epilogue_vec8<T>(p, c_off, idx, x);
  }
}

template <typename T, int BM, int BN, int AMAJ, int BMAJ>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs p) {
  typedef OperandTile<T, BM, AMAJ> TA;
  typedef OperandTile<T, BN, BMAJ> TB;
  constexpr int KT = Mma<T>::KT;
  constexpr int TM = BM / 64, TN = BN / 64;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128;
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int tile_m, tile_n;
  xcd_tile(p, blockIdx.x, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int z = blockIdx.z / p.splitk, ks_id = blockIdx.z % p.splitk;
  const int zo = z / p.batch_inner, zi = z % p.batch_inner;
  const T* A = reinterpret_cast<const T*>(p.a) + zo * p.a_so + zi * p.a_si;
  const T* B = reinterpret_cast<const T*>(p.b) + zo * p.b_so + zi * p.b_si;
  const int64_t c_off = zo * p.c_so + zi * p.c_si;

  const int kt_begin = ks_id * p.ktiles_per_split;
  const int kt_total = (p.k + KT - 1) / KT;
  int kt_end = kt_begin + p.ktiles_per_split;
  if (kt_end > kt_total) kt_end = kt_total;
  const int nkt = kt_end - kt_begin;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  typename TA::V ra[TA::NV];
  typename TB::V rb[TB::NV];
  if (nkt > 0) {
    TA::load(ra, A, p.lda, m0, p.m, kt_begin * KT, p.k, tid);
    TB::load(rb, B, p.ldb, n0, p.n, kt_begin * KT, p.k, tid);
  }
  for (int kt = 0; kt < nkt; ++kt) {
    char* sa = lds + (kt & 1) * (A_BYTES + B_BYTES);
    char* sb = sa + A_BYTES;
    TA::store(ra, sa, tid);
    TB::store(rb, sb, tid);
    __syncthreads();
    if (kt + 1 < nkt) {
      TA::load(ra, A, p.lda, m0, p.m, (kt_begin + kt + 1) * KT, p.k, tid);
      TB::load(rb, B, p.ldb, n0, p.n, (kt_begin + kt + 1) * KT, p.k, tid);
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      typename Mma<T>::Frag fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = TA::frag(sa, wm * (BM / 2) + i * 32, ks, lane);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = TB::frag(sb, wn * (BN / 2) + j * 32, ks, lane);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) Mma<T>::mma(acc[i][j], fa[i], fb[j]);
    }
  }

  gemm_epilogue<T, BM, BN>(p, acc, m0, n0, wm, wn, lane, c_off);
}


// ------------------------------------------------------------------------------------------
// Pipelined variant for k % KT == 0: tiles go global -> LDS directly (global_load_lds_dwordx4,
// no VGPR staging), STAGES k-tiles deep, so several k-tiles of loads are in flight while one is
// multiplied.  A wave's DMA writes 64 consecutive 16-byte LDS slots, so the swizzle is applied
// to the global address each lane fetches instead of to the LDS address it stores to.
// Out-of-range free indices are clamped to the last valid row/vector: they only feed
// accumulators of rows/columns the epilogue never stores.
template <typename T, int W, int MAJOR> struct PlainDma {
  static constexpr int VEC = Vec16<T>::N;
  static constexpr int KT = Mma<T>::KT;
  static constexpr int NV = W / 32;
  static constexpr int ROW_BYTES = W * (int)sizeof(T);
  static constexpr int CPR = ROW_BYTES / 16;
  const T* src[NV];
  int64_t step;

  // per-lane source pointers for k-tile kt0; slot i of wave w covers LDS positions (i*4+w)*64 + lane
  __device__ __forceinline__ void init(const GemmArgs&, const T* base, int64_t ld, int f0, int F, int kt0, int wave,
                                       int lane) {
    const int k0 = kt0 * KT;
    step = (MAJOR == DS_K_MAJOR) ? (int64_t)KT : (int64_t)KT * ld;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int p = (i * 4 + wave) * 64 + lane;
      if (MAJOR == DS_K_MAJOR) {
        const int row = p >> 3, c = (p & 7) ^ kmajor_swz(row);
        int f = f0 + row;
        if (f > F - 1) f = F - 1;
        src[i] = base + (int64_t)f * ld + k0 + c * VEC;
      } else {
        constexpr int NG = ROW_BYTES / 32;
        const int r = p / CPR, pc = p % CPR;
        const int g = (pc >> 1) ^ mnmajor_swz<ROW_BYTES>(r);
        int f = f0 + (g * 2 + (pc & 1)) * VEC;
        if (f > F - VEC) f = F - VEC;
        src[i] = base + (int64_t)(k0 + r) * ld + f;
      }
    }
  }
  // load i of the current k-tile (i = 0 .. NV-1, each exactly once per k-tile), then advance()
  __device__ __forceinline__ void issue_one(uint32_t lds_tile, int wave, int i) {
    __builtin_amdgcn_global_load_lds((glb_vptr)src[i], lds_at(lds_tile + (i * 4 + wave) * 1024), 16, 0, 0);
    src[i] += step;
  }
  __device__ __forceinline__ void advance() {}
  __device__ __forceinline__ void issue(uint32_t lds_tile, int wave) {
#pragma unroll
    for (int i = 0; i < NV; ++i) issue_one(lds_tile, wave, i);
    advance();
  }
};

// Source of zeros for the taps of a 3x3 'same' convolution that fall outside the image.
__device__ __attribute__((aligned(16))) float g_zero16[4] = {0.f, 0.f, 0.f, 0.f};

// Implicit-GEMM gather of a 3x3, stride 1, 'same' convolution over an NHWC tensor X[P = N*H*W, C]:
//   MODE 1 (K-major A, forward / dgrad): A(m = pixel p, k = (tap, c)) = X[p shifted by tap][c];
//           one k-tile is KT consecutive channels of one tap (needs C % KT == 0).
//   MODE 2 (MN-major A, wgrad): A(m = (tap, c), k = pixel p) = X[p shifted by tap][c]; a 16-byte
//           vector is VEC consecutive channels of one tap (needs C % VEC == 0).
// Shifted pixels outside the image read g_zero16 instead.
template <typename T, int W, int MODE> struct ConvDma {
  static constexpr int VEC = Vec16<T>::N;
  static constexpr int KT = Mma<T>::KT;
  static constexpr int NV = W / 32;
  static constexpr int ROW_BYTES = W * (int)sizeof(T);
  static constexpr int CPR = ROW_BYTES / 16;
  const T* base;
  int H, Wd, C;
  // MODE 1
  int64_t off[NV];
  int y[NV], x[NV];
  int tap, c0;
  // MODE 2
  int shift[NV];  // (dy * Wd + dx) * C + c
  int dyx[NV];    // (dy + 1) * 4 + (dx + 1)
  int r[NV];
  int64_t pix0;

  __device__ __forceinline__ void init(const GemmArgs& p, const T* b, int64_t, int f0, int F, int kt0, int wave, int lane, int64_t = 0) {
    base = b; H = p.conv_h; Wd = p.conv_w; C = p.conv_c;
    if (MODE == 1) {
      const int kpt = C / KT;
      tap = kt0 / kpt;
      c0 = (kt0 - tap * kpt) * KT;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int pos = (i * 4 + wave) * 64 + lane;
        const int row = pos >> 3, c = (pos & 7) ^ kmajor_swz(row);
        int pix = f0 + row;
        if (pix > F - 1) pix = F - 1;
        x[i] = pix % Wd;
        y[i] = (pix / Wd) % H;
        off[i] = (int64_t)pix * C + c * VEC;
      }
    } else {
      pix0 = (int64_t)kt0 * KT;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        constexpr int NG = ROW_BYTES / 32;
        const int pos = (i * 4 + wave) * 64 + lane;
        const int rr = pos / CPR, pc = pos % CPR;
        const int g = (pc >> 1) ^ mnmajor_swz<ROW_BYTES>(rr);
        int mi = f0 + (g * 2 + (pc & 1)) * VEC;
        if (mi > F - VEC) mi = F - VEC;
        const int t = mi / C, c = mi - t * C;
        const int dy = t / 3 - 1, dx = t - (t / 3) * 3 - 1;
        shift[i] = (dy * Wd + dx) * C + c;
        dyx[i] = (dy + 1) * 4 + (dx + 1);
        r[i] = rr;
      }
    }
  }
  // load i of the current k-tile (i = 0 .. NV-1, each exactly once per k-tile), then advance()
  __device__ __forceinline__ void issue_one(uint32_t lds_tile, int wave, int i) {
    if (MODE == 1) {
      const int dy = tap / 3 - 1, dx = tap - (tap / 3) * 3 - 1;
      const int sh = (dy * Wd + dx) * C + c0;
      const bool ok = (unsigned)(y[i] + dy) < (unsigned)H && (unsigned)(x[i] + dx) < (unsigned)Wd;
      const T* src = ok ? base + off[i] + sh : reinterpret_cast<const T*>(g_zero16);
      __builtin_amdgcn_global_load_lds((glb_vptr)src, lds_at(lds_tile + (i * 4 + wave) * 1024), 16, 0, 0);
    } else {
      const int64_t pix = pix0 + r[i];
      const int q = (int)(pix / Wd);
      const int xx = (int)(pix - (int64_t)q * Wd), yy = q % H;
      const int dy = (dyx[i] >> 2) - 1, dx = (dyx[i] & 3) - 1;
      const bool ok = (unsigned)(yy + dy) < (unsigned)H && (unsigned)(xx + dx) < (unsigned)Wd;
      const T* src = ok ? base + pix * C + shift[i] : reinterpret_cast<const T*>(g_zero16);
      __builtin_amdgcn_global_load_lds((glb_vptr)src, lds_at(lds_tile + (i * 4 + wave) * 1024), 16, 0, 0);
    }
  }
  __device__ __forceinline__ void advance() {
    if (MODE == 1) {
      c0 += KT;
      if (c0 == C) { c0 = 0; ++tap; }
    } else {
      pix0 += KT;
    }
  }
  __device__ __forceinline__ void issue(uint32_t lds_tile, int wave) {
#pragma unroll
    for (int i = 0; i < NV; ++i) issue_one(lds_tile, wave, i);
    advance();
  }
};

template <typename T, int W, int MAJOR, int CONV> struct DmaSelect { typedef AsmDma<T, W, MAJOR> type; };
template <typename T, int W> struct DmaSelect<T, W, DS_K_MAJOR, 1> { typedef ConvDma<T, W, 1> type; };
template <typename T, int W> struct DmaSelect<T, W, DS_MN_MAJOR, 2> { typedef ConvDma<T, W, 2> type; };

// Waits until at most min(later, MAXL) k-tiles' loads (LPT per thread each) are still outstanding.
template <int LPT, int MAXL> __device__ __forceinline__ void wait_tiles_in_flight(int later) {
  static_assert(LPT * MAXL <= 63, "the vmcnt field holds 6 bits");
  if constexpr (MAXL <= 0) {
    __builtin_amdgcn_s_waitcnt(DS_VMCNT(0));
  } else {
    if (later >= MAXL) __builtin_amdgcn_s_waitcnt(DS_VMCNT(LPT * MAXL));
    else wait_tiles_in_flight<LPT, MAXL - 1>(later);
  }
}

template <typename T, int BM, int BN, int AMAJ, int BMAJ, int STAGES, int CONVA = 0>
__global__ __launch_bounds__(256) void gemm_dma_kernel(GemmArgs p) {
  typedef typename DmaSelect<T, BM, AMAJ, CONVA>::type DA;
  typedef AsmDma<T, BN, BMAJ> DB;
  constexpr int KT = Mma<T>::KT;
  constexpr int TM = BM / 64, TN = BN / 64;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int LPT = DA::NV + DB::NV;  // DMA loads per thread per k-tile
  extern __shared__ __attribute__((aligned(16))) char lds[];

  ds_wave_prio(p.prio);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int tile_m, tile_n;
  xcd_tile(p, blockIdx.x, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int z = blockIdx.z / p.splitk, ks_id = blockIdx.z % p.splitk;
  const int zo = z / p.batch_inner, zi = z % p.batch_inner;
  const T* A = reinterpret_cast<const T*>(p.a) + zo * p.a_so + zi * p.a_si;
  const T* B = reinterpret_cast<const T*>(p.b) + zo * p.b_so + zi * p.b_si;
  const int64_t c_off = zo * p.c_so + zi * p.c_si;

  const int kt_begin = ks_id * p.ktiles_per_split;
  const int kt_total = p.k / KT;
  int kt_end = kt_begin + p.ktiles_per_split;
  if (kt_end > kt_total) kt_end = kt_total;
  const int nkt = kt_end - kt_begin;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  DA da;
  DB db;
  da.init(p, A, p.lda, m0, p.m, kt_begin, wave, lane, p.a_seg);
  db.init(p, B, p.ldb, n0, p.n, kt_begin, wave, lane, p.b_seg);
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);  // scalar copy: LDS slot addresses stay in SGPRs
  const uint32_t lds0 = lds_addr(lds);
  // Ring of STAGES tile buffers, tile t in buffer t % STAGES.  All STAGES buffers are filled up front.
  // Inside tile kt, under the first MFMA of its last k-step: every wave has read all of tile kt (its
  // fragment reads are waited for), waits for its own loads of tile kt+1 and meets the others at the
  // one barrier of the k-tile.  After it, tile kt+1 is visible, its first fragments are fetched under
  // the remaining MFMAs of tile kt, and buffer kt % STAGES is free: the loads of tile kt+STAGES go
  // there, issued one at a time between the next 4*TM*TN MFMAs (last k-step of tile kt, first three of
  // tile kt+1).  With one wave per SIMD a load or fragment read only hides behind an MFMA when it sits
  // between two MFMAs of the same instruction stream (a block of reads in front of the MFMAs is not
  // free): the order below is pinned with scheduling barriers.
#pragma unroll
  for (int s = 0; s < STAGES; ++s) {
    if (s < nkt) {
      da.issue(lds0 + s * STAGE_BYTES, wave_s);
      db.issue(lds0 + s * STAGE_BYTES + A_BYTES, wave_s);
    }
  }
  FragReader<T, BM, AMAJ, TM> ra;
  FragReader<T, BN, BMAJ, TN> rb;
  ra.init(wm * (BM / 2), lane);
  rb.init(wn * (BN / 2), lane);
  constexpr int NSLOT = TM * TN;      // MFMA groups per k-step
  constexpr int NMMA = 4 * NSLOT;     // per k-tile
  constexpr int NFR = TM + TN;        // fragments per k-step
  // Fragments run two k-steps ahead of the MFMAs in four register sets (set = k-step).  LDS reads complete
  // in order, so "at most one k-step's reads outstanding" means the older set has arrived; the lgkmcnt field
  // has 4 bits, a k-step with more reads than that waits for everything instead.
  constexpr int RPS = TM * FragReader<T, BM, AMAJ, TM>::READS + TN * FragReader<T, BN, BMAJ, TN>::READS;
  constexpr int WAITN = RPS <= 15 ? RPS : 0;
  RawFrag<T, AMAJ> fa[4][TM];
  RawFrag<T, BMAJ> fb[4][TN];
  {
    // tile 0 is complete once only the tiles issued after it are outstanding
    const int later = (nkt < STAGES ? nkt : STAGES) - 1;
    wait_tiles_in_flight<LPT, STAGES - 1>(later);
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int i = 0; i < TM; ++i) ra.read(fa[ks][i], lds0, i, ks);
#pragma unroll
      for (int j = 0; j < TN; ++j) rb.read(fb[ks][j], lds0 + A_BYTES, j, ks);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {  // landed before the loops are entered (see the end of k_tile)
#pragma unroll
      for (int i = 0; i < TM; ++i) lds_wait(fa[ks][i]);
#pragma unroll
      for (int j = 0; j < TN; ++j) lds_wait(fb[ks][j]);
    }
  }
  int buf = 0;  // kt % STAGES
  // One k-tile.  `steady` (a compile-time flag) says that tile kt-1+STAGES and tile kt+STAGES both exist: then
  // every refill load and fragment read below is unconditional and the k-tile is one straight run of code.
  auto k_tile = [&](auto steady, int kt) {
    constexpr bool ST = decltype(steady)::value;
    const uint32_t sa = lds0 + buf * STAGE_BYTES, sb = sa + A_BYTES;
    int pb = buf - 1;  // buffer of tile kt-1, being refilled with tile kt-1+STAGES
    if (pb < 0) pb += STAGES;
    const bool refill_prev = ST || (kt >= 1 && kt - 1 + STAGES < nkt);
    const bool refill_cur = ST || kt + STAGES < nkt;
    int nbuf = buf + 1;
    if (nbuf == STAGES) nbuf = 0;
    const uint32_t prev_tile = lds0 + pb * STAGE_BYTES, next_tile = lds0 + nbuf * STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      // set ks must have arrived; the set issued after it (k-step ks+1) may still be in flight
      if (ks < 3) {
#pragma unroll
        for (int i = 0; i < TM; ++i) lds_wait_n<WAITN>(fa[ks][i]);
#pragma unroll
        for (int j = 0; j < TN; ++j) lds_wait_n<WAITN>(fb[ks][j]);
      } else {
#pragma unroll
        for (int i = 0; i < TM; ++i) lds_wait(fa[ks][i]);
#pragma unroll
        for (int j = 0; j < TN; ++j) lds_wait(fb[ks][j]);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int slot = i * TN + j;            // compile-time after unrolling
          const int q = ks * NSLOT + slot;
          Mma<T>::mma(acc[i][j], to_frag(fa[ks][i]), to_frag(fb[ks][j]));
          __builtin_amdgcn_sched_barrier(0);
          if (ks == 3 && slot == 0) {
            // (also after the last tile, where it is a no-op wait and one more barrier: the fragment reads
            // below must not sit inside a conditional, see the end of k_tile)
            // tile kt+1 is complete once only the tiles issued after it are outstanding:
            // kt+2 .. kt-1+STAGES, as far as they exist
            if (ST) __builtin_amdgcn_s_waitcnt(DS_VMCNT(LPT * (STAGES - 2)));
            else wait_tiles_in_flight<LPT, STAGES - 2>(nkt - (kt + 2));
            __builtin_amdgcn_s_barrier();
          }
          // this slot's share of the fragment reads: k-steps 2 and 3 of this tile during k-steps 0 and 1, nothing
          // during k-step 2 (the next tile is not visible yet), k-steps 0 AND 1 of the next tile during k-step 3
          if (ks < 2) {
#pragma unroll
            for (int r = 0; r < NFR; ++r)
              if ((r * NSLOT) / NFR == slot) {
                if (r < TM) ra.read(fa[ks + 2][r], sa, r, ks + 2);
                else rb.read(fb[ks + 2][r - TM], sb, r - TM, ks + 2);
              }
          } else if (ks == 3) {
            // after the last tile these read a stale buffer into registers nobody uses
#pragma unroll
            for (int r = 0; r < 2 * NFR; ++r)
              if ((r * NSLOT) / (2 * NFR) == slot) {
                const int nks = r / NFR, rr = r % NFR;
                if (rr < TM) ra.read(fa[nks][rr], next_tile, rr, nks);
                else rb.read(fb[nks][rr - TM], next_tile + A_BYTES, rr - TM, nks);
              }
          }
          // this slot's share of the refill loads
          if (ks < 3) {
            // slots NSLOT .. NMMA-1 of the window that refills the buffer of tile kt-1
            if (refill_prev) {
#pragma unroll
              for (int l = 0; l < LPT; ++l)
                if ((l * NMMA) / LPT == q + NSLOT) {
                  if (l < DA::NV) da.issue_one(prev_tile, wave_s, l);
                  else db.issue_one(prev_tile + A_BYTES, wave_s, l - DA::NV);
                }
            }
          } else {
            // slots 0 .. NSLOT-1 of the window that refills the buffer of tile kt
            if (refill_cur) {
#pragma unroll
              for (int l = 0; l < LPT; ++l)
                if ((l * NMMA) / LPT == slot) {
                  if (l < DA::NV) da.issue_one(sa, wave_s, l);
                  else db.issue_one(sb, wave_s, l - DA::NV);
                }
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      if (ks == 2 && refill_prev) { da.advance(); db.advance(); }
    }
    // No LDS read may be in flight across a loop back-edge or between the loops below: the compiler is free
    // to copy a fragment register there, and a copy taken before the data has landed copies stale contents.
    // The first two k-steps of the next tile, fetched under the last four MFMA groups, are waited for here.
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int i = 0; i < TM; ++i) lds_wait(fa[ks][i]);
#pragma unroll
      for (int j = 0; j < TN; ++j) lds_wait(fb[ks][j]);
    }
    buf = nbuf;
  };
  // three loops, so that the straight-line steady state does not share an iteration with the general form
  // fp32 products add blocked partial sums: every FLUSH k-tiles (128 terms) the running accumulators are added to a
  // second set and start again from zero, so a reduction of k terms rounds like one of 128 followed by one of k / 128
  // (a plain run over 3000 terms loses about three times as much).  Folding after every k-tile instead gains another
  // 10 % on the GNMT encoder's gradients and costs 2.5 % of its step.  bf16 products round their inputs far above this.
  constexpr bool BLOCKED = std::is_same<T, float>::value && CONVA == 0;  // (the convolutions hold 1e-4 without, and pay 4 % for it)
  constexpr int FLUSH = 4;
  f32x16 tot[BLOCKED ? TM : 1][BLOCKED ? TN : 1];
  if (BLOCKED) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) tot[i][j][e] = 0.f;
  }
  auto flush = [&](int kt) {
    if (BLOCKED && (kt & (FLUSH - 1)) == FLUSH - 1) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            tot[BLOCKED ? i : 0][BLOCKED ? j : 0][e] += acc[i][j][e];
            acc[i][j][e] = 0.f;
          }
    }
  };
  int kt = 0;
  for (; kt < nkt && !(kt >= 1 && kt + STAGES < nkt); ++kt) { k_tile(std::false_type(), kt); flush(kt); }
  for (; kt + STAGES < nkt; ++kt) { k_tile(std::true_type(), kt); flush(kt); }
  for (; kt < nkt; ++kt) { k_tile(std::false_type(), kt); flush(kt); }
  if (BLOCKED) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] += tot[BLOCKED ? i : 0][BLOCKED ? j : 0][e];
  }
  if (p.vec_epi) gemm_epilogue_staged<T, BM, BN>(p, acc, m0, n0, wm, wn, lane, tid, c_off, lds);
  else gemm_epilogue<T, BM, BN>(p, acc, m0, n0, wm, wn, lane, c_off);
}

template <typename T, int BM, int BN, int AMAJ, int BMAJ, int STAGES>
int launch_dma(const GemmArgs& a, dim3 grid, hipStream_t stream) {
  constexpr size_t lds = (size_t)STAGES * (BM + BN) * 128;
  static std::atomic<bool> attr_set(false);  // two threads may both set the (idempotent) attribute; neither launches before it is set
  if (!attr_set) {
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)gemm_dma_kernel<T, BM, BN, AMAJ, BMAJ, STAGES>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  hipLaunchKernelGGL((gemm_dma_kernel<T, BM, BN, AMAJ, BMAJ, STAGES>), grid, dim3(256), lds, stream, a);
  return DS_OK;
}

template <typename T, int BM, int BN, int AMAJ, int BMAJ>
int launch_cfg(GemmArgs a, int batch, hipStream_t stream) {
  a.grid_m = (a.m + BM - 1) / BM;
  a.grid_n = (a.n + BN - 1) / BN;
  choose_xcd_block(a);
  dim3 grid(a.grid_m * a.grid_n, 1, batch * a.splitk);
  if (a.k % Mma<T>::KT == 0) {
    // 3 buffers: 96 KB for a 128x128 block, 48 KB for 64x64 - a CU's 160 KB of LDS then holds blocks of two or
    // three kernels at once.  With several streams feeding the GPU that co-residency is worth more than a deeper
    // ring: 6 buffers under the 64x64 block (long reductions, one block per CU) made the BERT-48 half-stage step
    // 3.6 % shorter with all its kernels on one stream and 7 % longer on three; 4 buffers (64 KB: the products of
    // 1024 x 1024 x 3072..4096 run 2 us faster alone) still 6 % longer - a third block no longer fits beside two.
    int rc = launch_dma<T, BM, BN, AMAJ, BMAJ, 3>(a, grid, stream);
    if (rc != DS_OK) return rc;
  } else {
    const size_t lds = 2 * (BM + BN) * 128;
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, AMAJ, BMAJ>), grid, dim3(256), lds, stream, a);
  }
  DS_CHECK_LAUNCH();
  return DS_OK;
}

template <typename T, int AMAJ, int BMAJ>
int launch_tile(const GemmArgs& a, int batch, int tile, hipStream_t stream) {
  switch (tile) {
    case 0: return launch_cfg<T, 128, 128, AMAJ, BMAJ>(a, batch, stream);
    case 1: return launch_cfg<T, 128, 64, AMAJ, BMAJ>(a, batch, stream);
    default: return launch_cfg<T, 64, 64, AMAJ, BMAJ>(a, batch, stream);
  }
}

template <typename T>
int launch_major(const GemmArgs& a, int batch, int tile, int am, int bm, hipStream_t stream) {
  if (am == DS_K_MAJOR && bm == DS_K_MAJOR) return launch_tile<T, DS_K_MAJOR, DS_K_MAJOR>(a, batch, tile, stream);
  if (am == DS_K_MAJOR && bm == DS_MN_MAJOR) return launch_tile<T, DS_K_MAJOR, DS_MN_MAJOR>(a, batch, tile, stream);
  if (am == DS_MN_MAJOR && bm == DS_MN_MAJOR) return launch_tile<T, DS_MN_MAJOR, DS_MN_MAJOR>(a, batch, tile, stream);
  return launch_tile<T, DS_MN_MAJOR, DS_K_MAJOR>(a, batch, tile, stream);
}

}  // namespace

// Picks the tile shape.  Measured on MI355X (bf16, 3-buffer ring): one k-tile costs about 0.5 us in a
// 128x128 block, and roughly in proportion to the tile's bytes below that; the k-loop repeats once
// per round of resident blocks.  With several streams feeding the GPU the choice is flat between
// 128x64 and 64x64 for narrow outputs; 128x128 on a grid of fewer than ~256 tiles loses.  Split-K is
// never chosen: its atomic epilogue was slower than the under-filled grid on every shape tried.
static void choose_tiling(int m, int n, int k, int kt, int batch, bool can_split, int* tile, int* splitk) {
  static const int bm[3] = {128, 128, 64}, bn[3] = {128, 64, 64};
  static const double slots[3] = {256, 512, 512}, t_round[3] = {0.6, 1.06, 0.45};
  double best = 1e300;
  *tile = 0;
  *splitk = 1;
  double best_blocks = 0;
  for (int t = 0; t < 3; ++t) {
    const double blocks = (double)((m + bm[t] - 1) / bm[t]) * ((n + bn[t] - 1) / bn[t]) * batch;
    const double rounds = (double)((long long)((blocks + slots[t] - 1) / slots[t]));
    const double cost = rounds * t_round[t];
    if (cost < best) { best = cost; *tile = t; best_blocks = blocks; }
  }
  // fp32 accumulation (C += A B^T) of a few tiles under a long reduction - a weight gradient over thousands of pixels
  // into a small kernel: the reduction is cut into slices that add their parts atomically, so that every CU has work
  if (can_split && kt == 32 && best_blocks <= 64 && k / kt >= 64) {
    int sk = (int)(256 / best_blocks);
    const int most = k / kt / 8;
    if (sk > most) sk = most;
    if (sk > 64) sk = 64;
    if (sk > 1) *splitk = sk;
  }
}

// C (fp32) = alpha * A B^T for bf16 operands with a reduction of exactly 64 (one attention head), both K-major:
// the score products q k^T / dO v^T.  A 64x64 tile of such a product is 16 KB of operands and 16 KB of output -
// nothing is reused often enough to stage it: every wave loads its fragments straight from global memory in MFMA
// operand order (lane = row, 8 consecutive k), multiplies 4 x 4 MFMAs and stores its accumulators, whose lanes run
// along n (128 contiguous bytes per half wave).  No LDS, no barrier: four such blocks fit a CU beside anything else.
__global__ __launch_bounds__(256) void gemm_k64_f32out_kernel(GemmArgs p) {
  ds_wave_prio(p.prio);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5, r = lane & 31;
  const int tiles_n = p.n / 64;
  const int64_t wt = (int64_t)blockIdx.x * 4 + wave;
  if (wt >= (int64_t)(p.m / 64) * tiles_n) return;
  const int m0 = (int)(wt / tiles_n) * 64, n0 = (int)(wt % tiles_n) * 64;
  const int z = blockIdx.z, zo = z / p.batch_inner, zi = z % p.batch_inner;
  const bf16* A = reinterpret_cast<const bf16*>(p.a) + zo * p.a_so + zi * p.a_si + (int64_t)(m0 + r) * p.lda + half * 8;
  const bf16* B = reinterpret_cast<const bf16*>(p.b) + zo * p.b_so + zi * p.b_si + (int64_t)(n0 + r) * p.ldb + half * 8;
  float* C = reinterpret_cast<float*>(p.c) + zo * p.c_so + zi * p.c_si;
  bf16x8 fa[2][4], fb[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      fa[i][ks] = *reinterpret_cast<const bf16x8*>(A + (int64_t)i * 32 * p.lda + ks * 16);
      fb[i][ks] = *reinterpret_cast<const bf16x8*>(B + (int64_t)i * 32 * p.ldb + ks * 16);
    }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      f32x16 acc;
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[e] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i][ks], fb[j][ks], acc, 0, 0, 0);
      float* c = C + (int64_t)(m0 + i * 32) * p.ldc + n0 + j * 32 + r;
#pragma unroll
      for (int e = 0; e < 16; ++e) c[(int64_t)((e >> 2) * 8 + half * 4 + (e & 3)) * p.ldc] = acc[e] * p.alpha;
    }
}

// Checks a descriptor and turns it into launch arguments (tiling, slicing and workspace fields are left to the caller).
int ds_gemm_make_args(const ds_gemm_desc* d, GemmArgs* out, int* batch_out) {
  DS_CHECK_ARG(d != nullptr, "ds_gemm: null descriptor");
  DS_CHECK_ARG(d->dtype == DS_F32 || d->dtype == DS_BF16, "ds_gemm: dtype %d", d->dtype);
  DS_CHECK_ARG((d->a_major | 1) == 1 && (d->b_major | 1) == 1, "ds_gemm: operand major must be 0 or 1");
  DS_CHECK_ARG(d->m > 0 && d->n > 0 && d->k > 0, "ds_gemm: m, n, k must be positive (%d %d %d)", d->m, d->n, d->k);
  DS_CHECK_ARG(d->a && d->b && d->c, "ds_gemm: null operand");
  const int vec = d->dtype == DS_BF16 ? 8 : 4;
  const int esz = d->dtype == DS_BF16 ? 2 : 4;
  const int batch = d->batch > 0 ? d->batch : 1;
  const int inner = d->batch_inner > 0 ? d->batch_inner : 1;
  // every 16-byte vector the loaders issue must be aligned and lie inside one row
  if (d->a_major == DS_K_MAJOR) DS_CHECK_ARG(d->k % vec == 0, "ds_gemm: k=%d must be a multiple of %d for a K-major A", d->k, vec);
  else DS_CHECK_ARG(d->m % vec == 0, "ds_gemm: m=%d must be a multiple of %d for an MN-major A", d->m, vec);
  if (d->b_major == DS_K_MAJOR) DS_CHECK_ARG(d->k % vec == 0, "ds_gemm: k=%d must be a multiple of %d for a K-major B", d->k, vec);
  else DS_CHECK_ARG(d->n % vec == 0, "ds_gemm: n=%d must be a multiple of %d for an MN-major B", d->n, vec);
  DS_CHECK_ARG(d->lda % vec == 0 && d->ldb % vec == 0, "ds_gemm: lda/ldb must be multiples of %d", vec);
  DS_CHECK_ARG(d->lda >= (d->a_major == DS_K_MAJOR ? d->k : d->m), "ds_gemm: lda too small");
  DS_CHECK_ARG(d->ldb >= (d->b_major == DS_K_MAJOR ? d->k : d->n), "ds_gemm: ldb too small");
  DS_CHECK_ARG(d->ldc >= d->n, "ds_gemm: ldc too small");
  DS_CHECK_ARG(ds_aligned16(d->a) && ds_aligned16(d->b), "ds_gemm: A and B must be 16-byte aligned");
  if (batch > 1) {
    DS_CHECK_ARG(d->a_stride_outer % vec == 0 && d->a_stride_inner % vec == 0 && d->b_stride_outer % vec == 0 &&
                 d->b_stride_inner % vec == 0, "ds_gemm: batch strides of A/B must be multiples of %d", vec);
    DS_CHECK_ARG(batch % inner == 0, "ds_gemm: batch %% batch_inner != 0");
  }
  const int f = d->flags;
  if (f & DS_EPI_BIAS) DS_CHECK_ARG(d->bias != nullptr, "ds_gemm: DS_EPI_BIAS without bias");
  if (f & DS_EPI_RESIDUAL) DS_CHECK_ARG(d->residual != nullptr, "ds_gemm: DS_EPI_RESIDUAL without residual");
  DS_CHECK_ARG(!(f & DS_EPI_RESIDUAL_F32) || (f & DS_EPI_RESIDUAL), "ds_gemm: DS_EPI_RESIDUAL_F32 needs DS_EPI_RESIDUAL");
  if (f & (DS_EPI_GELU | DS_EPI_DGELU | DS_EPI_MUL)) DS_CHECK_ARG(d->c2 != nullptr, "ds_gemm: GELU / MUL epilogue without c2");
  DS_CHECK_ARG(!(f & DS_EPI_GELU_GRAD) || (f & DS_EPI_GELU), "ds_gemm: DS_EPI_GELU_GRAD needs DS_EPI_GELU");
  DS_CHECK_ARG(!((f & DS_EPI_GELU) && (f & DS_EPI_DGELU)), "ds_gemm: GELU and DGELU are exclusive");
  DS_CHECK_ARG(!((f & DS_EPI_ACCUM) && (f & (DS_EPI_GELU | DS_EPI_DGELU))), "ds_gemm: ACCUM with GELU");
  DS_CHECK_ARG((f & ~0xFFF) == 0, "ds_gemm: unknown epilogue flags 0x%x", f & ~0xFFF);
  (void)esz;
  if (d->k_segment != 0) {
    const int kt = d->dtype == DS_BF16 ? 64 : 32;
    // (a K-major operand runs on along its rows whatever the segments: its segment stride is not used)
    DS_CHECK_ARG(d->a_major == DS_MN_MAJOR || d->b_major == DS_MN_MAJOR, "ds_gemm: a segmented reduction needs an MN-major operand");
    DS_CHECK_ARG(d->k_segment > 0 && d->k_segment % kt == 0 && d->k % d->k_segment == 0,
                 "ds_gemm: k_segment %d must be a multiple of %d that divides k = %d", d->k_segment, kt, d->k);
    DS_CHECK_ARG(d->a_segment_stride % vec == 0 && d->b_segment_stride % vec == 0, "ds_gemm: segment strides must be multiples of %d", vec);
  }

  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.a = (const char*)d->a; a.b = (const char*)d->b; a.c = (char*)d->c;
  a.bias = d->bias; a.residual = (const char*)d->residual; a.c2 = (char*)d->c2;
  a.m = d->m; a.n = d->n; a.k = d->k;
  a.lda = d->lda; a.ldb = d->ldb; a.ldc = d->ldc;
  a.batch_inner = inner;
  a.a_so = d->a_stride_outer; a.a_si = d->a_stride_inner;
  a.b_so = d->b_stride_outer; a.b_si = d->b_stride_inner;
  a.c_so = d->c_stride_outer; a.c_si = d->c_stride_inner;
  a.flags = f;
  a.alpha = d->alpha;
  a.prio = ds_launch_prio;
  a.ws_part = nullptr; a.ws_count = nullptr;
  if (d->k_segment != 0 && d->k_segment != d->k) {
    a.seg_ktiles = d->k_segment / (d->dtype == DS_BF16 ? 64 : 32);
    a.a_seg = d->a_segment_stride; a.b_seg = d->b_segment_stride;
  }
  a.vec_epi = d->n % 8 == 0 && d->ldc % 8 == 0 && d->c_stride_outer % 8 == 0 && d->c_stride_inner % 8 == 0 &&
              ds_aligned16(d->c) && ds_aligned16(d->residual) && ds_aligned16(d->c2);
  a.splitk = 1;
  *out = a;
  *batch_out = batch;
  return DS_OK;
}

static int gemm_run(const ds_gemm_desc* d, int splitk_req, void* stream, bool must_split = false) {
  GemmArgs a;
  int batch = 1;
  DS_PROPAGATE(ds_gemm_make_args(d, &a, &batch));
  const int f = d->flags;
  if (d->dtype == DS_BF16 && d->a_major == DS_K_MAJOR && d->b_major == DS_K_MAJOR && d->k == 64 && f == DS_EPI_OUT_F32 &&
      d->m % 64 == 0 && d->n % 64 == 0 && batch <= 65535) {
    hipStream_t s = (hipStream_t)stream;
    ds_prof_scope prof(s, "gemm_k64_f32out_kernel<bf16>", 2.0 * d->m * d->n * d->k * batch, "FLOP");
    const int64_t wave_tiles = (int64_t)(d->m / 64) * (d->n / 64);
    hipLaunchKernelGGL(gemm_k64_f32out_kernel, dim3((unsigned)((wave_tiles + 3) / 4), 1, batch), dim3(256), 0, s, a);
    DS_CHECK_LAUNCH();
    return DS_OK;
  }
  const int kt = d->dtype == DS_BF16 ? 64 : 32;
  int tile, splitk;
  choose_tiling(d->m, d->n, d->k, kt, batch, (f & DS_EPI_ACCUM) != 0, &tile, &splitk);
  {  // tuning overrides: DS_GEMM_TILE=0|1|2, DS_GEMM_SPLITK=n (accumulating outputs only)
    static const char* env_tile = getenv("DS_GEMM_TILE");
    static const char* env_split = getenv("DS_GEMM_SPLITK");
    if (env_tile) tile = atoi(env_tile) % 3;

    if (env_split && (f & DS_EPI_ACCUM)) splitk = atoi(env_split) > 0 ? atoi(env_split) : 1;
  }
  const int ktiles = (d->k + kt - 1) / kt;
  if (splitk_req > 1 && (f & DS_EPI_ACCUM)) splitk = splitk_req < ktiles ? splitk_req : ktiles;
  if (splitk > 1) a.vec_epi = 0;  // atomics want neighbouring lanes on neighbouring addresses
  a.ktiles_per_split = (ktiles + splitk - 1) / splitk;
  splitk = (ktiles + a.ktiles_per_split - 1) / a.ktiles_per_split;   // no slice without a k-tile
  a.splitk = splitk;
  hipStream_t s = (hipStream_t)stream;
  if (d->dtype == DS_BF16 && d->k % 64 == 0 && a.vec_epi && splitk == 1) {
    // 8-wave kernels (gemm8.hip).  Block shape by the number of output tiles: 256x256 and 256x128 blocks need about a
    // tile per CU to pay (0.8 -> 1.1 PFLOP/s on 4096^3); 128x128 with the same 96 KB of LDS as the 4-wave block it
    // replaces (what else fits on the CU beside a block decides a multi-stream step more than the block's own speed).
    // DS_GEMM8 = -1 switches them off, 0..4 forces a shape wherever it applies.
    static const char* env8 = getenv("DS_GEMM8");
    static const char* env_sk = getenv("DS_GEMM_SPLITK_WS");  // 0: never split, n > 1: n slices wherever k divides
    static const int bm8[6] = {256, 256, 128, 128, 128, 128}, bn8[6] = {256, 128, 128, 128, 128, 64};
    auto tiles_of = [&](int c) { return (int64_t)((d->m + bm8[c] - 1) / bm8[c]) * ((d->n + bn8[c] - 1) / bn8[c]) * batch; };
    int cfg8 = -1;
    if (env8) {
      cfg8 = atoi(env8);
      if (cfg8 > 5) cfg8 = -1;
    } else if (tiles_of(0) >= 200) {
      cfg8 = 0;
    } else if (tiles_of(1) >= 200) {
      cfg8 = 1;
    } else if (tiles_of(4) >= 192) {
      cfg8 = 4;
    }
    // Split-K through the caller's workspace: a handful of output tiles under a very long k (a few tiles cannot fill
    // the GPU; the exchange of partial tiles costs about 8 us, so it only pays when a slice is still long).
    if (batch == 1 && d->workspace != nullptr) {
      const int64_t tiles = tiles_of(4);
      int slices = 0;
      for (int c = 4; c >= 2 && !slices; --c)
        if (tiles * c <= 64 && ktiles % c == 0 && ktiles / c >= 32) slices = c;
      if (env_sk) {
        const int forced = atoi(env_sk);
        slices = forced <= 1 || forced > 4 || tiles > 1024 ? 0 : (ktiles % forced == 0 && ktiles / forced > ds_gemm8_stages(4) ? forced : 0);
      }
      if (must_split && slices <= 1) {
        ds_set_error("ds_gemm_static_scratch: %d x %d x %d is not a shape that is cut into k slices (at most 64 tile-slices of "
                     "128 x 128, every slice at least 32 k-tiles of 64)", d->m, d->n, d->k);
        return DS_EINVAL;
      }
      if (slices > 1) {
        DS_CHECK_ARG(((uintptr_t)d->workspace & 255) == 0 && d->workspace_bytes >= ds_gemm_workspace_bytes(d->m, d->n),
                     "ds_gemm: workspace must be 256-byte aligned and hold ds_gemm_workspace_bytes(m, n) = %zu bytes (got %zu)",
                     ds_gemm_workspace_bytes(d->m, d->n), d->workspace_bytes);
        a.splitk = slices;
        a.ktiles_per_split = ktiles / slices;
        a.ws_count = (unsigned*)d->workspace;
        a.ws_part = (float*)((char*)d->workspace + 4096);
        a.ws_bytes = d->workspace_bytes - 4096;
        char tagk[96];
        snprintf(tagk, sizeof(tagk), "gemm8_kernel<bf16,128,128,%s,%s>/k%d", d->a_major == DS_K_MAJOR ? "K" : "MN",
                 d->b_major == DS_K_MAJOR ? "K" : "MN", slices);
        ds_prof_scope profk(s, tagk, 2.0 * d->m * d->n * d->k, "FLOP");
        return ds_gemm8_launch(a, 4, d->a_major, d->b_major, 1, s);
      }
    }
    if (must_split) {
      ds_set_error("ds_gemm_static_scratch: batched GEMMs are not cut into k slices");
      return DS_EINVAL;
    }
    if (cfg8 >= 0 && ktiles > ds_gemm8_stages(cfg8)) {
      char tag8[96];
      snprintf(tag8, sizeof(tag8), "gemm8_kernel<bf16,%d,%d,%s,%s>", bm8[cfg8], bn8[cfg8],
               d->a_major == DS_K_MAJOR ? "K" : "MN", d->b_major == DS_K_MAJOR ? "K" : "MN");
      ds_prof_scope prof8(s, tag8, 2.0 * d->m * d->n * d->k * batch, "FLOP");
      return ds_gemm8_launch(a, cfg8, d->a_major, d->b_major, batch, s);
    }
  }
  if (must_split) {
    ds_set_error("ds_gemm_static_scratch: needs bf16 operands, k a multiple of 64 and 16-byte aligned, 8-column outputs");
    return DS_EINVAL;
  }
  {
    // 64x64 blocks under a long reduction: the four waves split the k-steps of every k-tile instead of the tile (half the
    // LDS fragment reads for the same 48 KB; gemm8_core.h).  DS_GEMM_KS4 = 0 switches it off, n sets the least number of k-tiles.
    static const char* env_ks = getenv("DS_GEMM_KS4");
    const int least = env_ks ? atoi(env_ks) : 16;
    if (least > 0 && tile == 2 && d->dtype == DS_BF16 && d->k % 64 == 0 && a.vec_epi && splitk == 1 && ktiles % 2 == 0 && ktiles >= 4 &&
        ktiles >= least) {
      char tagk[96];
      snprintf(tagk, sizeof(tagk), "gemm_ks4_kernel<bf16,64,64,%s,%s>", d->a_major == DS_K_MAJOR ? "K" : "MN",
               d->b_major == DS_K_MAJOR ? "K" : "MN");
      ds_prof_scope profk(s, tagk, 2.0 * d->m * d->n * d->k * batch, "FLOP");
      return ds_gemm_ks4_launch(a, d->a_major, d->b_major, batch, s);
    }
  }
  static const int tbm[3] = {128, 128, 64}, tbn[3] = {128, 64, 64};
  char tag[96];
  snprintf(tag, sizeof(tag), "%s<%s,%d,%d,%s,%s>", d->k % kt == 0 ? "gemm_dma_kernel" : "gemm_kernel",
           d->dtype == DS_BF16 ? "bf16" : "float", tbm[tile], tbn[tile],
           d->a_major == DS_K_MAJOR ? "K" : "MN", d->b_major == DS_K_MAJOR ? "K" : "MN");
  ds_prof_scope prof(s, tag, 2.0 * d->m * d->n * d->k * batch, "FLOP");
  if (d->dtype == DS_BF16) return launch_major<bf16>(a, batch, tile, d->a_major, d->b_major, s);
  return launch_major<float>(a, batch, tile, d->a_major, d->b_major, s);
}


extern "C" int ds_gemm(const ds_gemm_desc* d, void* stream) { return gemm_run(d, 1, stream); }

// ------------------------------------------------------------------------------------------
// ds_gemm for callers that cannot allocate (code under HIP graph capture, serving loops): the split-K workspace is
// this array instead of caller memory.  Every GPU the library runs on holds its own copy until the process ends.
namespace {
constexpr int SCRATCH_MAX_TILES = 16;  // 128x128 output tiles, e.g. 512 x 512 or 128 x 2048
constexpr size_t SCRATCH_BYTES = 4096 + (size_t)SCRATCH_MAX_TILES * 4 * 128 * 128 * sizeof(float);  // 4 MiB + 4 KiB
constexpr int SCRATCH_MAX_DEVICES = 64;
void* g_scratch_ptr[SCRATCH_MAX_DEVICES] = {};
}  // namespace
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

// Resolves the device address of the library's scratch on the current device (once per device; the array's name is only
// a host-side handle).  Launches nothing and allocates nothing: a file-scope device array is zero when its code object
// is loaded, and every split-K launch leaves the arrival counters at zero again.  A caller that is going to capture
// ds_gemm_static_scratch into a graph calls this first, outside the capture; otherwise the first call does it.
extern "C" int ds_gemm_static_scratch_init(void) {
  int dev = -1;
  DS_CHECK_HIP(hipGetDevice(&dev));
  DS_CHECK_ARG(dev >= 0 && dev < SCRATCH_MAX_DEVICES, "ds_gemm_static_scratch: device %d", dev);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    DS_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    g_scratch_ptr[dev] = ptr;
  }
  return DS_OK;
}

extern "C" int ds_gemm_static_scratch(const ds_gemm_desc* d, void* stream) {
  DS_CHECK_ARG(d != nullptr, "ds_gemm_static_scratch: null descriptor");
  DS_CHECK_ARG(d->m > 0 && d->n > 0, "ds_gemm_static_scratch: m, n must be positive (%d %d)", d->m, d->n);
  const int64_t tiles = (int64_t)((d->m + 127) / 128) * ((d->n + 127) / 128);
  DS_CHECK_ARG(tiles <= SCRATCH_MAX_TILES,
               "ds_gemm_static_scratch: a %d x %d output has %lld tiles of 128 x 128, the library's scratch holds %d (%zu bytes)",
               d->m, d->n, (long long)tiles, SCRATCH_MAX_TILES, SCRATCH_BYTES);
  DS_PROPAGATE(ds_gemm_static_scratch_init());
  int dev = -1;
  DS_CHECK_HIP(hipGetDevice(&dev));
  ds_gemm_desc c = *d;
  c.workspace = g_scratch_ptr[dev];
  c.workspace_bytes = SCRATCH_BYTES;
  return gemm_run(&c, 1, stream, true);
}

// 4 KiB of arrival counters (one per 128x128 tile, at most 1024 tiles), then up to 4 fp32 partial tiles per tile
extern "C" size_t ds_gemm_workspace_bytes(int m, int n) {
  if (m <= 0 || n <= 0) return 0;
  const size_t tiles = (size_t)((m + 127) / 128) * ((n + 127) / 128);
  return 4096 + tiles * 4 * 128 * 128 * sizeof(float);
}

// Split-K variant for accumulating outputs whose reduction dimension dwarfs m*n (atomic fp32 adds).
int ds_gemm_splitk(const ds_gemm_desc* d, int splitk, void* stream) { return gemm_run(d, splitk, stream); }

// ------------------------------------------------------------------------------------------
// 3x3 / stride 1 / 'same' convolution over NHWC tensors as an implicit GEMM (fp32 MFMA).
namespace {
template <int BM, int BN, int AMAJ, int MODE>
int launch_conv_cfg(GemmArgs a, hipStream_t stream) {
  a.grid_m = (a.m + BM - 1) / BM;
  a.grid_n = (a.n + BN - 1) / BN;
  choose_xcd_block(a);
  dim3 grid(a.grid_m * a.grid_n, 1, a.splitk);
  constexpr int STAGES = 4;
  constexpr size_t lds = (size_t)STAGES * (BM + BN) * 128;
  static std::atomic<bool> attr_set(false);  // two threads may both set the (idempotent) attribute; neither launches before it is set
  if (!attr_set) {
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)gemm_dma_kernel<float, BM, BN, AMAJ, DS_MN_MAJOR, STAGES, MODE>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  hipLaunchKernelGGL((gemm_dma_kernel<float, BM, BN, AMAJ, DS_MN_MAJOR, STAGES, MODE>), grid, dim3(256), lds, stream, a);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

int conv_check(const char* who, int dtype, int n, int h, int w, int cin, int cout) {
  DS_CHECK_ARG(dtype == DS_F32, "%s: only fp32 is built (dtype %d)", who, dtype);
  DS_CHECK_ARG(n > 0 && h > 0 && w > 0 && cin > 0 && cout > 0, "%s: non-positive shape", who);
  DS_CHECK_ARG(cin % 32 == 0, "%s: input channels (%d) must be a multiple of 32 (use ds_im2col3x3 + ds_gemm otherwise)", who, cin);
  DS_CHECK_ARG(cout % 4 == 0, "%s: output channels (%d) must be a multiple of 4", who, cout);
  DS_CHECK_ARG((int64_t)n * h * w < (int64_t)1 << 31, "%s: more than 2^31 pixels", who);
  return DS_OK;
}
}  // namespace

extern "C" int ds_conv3x3_fwd(int dtype, int n, int h, int w, int cin, int cout, const void* x, const void* kernel_hwio,
                              const float* bias, int flags, const void* mask_src, void* y, void* stream) {
  DS_PROPAGATE(conv_check("ds_conv3x3_fwd", dtype, n, h, w, cin, cout));
  DS_CHECK_ARG(x && kernel_hwio && y, "ds_conv3x3_fwd: null pointer");
  DS_CHECK_ARG((flags & ~(DS_EPI_BIAS | DS_EPI_RELU | DS_EPI_MASK)) == 0, "ds_conv3x3_fwd: unsupported flags %d", flags);
  if (flags & DS_EPI_BIAS) DS_CHECK_ARG(bias != nullptr, "ds_conv3x3_fwd: DS_EPI_BIAS without bias");
  if (flags & DS_EPI_MASK) DS_CHECK_ARG(mask_src != nullptr, "ds_conv3x3_fwd: DS_EPI_MASK without mask_src");
  DS_CHECK_ARG(ds_aligned16(x) && ds_aligned16(kernel_hwio) && ds_aligned16(y) && ds_aligned16(mask_src),
               "ds_conv3x3_fwd: tensors must be 16-byte aligned");
  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.a = (const char*)x; a.b = (const char*)kernel_hwio; a.c = (char*)y;
  a.bias = bias; a.c2 = (char*)mask_src;
  a.m = n * h * w; a.n = cout; a.k = 9 * cin;
  a.lda = cin; a.ldb = cout; a.ldc = cout;
  a.batch_inner = 1; a.flags = flags; a.alpha = 1.f; a.splitk = 1; a.ktiles_per_split = a.k / 32;
  a.vec_epi = cout % 8 == 0;
  a.conv_h = h; a.conv_w = w; a.conv_c = cin; a.prio = ds_launch_prio;
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, cout <= 64 ? "conv3x3_fwd<float,128,64>" : "conv3x3_fwd<float,128,128>", 2.0 * a.m * a.n * a.k, "FLOP");
  if (cout <= 64) return launch_conv_cfg<128, 64, DS_K_MAJOR, 1>(a, s);
  return launch_conv_cfg<128, 128, DS_K_MAJOR, 1>(a, s);
}

extern "C" int ds_conv3x3_wgrad(int dtype, int n, int h, int w, int cin, int cout, const void* x, const void* dz,
                                float* dkernel_hwio, void* stream) {
  DS_PROPAGATE(conv_check("ds_conv3x3_wgrad", dtype, n, h, w, cin, cout));
  DS_CHECK_ARG(x && dz && dkernel_hwio, "ds_conv3x3_wgrad: null pointer");
  DS_CHECK_ARG(ds_aligned16(x) && ds_aligned16(dz) && ds_aligned16(dkernel_hwio), "ds_conv3x3_wgrad: tensors must be 16-byte aligned");
  const int64_t pixels = (int64_t)n * h * w;
  DS_CHECK_ARG(pixels % 32 == 0, "ds_conv3x3_wgrad: n*h*w (%lld) must be a multiple of 32", (long long)pixels);
  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.a = (const char*)x; a.b = (const char*)dz; a.c = (char*)dkernel_hwio;
  a.m = 9 * cin; a.n = cout; a.k = (int)pixels;
  a.lda = cin; a.ldb = cout; a.ldc = cout;
  a.batch_inner = 1; a.flags = DS_EPI_ACCUM; a.alpha = 1.f;
  a.conv_h = h; a.conv_w = w; a.conv_c = cin; a.prio = ds_launch_prio;
  const int bn = cout <= 64 ? 64 : 128;
  const int tiles = ((a.m + 127) / 128) * ((a.n + bn - 1) / bn);
  const int ktiles = a.k / 32;
  int splitk = 1024 / tiles;  // the reduction runs over every pixel of the micro-batch: split it across the chip
  if (splitk > ktiles / 8) splitk = ktiles / 8;
  if (splitk < 1) splitk = 1;
  a.splitk = splitk;
  a.ktiles_per_split = (ktiles + splitk - 1) / splitk;
  a.vec_epi = splitk == 1 && cout % 8 == 0;
  hipStream_t s = (hipStream_t)stream;
  ds_prof_scope prof(s, cout <= 64 ? "conv3x3_wgrad<float,128,64>" : "conv3x3_wgrad<float,128,128>", 2.0 * a.m * a.n * a.k, "FLOP");
  if (cout <= 64) return launch_conv_cfg<128, 64, DS_MN_MAJOR, 2>(a, s);
  return launch_conv_cfg<128, 128, DS_MN_MAJOR, 2>(a, s);
}
