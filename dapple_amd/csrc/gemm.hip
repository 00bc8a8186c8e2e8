// MFMA GEMM for gfx950: C[m][n] (+)= alpha * sum_k A(m,k) * B(n,k), bf16 or fp32 operands,
// fp32 accumulation, either operand K-major or MN-major, optional two-level batch strides.
//
// Tiling: a 256-thread block (4 waves as 2x2) owns a BM x BN tile of C; each wave owns
// (BM/2) x (BN/2) as 32x32 MFMA tiles.  The reduction runs in k-tiles of 128 bytes per row
// (64 bf16 / 32 fp32).  Global -> registers -> LDS with two LDS stages and one barrier per
// k-tile; the next k-tile's global loads are in flight while the current one is multiplied.
//
// LDS layouts (both XOR-swizzled so that fragment reads and tile stores are conflict free):
//   K-major operand : [free row][128 B of k]; 16-byte chunk c of row r lives at chunk c ^ (r & 7).
//                     A lane reads its MFMA fragment as one 16-byte load.
//   MN-major operand: [k row][free index contiguous]; 32-byte granule g of row r lives at
//                     g ^ (((r & 3) << 1) & (granules-1)).  bf16 fragments come from
//                     ds_read_b64_tr_b16 (a 4x16 transpose per 16 lanes), fp32 from 4-byte loads.
#include "common.h"

namespace {

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
};

__device__ __forceinline__ int kmajor_off(int row, int chunk) { return row * 128 + ((chunk ^ (row & 7)) << 4); }
template <int ROW_BYTES> __device__ __forceinline__ int mnmajor_off(int r, int cbyte) {
  constexpr int NG = ROW_BYTES / 32;
  const int g = (cbyte >> 5) ^ (((r & 3) << 1) & (NG - 1));
  return r * ROW_BYTES + (g << 5) + (cbyte & 31);
}

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
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
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

  // epilogue: lane holds column (lane & 31), rows (e/4)*8 + (lane>>5)*4 + (e&3) of each 32x32 tile
  const int flags = p.flags;
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
        if (flags & DS_EPI_RESIDUAL) v += to_f32(R[idx]);
        if (flags & DS_EPI_DGELU) v *= gelu_erf_grad(to_f32(C2[idx]));
        if (flags & DS_EPI_RELU) v = fmaxf(v, 0.f);
        if (flags & DS_EPI_ACCUM) {
          if (p.splitk > 1) atomicAdd(Cf + idx, v); else Cf[idx] += v;
        } else if (out_f32) {
          Cf[idx] = v;
        } else {
          Ct[idx] = from_f32<T>(v);
        }
        if (flags & DS_EPI_GELU) C2[idx] = from_f32<T>(gelu_erf(v));
      }
    }
}

template <typename T, int BM, int BN, int AMAJ, int BMAJ>
int launch_cfg(const GemmArgs& a, int batch, hipStream_t stream) {
  dim3 grid((a.n + BN - 1) / BN, (a.m + BM - 1) / BM, batch * a.splitk);
  const size_t lds = 2 * (BM + BN) * 128;
  hipLaunchKernelGGL((gemm_kernel<T, BM, BN, AMAJ, BMAJ>), grid, dim3(256), lds, stream, a);
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

// Picks the tile shape (and split-K for accumulating outputs) that keeps the 256 CUs busiest.
static void choose_tiling(int m, int n, int k, int kt, int batch, bool can_split, int* tile, int* splitk) {
  static const int bm[3] = {128, 128, 64}, bn[3] = {128, 64, 64};
  static const double eff[3] = {1.0, 0.8, 0.55};
  const double slots = 512.0;  // 256 CUs x 2 resident blocks
  double best = 1e300;
  *tile = 0;
  *splitk = 1;
  const int ktiles = (k + kt - 1) / kt;
  for (int t = 0; t < 3; ++t) {
    const double blocks = (double)((m + bm[t] - 1) / bm[t]) * ((n + bn[t] - 1) / bn[t]) * batch;
    for (int s = 1; s <= (can_split ? 8 : 1); s *= 2) {
      if (s > ktiles) break;
      const double rounds = (double)((long long)((blocks * s + slots - 1) / slots));
      const double per_block = (double)bm[t] * bn[t] * ((ktiles + s - 1) / s) / eff[t] + 4.0 * bm[t] * bn[t] / 64;
      const double cost = rounds * per_block;
      if (cost < best) { best = cost; *tile = t; *splitk = s; }
    }
  }
}

extern "C" int ds_gemm(const ds_gemm_desc* d, void* stream) {
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
  if (f & (DS_EPI_GELU | DS_EPI_DGELU)) DS_CHECK_ARG(d->c2 != nullptr, "ds_gemm: GELU epilogue without c2");
  DS_CHECK_ARG(!((f & DS_EPI_GELU) && (f & DS_EPI_DGELU)), "ds_gemm: GELU and DGELU are exclusive");
  DS_CHECK_ARG(!((f & DS_EPI_ACCUM) && (f & (DS_EPI_GELU | DS_EPI_DGELU))), "ds_gemm: ACCUM with GELU");
  (void)esz;

  GemmArgs a;
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
  const int kt = d->dtype == DS_BF16 ? 64 : 32;
  int tile, splitk;
  choose_tiling(d->m, d->n, d->k, kt, batch, (f & DS_EPI_ACCUM) != 0, &tile, &splitk);
  const int ktiles = (d->k + kt - 1) / kt;
  a.splitk = splitk;
  a.ktiles_per_split = (ktiles + splitk - 1) / splitk;
  hipStream_t s = (hipStream_t)stream;
  if (d->dtype == DS_BF16) return launch_major<bf16>(a, batch, tile, d->a_major, d->b_major, s);
  return launch_major<float>(a, batch, tile, d->a_major, d->b_major, s);
}
