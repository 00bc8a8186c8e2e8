// bf16 MFMA GEMM with 512-thread blocks (8 waves, two per SIMD) for gfx950: C[m][n] (+)= alpha * sum_k A(m,k) B(n,k).
//
// Why a second kernel family beside the 4-wave blocks of gemm.hip: with one wave per SIMD every wait of that wave
// (a fragment read, the k-tile barrier) idles the SIMD's matrix pipe, and a 64x64 wave tile reads 4 KB of fragments
// from LDS per 4 MFMAs while the tile loads write the same LDS.  Here a SIMD holds two waves (one runs MFMAs while
// the other waits), and the block shapes keep LDS and vector-memory traffic per MFMA low:
//   cfg 0: 256x256 block, waves 2(m) x 4(n), 128x64 per wave, 2 tile buffers (128 KB)
//   cfg 1: 256x128 block, waves 2 x 2 x 2(k), 128x64 per wave pair, 3 tile buffers (144 KB)
//   cfg 2: 128x128 block, waves 2 x 2 x 2(k),  64x64 per wave pair, 4 tile buffers (128 KB; cfg 3 / 4: 2 / 3 buffers)
//   cfg 5: 128x64  block, waves 2 x 2 x 2(k),  64x32 per wave pair, 4 tile buffers (96 KB)
// In the 2 x 2 x 2 shapes the two waves of a SIMD own the same output sub-tile and split the four 16-deep k-steps of
// every 64-deep k-tile between them (each fragment is still read from LDS once); their partial sums meet in LDS in
// the epilogue.  Tiles move global -> LDS by LDS-DMA, one barrier per k-tile, fragments one k-step ahead of the
// MFMAs in two register sets; layouts, swizzles and the asm discipline are those of gemm_core.h.
#include "gemm8_core.h"

using namespace dsgemm;

namespace {

template <int BM, int BN, int WM, int WN, int WK, int STAGES, int AMAJ, int BMAJ>
__global__ __launch_bounds__(512) void gemm8_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  ds_wave_prio(p.prio);
  gemm8_tile<BM, BN, WM, WN, WK, STAGES, AMAJ, BMAJ>(p, lds, blockIdx.x, blockIdx.z);
}

template <int BM, int BN, int WM, int WN, int WK, int STAGES, int AMAJ, int BMAJ>
int launch8(GemmArgs a, int batch, hipStream_t stream) {
  a.grid_m = (a.m + BM - 1) / BM;
  a.grid_n = (a.n + BN - 1) / BN;
  choose_xcd_block(a);
  dim3 grid(a.grid_m * a.grid_n, 1, batch * a.splitk);
  if (a.ws_part != nullptr) {
    // every k-slice of every tile parks BM x BN floats at ws_part[(tile * splitk + slice) * BM * BN]; the counters (one
    // unsigned per tile) sit in the 4096 bytes in front of ws_part
    const size_t need = (size_t)a.grid_m * a.grid_n * a.splitk * BM * BN * sizeof(float);
    DS_CHECK_ARG((size_t)a.grid_m * a.grid_n * sizeof(unsigned) <= 4096 && need <= a.ws_bytes,
                 "ds_gemm8_launch: %d x %d tiles in %d slices need %zu bytes of workspace behind the counters, the caller's holds %zu",
                 a.grid_m, a.grid_n, a.splitk, need, a.ws_bytes);
  }
  constexpr size_t lds = (size_t)STAGES * (BM + BN) * 128;
  static std::atomic<bool> attr_set(false);  // two threads may both set the (idempotent) attribute; neither launches before it is set
  if (!attr_set) {
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)gemm8_kernel<BM, BN, WM, WN, WK, STAGES, AMAJ, BMAJ>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  hipLaunchKernelGGL((gemm8_kernel<BM, BN, WM, WN, WK, STAGES, AMAJ, BMAJ>), grid, dim3(512), lds, stream, a);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

// The 64x64 block of four waves that split the k-steps of every k-tile (gemm8_core.h): 48 KB of LDS like the 4-wave
// kernel of gemm.hip, half its fragment reads.
template <int AMAJ, int BMAJ>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4))) void gemm_ks4_kernel(GemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  ds_wave_prio(p.prio);
  gemm8_tile<64, 64, 1, 1, 4, 3, AMAJ, BMAJ>(p, lds, blockIdx.x, blockIdx.z);
}

template <int AMAJ, int BMAJ>
int launch_ks4(GemmArgs a, int batch, hipStream_t stream) {
  a.grid_m = (a.m + 63) / 64;
  a.grid_n = (a.n + 63) / 64;
  choose_xcd_block(a);
  dim3 grid(a.grid_m * a.grid_n, 1, batch);
  constexpr size_t lds = (size_t)3 * (64 + 64) * 128;
  static std::atomic<bool> attr_set(false);  // two threads may both set the (idempotent) attribute; neither launches before it is set
  if (!attr_set) {
    DS_CHECK_HIP(hipFuncSetAttribute((const void*)gemm_ks4_kernel<AMAJ, BMAJ>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  hipLaunchKernelGGL((gemm_ks4_kernel<AMAJ, BMAJ>), grid, dim3(256), lds, stream, a);
  DS_CHECK_LAUNCH();
  return DS_OK;
}

template <int AMAJ, int BMAJ>
int launch8_cfg(const GemmArgs& a, int cfg, int batch, hipStream_t stream) {
  switch (cfg) {
    case 0: return launch8<256, 256, 2, 4, 1, 2, AMAJ, BMAJ>(a, batch, stream);
    case 1: return launch8<256, 128, 2, 2, 2, 3, AMAJ, BMAJ>(a, batch, stream);
    case 3: return launch8<128, 128, 2, 2, 2, 2, AMAJ, BMAJ>(a, batch, stream);
    case 4: return launch8<128, 128, 2, 2, 2, 3, AMAJ, BMAJ>(a, batch, stream);
    case 5: return launch8<128, 64, 2, 2, 2, 4, AMAJ, BMAJ>(a, batch, stream);
    default: return launch8<128, 128, 2, 2, 2, 4, AMAJ, BMAJ>(a, batch, stream);
  }
}

}  // namespace

int ds_gemm8_stages(int cfg) { return cfg == 0 || cfg == 3 ? 2 : cfg == 1 || cfg == 4 ? 3 : 4; }  // cfg 2 and 5: 4

int ds_gemm8_launch(const GemmArgs& a, int cfg, int a_major, int b_major, int batch, hipStream_t stream) {
  DS_CHECK_ARG(a.k % 64 == 0 && a.vec_epi, "ds_gemm8_launch: needs k %% 64 == 0 and the vector epilogue");
  DS_CHECK_ARG(cfg >= 0 && cfg <= 5, "ds_gemm8_launch: cfg %d", cfg);
  DS_CHECK_ARG(a.splitk == 1 || (a.ws_part && a.ws_count && batch == 1 && a.splitk <= 4),
               "ds_gemm8_launch: split-K needs a workspace, batch 1 and at most 4 slices");
  DS_CHECK_ARG(a.ktiles_per_split > ds_gemm8_stages(cfg) && (a.k / 64) % a.ktiles_per_split == 0,
               "ds_gemm8_launch: every k-slice needs more than %d k-tiles", ds_gemm8_stages(cfg));
  if (a_major == DS_K_MAJOR && b_major == DS_K_MAJOR) return launch8_cfg<DS_K_MAJOR, DS_K_MAJOR>(a, cfg, batch, stream);
  if (a_major == DS_K_MAJOR && b_major == DS_MN_MAJOR) return launch8_cfg<DS_K_MAJOR, DS_MN_MAJOR>(a, cfg, batch, stream);
  if (a_major == DS_MN_MAJOR && b_major == DS_MN_MAJOR) return launch8_cfg<DS_MN_MAJOR, DS_MN_MAJOR>(a, cfg, batch, stream);
  return launch8_cfg<DS_MN_MAJOR, DS_K_MAJOR>(a, cfg, batch, stream);
}

int ds_gemm_ks4_launch(const GemmArgs& a, int a_major, int b_major, int batch, hipStream_t stream) {
  const int nkt = a.k / 64;
  DS_CHECK_ARG(a.k % 64 == 0 && a.vec_epi && a.splitk == 1 && a.ws_part == nullptr && nkt >= 4 && nkt % 2 == 0 && a.ktiles_per_split == nkt,
               "ds_gemm_ks4_launch: needs the vector epilogue, no k-slices and an even number (at least 4) of 64-deep k-tiles");
  if (a_major == DS_K_MAJOR && b_major == DS_K_MAJOR) return launch_ks4<DS_K_MAJOR, DS_K_MAJOR>(a, batch, stream);
  if (a_major == DS_K_MAJOR && b_major == DS_MN_MAJOR) return launch_ks4<DS_K_MAJOR, DS_MN_MAJOR>(a, batch, stream);
  if (a_major == DS_MN_MAJOR && b_major == DS_MN_MAJOR) return launch_ks4<DS_MN_MAJOR, DS_MN_MAJOR>(a, batch, stream);
  return launch_ks4<DS_MN_MAJOR, DS_K_MAJOR>(a, batch, stream);
}
