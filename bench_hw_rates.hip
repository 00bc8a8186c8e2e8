// Measured rates of the parts of a CU the GEMM kernels are built from (MI355X, gfx950): LDS read rate per instruction
// form, LDS-DMA (global_load_lds_dwordx4) rate under several address patterns, MFMA rate with 1 and 2 waves per SIMD and
// with one or all CUs busy, an MFMA wave beside a loader wave on one SIMD, and loads interleaved with MFMAs in one wave.
// A stand-alone program, not part of libdapple_hip.so:
//   hipcc -O3 -std=c++17 --offload-arch=gfx950 -Wno-inline-asm -Xclang -target-feature -Xclang -packed-fp32-ops bench_hw_rates.hip -o bench_hw_rates && ./bench_hw_rates
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
#define VMCNT(n) (((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1); } } while (0)
#define MFMA32(c, a, b) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b))
#define MFMA16(c, a, b) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b))
#define LOAD(m0v, off, base) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(m0v), "v"(off), "s"(base) : "memory")

static hipEvent_t e0, e1;
template <typename F> float time_us(F f, int reps = 3) {
  f(); f();
  CK(hipEventRecord(e0));
  for (int i = 0; i < reps; ++i) f();
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  return ms * 1e3f / reps;
}

// ---------------- A: LDS read rate
template <int MODE>  // 0: ds_read_b128, 1: ds_read_b64, 2: ds_read_b64_tr_b16
__global__ __launch_bounds__(512) void lds_read_k(float* out, int iters) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 65536 / 4; i += blockDim.x) ((float*)lds)[i] = (float)i;
  __syncthreads();
  const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  unsigned a = lds0 + (MODE == 0 ? lane * 16 : lane * 8) + (tid >> 6) * 1024;
  f32x4 r[8];
  float acc = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (MODE == 0) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r[j]) : "v"(a), "n"(j * 4096));
      else if (MODE == 1) asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(*(double*)&r[j]) : "v"(a), "n"(j * 4096));
      else asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(*(double*)&r[j]) : "v"(a), "n"(j * 4096));
    }
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
    acc += r[0][0] + r[7][1];
  }
  if (acc == 12345.f) out[blockIdx.x * blockDim.x + tid] = acc;
}

// ---------------- B: LDS-DMA rate.  Every wave issues `per` loads of 1 KiB per tile into a ring of 2 tiles.
// PAT 0: block-private contiguous stream (HBM);  1: all blocks the same 2 MB window, contiguous (L2 hits)
// PAT 2: K-major GEMM operand tile, row stride RS bytes, 128 B per row per k-tile, rows (block % 8) * ROWS.., shared window
// PAT 3: as 2, the k-tile sequence rotated by the block id
template <int PAT, int NW>
__global__ __launch_bounds__(NW * 64) void dma_k(const char* __restrict__ src, float* out, int ntiles, int RS, int kt_total) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int PER = 32 / NW;  // 32 KiB per tile and block
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const char* base = src;
  if (PAT == 0) base += (size_t)blockIdx.x * ((size_t)ntiles * 32768);
  unsigned voff[PER];
  for (int l = 0; l < PER; ++l) {
    const int p = (l * NW + wave) * 64 + lane;  // 16-byte slot in the tile
    if (PAT <= 1) voff[l] = p * 16;
    else voff[l] = ((blockIdx.x & 7) * 256 + (p >> 3)) * RS + (p & 7) * 16;
  }
  const unsigned long long b0 = (unsigned long long)base;
  for (int t = 0; t < ntiles; ++t) {
    unsigned long long tb;
    if (PAT == 0) tb = b0 + (size_t)t * 32768;
    else if (PAT == 1) tb = b0 + (size_t)(t & 63) * 32768;
    else if (PAT == 2) tb = b0 + (size_t)(t % kt_total) * 128;
    else tb = b0 + (size_t)((t + blockIdx.x * 5) % kt_total) * 128;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)tb), hi = __builtin_amdgcn_readfirstlane((unsigned)(tb >> 32));
    const unsigned long long tbs = ((unsigned long long)hi << 32) | lo;
#pragma unroll
    for (int l = 0; l < PER; ++l) {
      const unsigned m0v = lds0 + (t & 1) * 32768 + (l * NW + wave) * 1024;
      LOAD(m0v, voff[l], tbs);
    }
    __builtin_amdgcn_s_waitcnt(VMCNT(PER));  // the previous tile has landed
  }
  __builtin_amdgcn_s_waitcnt(VMCNT(0));
  __syncthreads();
  if (((float*)lds)[tid] == 12345.f) out[blockIdx.x * blockDim.x + tid] = 1.f;
}

// ---------------- C/D: MFMA rate and MFMA wave beside loader wave
// waves [0, mw) run `nm` groups of 4 MFMAs each; waves [mw, mw+lw) run `nl` groups of 4 loads (1 KiB each) from an L2 window
template <int KIND>  // 0: 32x32x16, 1: 16x16x32
__global__ __launch_bounds__(512) void mix_k(const char* __restrict__ src, float* out, int mw, int nm, int nl) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  if (wave < mw) {
    f32x16 acc[4] = {};
    f32x4 acc4[4] = {};
    bf16x8 a, b;
    for (int j = 0; j < 8; ++j) { a[j] = (__bf16)(float)((lane + j) % 5 - 2); b[j] = (__bf16)(float)((lane * 3 + j) % 7 - 3); }
    for (int i = 0; i < nm; ++i) {
      if (KIND == 0) { MFMA32(acc[0], a, b); MFMA32(acc[1], a, b); MFMA32(acc[2], a, b); MFMA32(acc[3], a, b); }
      else {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc4[0]) : "v"(a), "v"(b));
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc4[1]) : "v"(a), "v"(b));
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc4[2]) : "v"(a), "v"(b));
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc4[3]) : "v"(a), "v"(b));
      }
    }
    float s = 0;
    for (int q = 0; q < 4; ++q) { for (int e = 0; e < 16; ++e) s += acc[q][e]; for (int e = 0; e < 4; ++e) s += acc4[q][e]; }
    if (s == 12345.f) out[blockIdx.x * 512 + tid] = s;
  } else {
    const int lwv = wave - mw;
    const unsigned long long b0 = (unsigned long long)src;
    for (int i = 0; i < nl; ++i) {
      const unsigned long long tb = b0 + (size_t)((i * 4 + lwv) & 255) * 8192;
      const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)tb), hi = __builtin_amdgcn_readfirstlane((unsigned)(tb >> 32));
      const unsigned long long tbs = ((unsigned long long)hi << 32) | lo;
#pragma unroll
      for (int l = 0; l < 4; ++l) {
        const unsigned m0v = lds0 + ((i & 1) * 16 + lwv * 4 + l) * 1024;
        LOAD(m0v, (unsigned)(l * 1024 + lane * 16), tbs);
      }
      __builtin_amdgcn_s_waitcnt(VMCNT(4));
    }
    __builtin_amdgcn_s_waitcnt(VMCNT(0));
  }
}

// MFMAs and loads alternating inside every wave: per group 4 MFMAs + `lp4` loads (0..4)
__global__ __launch_bounds__(512) void inter_k(const char* __restrict__ src, float* out, int nm, int lp4) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  f32x16 acc[4] = {};
  bf16x8 a, b;
  for (int j = 0; j < 8; ++j) { a[j] = (__bf16)(float)((lane + j) % 5 - 2); b[j] = (__bf16)(float)((lane * 3 + j) % 7 - 3); }
  const unsigned long long b0 = (unsigned long long)src;
  for (int i = 0; i < nm; ++i) {
    const unsigned long long tb = b0 + (size_t)((i * 8 + wave) & 255) * 8192;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)tb), hi = __builtin_amdgcn_readfirstlane((unsigned)(tb >> 32));
    const unsigned long long tbs = ((unsigned long long)hi << 32) | lo;
    const unsigned m0v = lds0 + ((i & 1) * 32 + wave * 4) * 1024;
    MFMA32(acc[0], a, b); if (lp4 > 0) LOAD(m0v, (unsigned)(lane * 16), tbs);
    MFMA32(acc[1], a, b); if (lp4 > 1) LOAD(m0v + 1024, (unsigned)(1024 + lane * 16), tbs);
    MFMA32(acc[2], a, b); if (lp4 > 2) LOAD(m0v + 2048, (unsigned)(2048 + lane * 16), tbs);
    MFMA32(acc[3], a, b); if (lp4 > 3) LOAD(m0v + 3072, (unsigned)(3072 + lane * 16), tbs);
    __builtin_amdgcn_s_waitcnt(VMCNT(4));
  }
  __builtin_amdgcn_s_waitcnt(VMCNT(0));
  float s = 0;
  for (int q = 0; q < 4; ++q) for (int e = 0; e < 16; ++e) s += acc[q][e];
  if (s == 12345.f) out[blockIdx.x * 512 + tid] = s;
}

int main() {
  CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  char* src; float* out;
  const size_t SRC = (size_t)1 << 30;
  CK(hipMalloc(&src, SRC)); CK(hipMemset(src, 0, SRC));
  CK(hipMalloc(&out, 1 << 24));
  hipDeviceProp_t prop; CK(hipGetDeviceProperties(&prop, 0));
  printf("device %s CUs %d clock %d kHz\n", prop.name, prop.multiProcessorCount, prop.clockRate);

  printf("== A: LDS read rate (bytes per CU per ns; x/2.4 = bytes per clock at 2.4 GHz)\n");
  {
    const int iters = 2000;
#define RUNA(MODE, name, bytes_per_lane) \
    for (int nw : {4, 8}) for (int blocks : {1, 256}) { \
      CK(hipFuncSetAttribute((const void*)lds_read_k<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072)); \
      float us = time_us([&] { hipLaunchKernelGGL(lds_read_k<MODE>, dim3(blocks), dim3(nw * 64), 131072, 0, out, iters); }); \
      double bytes = (double)iters * 8 * nw * 64 * bytes_per_lane; \
      printf("%-22s waves %d blocks %3d  %8.1f us  %7.1f B/ns/CU = %6.1f B/clk@2.4\n", name, nw, blocks, us, bytes / us / 1e3, bytes / us / 1e3 / 2.4); }
    RUNA(0, "ds_read_b128", 16)
    RUNA(1, "ds_read_b64", 8)
    RUNA(2, "ds_read_b64_tr_b16", 8)
  }

  printf("== B: LDS-DMA (global_load_lds_dwordx4) rate, 32 KiB tiles\n");
  {
#define RUNB(PAT, NW, name, blocks, ntiles, RS, ktt) { \
      CK(hipFuncSetAttribute((const void*)dma_k<PAT, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536)); \
      float us = time_us([&] { hipLaunchKernelGGL((dma_k<PAT, NW>), dim3(blocks), dim3(NW * 64), 65536, 0, src, out, ntiles, RS, ktt); }); \
      double bytes = (double)ntiles * 32768 * blocks; \
      printf("%-44s waves %d blocks %3d  %8.1f us  %7.2f TB/s total  %6.1f GB/s per block\n", name, NW, blocks, us, bytes / us / 1e6, bytes / us / 1e3 / blocks); }
    RUNB(0, 4, "private contiguous stream (HBM)", 256, 120, 0, 1)
    RUNB(0, 8, "private contiguous stream (HBM)", 256, 120, 0, 1)
    RUNB(1, 4, "shared 2 MB window contiguous (L2)", 1, 2000, 0, 1)
    RUNB(1, 8, "shared 2 MB window contiguous (L2)", 1, 2000, 0, 1)
    RUNB(1, 4, "shared 2 MB window contiguous (L2)", 256, 2000, 0, 1)
    RUNB(1, 8, "shared 2 MB window contiguous (L2)", 256, 2000, 0, 1)
    RUNB(1, 4, "shared 2 MB window contiguous (L2)", 512, 2000, 0, 1)
    RUNB(2, 4, "K-major rows stride 8 KB, 64 k-tiles", 256, 2048, 8192, 64)
    RUNB(3, 4, "K-major rows stride 8 KB, rotated k", 256, 2048, 8192, 64)
    RUNB(2, 4, "K-major rows stride 2 KB, 16 k-tiles", 256, 2048, 2048, 16)
    RUNB(3, 4, "K-major rows stride 2 KB, rotated k", 256, 2048, 2048, 16)
    RUNB(2, 4, "K-major rows stride 8320 B, 64 k-tiles", 256, 2048, 8320, 64)
    RUNB(2, 8, "K-major rows stride 8 KB, 64 k-tiles", 256, 2048, 8192, 64)
    RUNB(3, 8, "K-major rows stride 8 KB, rotated k", 256, 2048, 8192, 64)
  }

  printf("== D: MFMA rate (TFLOP/s per CU; peak 9.8 at 2.4 GHz)\n");
  {
    CK(hipFuncSetAttribute((const void*)mix_k<0>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    CK(hipFuncSetAttribute((const void*)mix_k<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    const int nm = 4000;
    for (int mw : {4, 8}) for (int blocks : {1, 256}) {
      float us = time_us([&] { hipLaunchKernelGGL(mix_k<0>, dim3(blocks), dim3(mw * 64), 131072, 0, src, out, mw, nm, 0); });
      printf("32x32x16 waves %d blocks %3d  %8.1f us  %6.2f TFLOP/s per CU\n", mw, blocks, us, (double)nm * 4 * mw * 32768.0 / us / 1e6);
      us = time_us([&] { hipLaunchKernelGGL(mix_k<1>, dim3(blocks), dim3(mw * 64), 131072, 0, src, out, mw, nm, 0); });
      printf("16x16x32 waves %d blocks %3d  %8.1f us  %6.2f TFLOP/s per CU\n", mw, blocks, us, (double)nm * 4 * mw * 16384.0 / us / 1e6);
    }
  }
  printf("== C: 4 MFMA waves beside 4 loader waves (one of each per SIMD), 1 KiB loads from an L2 window\n");
  {
    const int nm = 4000;
    for (int blocks : {1, 256}) for (int nl : {500, 1000, 2000}) {
      float tm = time_us([&] { hipLaunchKernelGGL(mix_k<0>, dim3(blocks), dim3(512), 131072, 0, src, out, 4, nm, 0); });
      float tl = time_us([&] { hipLaunchKernelGGL(mix_k<0>, dim3(blocks), dim3(512), 131072, 0, src, out, 4, 0, nl); });
      float tb = time_us([&] { hipLaunchKernelGGL(mix_k<0>, dim3(blocks), dim3(512), 131072, 0, src, out, 4, nm, nl); });
      printf("blocks %3d  mfma %d groups: %7.1f us | loads %d groups: %7.1f us (%5.1f GB/s per CU) | both: %7.1f us\n", blocks, nm, tm, nl, tl,
             (double)nl * 16 * 1024 / tl / 1e3, tb);
    }
    CK(hipFuncSetAttribute((const void*)inter_k, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    for (int nwv : {4, 8}) for (int blocks : {1, 256}) for (int lp4 = 0; lp4 <= 4; ++lp4) {
      float t = time_us([&] { hipLaunchKernelGGL(inter_k, dim3(blocks), dim3(nwv * 64), 131072, 0, src, out, nm, lp4); });
      printf("interleaved waves %d blocks %3d loads per 4 MFMA %d: %7.1f us  %6.2f TFLOP/s per CU  %6.1f GB/s per CU\n", nwv, blocks, lp4, t,
             (double)nm * 4 * nwv * 32768.0 / t / 1e6, (double)nm * lp4 * nwv * 1024.0 / t / 1e3);
    }
  }
  return 0;
}
