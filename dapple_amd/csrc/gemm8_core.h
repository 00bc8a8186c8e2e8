// The 8-wave bf16 GEMM tile of gemm8.hip as a device function, so that a kernel of its own (gemm8.hip) and the
// kernels that carry several problems per launch (group.hip) run the same code.
#pragma once
#include "gemm_core.h"

namespace dsgemm {


// Split-K partials cross from one workgroup to another inside a launch, and the L2 caches of the 8 XCDs are not
// coherent with each other: the values move as system-scope 16-byte accesses (sc0 sc1: stores go through to memory,
// loads come from there), which leaves the rest of the cache alone - a release / acquire fence pair at device scope
// would write back and invalidate the whole L2 (measured: 60 us per GEMM).
__device__ __forceinline__ void part_store4(float* p, const f32x4& v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void part_load4(const float* p, f32x4& v) {
  asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=v"(v) : "v"(p) : "memory");
}

// One output tile of C by one workgroup of WM x WN x WK waves (512 threads; 256 in the 1 x 1 x 4 shape).  `lds` is the
// workgroup's dynamic LDS (STAGES * (BM + BN) * 128 bytes), bx the workgroup's index among the tiles of the problem (what a
// launch of its own passes as blockIdx.x), bz its index among batch entries x k-slices (blockIdx.z).  All threads must enter.
// The 1 x 1 x 4 shape (a 64x64 block of four waves, 3 tile buffers = the 48 KB of the 4-wave kernel of gemm.hip): every
// wave multiplies the WHOLE 64x64 tile over one of the four 16-deep k-steps of each k-tile, so a fragment is read from LDS
// once per block instead of twice (16 KB of fragment reads per k-tile instead of 32 - with the 16 KB the tile loads write,
// the LDS port is what bounds that block); the four partial tiles meet in LDS at the end, every wave summing one 32x32
// quadrant.  Its k-tile has a single k-step, so the two fragment register sets alternate from k-tile to k-tile (PAR below)
// and the number of k-tiles must be even.
// COLSUM: the workgroups of the first tile row also sum the B operand over k (GemmArgs::colsum) - one more MFMA per B
// fragment with an A operand of ones, by the waves that hold the tile's first rows: all 32 rows of the result are the
// column sums of the 16 x 32 fragment.
template <int BM, int BN, int WM, int WN, int WK, int STAGES, int AMAJ, int BMAJ, bool COLSUM = false>
__device__ __forceinline__ void gemm8_tile(const GemmArgs& p, char* lds, int bx, int bz) {
  typedef bf16 T;
  constexpr int NW = WM * WN * WK;                     // waves of the workgroup
  typedef AsmDma<T, BM, AMAJ, NW> DA;
  typedef AsmDma<T, BN, BMAJ, NW> DB;
  constexpr int KT = 64;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;  // 32x32 MFMA tiles per wave
  constexpr int KS = 4 / WK;                           // k-steps of a k-tile that one wave multiplies
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int LPT = DA::NV + DB::NV;                 // DMA loads per thread and k-tile
  constexpr int NSLOT = TM * TN;                       // MFMAs per k-step
  constexpr int NMMA = KS * NSLOT;                     // MFMAs per k-tile and wave
  constexpr int NFR = TM + TN;                         // fragments per k-step
  static_assert((NW == 8 && (WK == 1 || WK == 2)) || (NW == 4 && WK == 4 && TM == 2 && TN == 2 && STAGES == 3),
                "8 waves, or the 64x64 block of four k-step waves");
  static_assert((STAGES - 2) * LPT <= 63, "vmcnt range");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // waves w and w + 4 share a SIMD: with WK == 2 they are the two k-halves of one output sub-tile
  const int wq = wave % (WM * WN), wk = wave / (WM * WN);
  const int wm = wq / WN, wn = wq % WN;
  int tile_m, tile_n;
  xcd_tile(p, bx, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int z = bz / p.splitk, ks_id = bz % p.splitk;
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

  static_assert(!COLSUM || (WK == 2 && NW == 8), "column sums: the 2 x 2 x 2 shapes");
  const bool cs_wave = COLSUM && tile_m == 0 && wm == 0;   // wave-uniform
  f32x16 cs[COLSUM ? TN : 1];
  bf16x8 ones;
  if (COLSUM) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) cs[j][e] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (bf16)1.0f;
  }

  DA da;
  DB db;
  da.init(p, A, p.lda, m0, p.m, kt_begin, wave, lane, p.a_seg);
  db.init(p, B, p.ldb, n0, p.n, kt_begin, wave, lane, p.b_seg);
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t lds0 = lds_addr(lds);
#pragma unroll
  for (int s = 0; s < STAGES; ++s) {
    if (s < nkt) {
      da.issue(lds0 + s * STAGE_BYTES, wave_s);
      db.issue(lds0 + s * STAGE_BYTES + A_BYTES, wave_s);
    }
  }
  FragReader<T, BM, AMAJ, TM> ra;
  FragReader<T, BN, BMAJ, TN> rb;
  // local k-step 0 is k-step wk * KS of the k-tile
  ra.init(wm * (BM / WM), lane, wk * KS);
  rb.init(wn * (BN / WN), lane, wk * KS);
  RawFrag<T, AMAJ> fa[2][TM];
  RawFrag<T, BMAJ> fb[2][TN];
  {
    // tile 0 has landed once only the tiles issued after it are outstanding
    const int later = (nkt < STAGES ? nkt : STAGES) - 1;
    if (later >= 3) __builtin_amdgcn_s_waitcnt(DS_VMCNT(LPT * 3));
    else if (later == 2) __builtin_amdgcn_s_waitcnt(DS_VMCNT(LPT * 2));
    else if (later == 1) __builtin_amdgcn_s_waitcnt(DS_VMCNT(LPT));
    else __builtin_amdgcn_s_waitcnt(DS_VMCNT(0));
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < TM; ++i) ra.read(fa[0][i], lds0, i, 0);
#pragma unroll
    for (int j = 0; j < TN; ++j) rb.read(fb[0][j], lds0 + A_BYTES, j, 0);
#pragma unroll
    for (int i = 0; i < TM; ++i) lds_wait(fa[0][i]);
#pragma unroll
    for (int j = 0; j < TN; ++j) lds_wait(fb[0][j]);
  }
  int buf = 0;  // kt % STAGES
  // One k-tile.  On entry the fragments of this wave's first k-step are in register set 0.  Under the first MFMA of
  // the last k-step every wave has finished reading tile kt (its reads are waited for), waits for its own loads of
  // tile kt+1 and meets the others at the one barrier of the k-tile; after it tile kt+1 is visible (its first
  // fragments are fetched under the remaining MFMAs) and buffer kt % STAGES is free: the loads of tile kt+STAGES go
  // there, one at a time between the next NMMA MFMAs (the rest of this k-step, then the first KS-1 k-steps of tile
  // kt+1).  All three parameters are compile-time so that a k-tile is one straight run of code: RP / RC say whether
  // tile kt-1+STAGES / kt+STAGES exist (their loads are issued in this k-tile), LATER is the number of tiles issued
  // after tile kt+1 that may still be in flight at the barrier.  No LDS read is in flight at the end (the compiler may
  // copy fragment registers where control flow joins; a copy taken before the data has landed would be stale).
  auto k_tile = [&](auto rp, auto rc, auto later, auto par) {
    constexpr bool RP = decltype(rp)::value, RC = decltype(rc)::value;
    constexpr int LATER = decltype(later)::value;
    constexpr int PAR = decltype(par)::value;   // register set that holds this k-tile's first fragments
    const uint32_t sa = lds0 + buf * STAGE_BYTES, sb = sa + A_BYTES;
    int pb = buf - 1;
    if (pb < 0) pb += STAGES;
    int nbuf = buf + 1;
    if (nbuf == STAGES) nbuf = 0;
    const uint32_t prev_tile = lds0 + pb * STAGE_BYTES, next_tile = lds0 + nbuf * STAGE_BYTES;
#pragma unroll
    for (int ksl = 0; ksl < KS; ++ksl) {
      const int cur = (ksl + PAR) & 1, nxt = cur ^ 1;
      const bool last = ksl == KS - 1;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int slot = i * TN + j;
          Mma<T>::mma(acc[i][j], to_frag(fa[cur][i]), to_frag(fb[cur][j]));
          if (COLSUM && i == 0) {
            if (cs_wave) Mma<T>::mma(cs[COLSUM ? j : 0], ones, to_frag(fb[cur][j]));
          }
          __builtin_amdgcn_sched_barrier(0);
          if (last && slot == 0) {
            __builtin_amdgcn_s_waitcnt(DS_VMCNT(LPT * LATER));
            __builtin_amdgcn_s_barrier();
          }
          // this slot's share of the next k-step's fragment reads (after the last tile: a stale buffer, unused)
#pragma unroll
          for (int r = 0; r < NFR; ++r)
            if (r / 2 == slot) {
              const uint32_t ta = last ? next_tile : sa;
              const int ks = last ? 0 : ksl + 1;
              if (r < TM) ra.read(fa[nxt][r], ta, r, ks);
              else rb.read(fb[nxt][r - TM], ta + A_BYTES, r - TM, ks);
            }
          // this slot's share of the refill loads
          if (!last && RP) {
            const int q = NSLOT + ksl * NSLOT + slot;
#pragma unroll
            for (int l = 0; l < LPT; ++l)
              if ((l * NMMA) / LPT == q) {
                if (l < DA::NV) da.issue_one(prev_tile, wave_s, l);
                else db.issue_one(prev_tile + A_BYTES, wave_s, l - DA::NV);
              }
          }
          if (last && RC) {
#pragma unroll
            for (int l = 0; l < LPT; ++l)
              if ((l * NMMA) / LPT == slot) {
                if (l < DA::NV) da.issue_one(sa, wave_s, l);
                else db.issue_one(sb, wave_s, l - DA::NV);
              }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      if ((KS > 1 && ksl == KS - 2 && RP) || (KS == 1 && RC)) { da.advance(); db.advance(); }
#pragma unroll
      for (int i = 0; i < TM; ++i) lds_wait(fa[nxt][i]);
#pragma unroll
      for (int j = 0; j < TN; ++j) lds_wait(fb[nxt][j]);
    }
    buf = nbuf;
  };
  // nkt > STAGES (checked on the host): head tile, steady loop, then the last STAGES tiles with compile-time counts
  typedef std::true_type Y;
  typedef std::false_type N;
  typedef std::integral_constant<int, 0> P0;
  typedef std::integral_constant<int, 1> P1;
  if constexpr (KS % 2 == 0) {
    k_tile(N(), Y(), std::integral_constant<int, STAGES - 2>(), P0());
    for (int kt = 1; kt + STAGES < nkt; ++kt) k_tile(Y(), Y(), std::integral_constant<int, STAGES - 2>(), P0());
    k_tile(Y(), N(), std::integral_constant<int, STAGES - 2>(), P0());
    if (STAGES >= 3) k_tile(N(), N(), std::integral_constant<int, (STAGES >= 3 ? STAGES - 3 : 0)>(), P0());
    if (STAGES >= 4) k_tile(N(), N(), std::integral_constant<int, (STAGES >= 4 ? STAGES - 4 : 0)>(), P0());
    k_tile(N(), N(), std::integral_constant<int, 0>(), P0());
  } else {
    // one k-step per k-tile: the register sets alternate; nkt is even (checked on the host) and STAGES is 3, so the steady
    // loop runs an even number of times and the last three tiles start from sets 1, 0, 1
    k_tile(N(), Y(), std::integral_constant<int, STAGES - 2>(), P0());
    for (int kt = 1; kt + STAGES < nkt; kt += 2) {
      k_tile(Y(), Y(), std::integral_constant<int, STAGES - 2>(), P1());
      k_tile(Y(), Y(), std::integral_constant<int, STAGES - 2>(), P0());
    }
    k_tile(Y(), N(), std::integral_constant<int, STAGES - 2>(), P1());
    k_tile(N(), N(), std::integral_constant<int, (STAGES >= 3 ? STAGES - 3 : 0)>(), P0());
    k_tile(N(), N(), std::integral_constant<int, 0>(), P1());
  }

  // With WK == 2 the two waves of a SIMD hold the two k-halves of one sub-tile: the upper half parks its accumulators in
  // LDS as they lie in the registers (16 bytes per lane and store: no bank conflicts), the lower half adds them and
  // carries the sub-tile from here on.
  constexpr int WAVE_ACC = TM * TN * 1024;  // floats of one wave's accumulators
  if (WK == 2) {
    static_assert(WK != 2 || 4 * WAVE_ACC * 4 <= STAGES * STAGE_BYTES, "pair merge fits the tile ring");
    float* park = reinterpret_cast<float*>(lds) + wq * WAVE_ACC;
    __syncthreads();  // every wave is out of the k loop
    if (wk == 1) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f32x4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
            *reinterpret_cast<f32x4*>(park + (((i * TN + j) * 4 + g) * 64 + lane) * 4) = v;
          }
    }
    __syncthreads();
    if (wk == 0) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(park + (((i * TN + j) * 4 + g) * 64 + lane) * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][4 * g + e] += v[e];
          }
    }
  }

  if constexpr (COLSUM) {
    // the two k-halves of the column sums meet like the accumulators above (one more round through the same LDS), then
    // lane n of the lower half adds column n of each of its 32-column blocks - row 0 of the result, like every row
    float* parkc = reinterpret_cast<float*>(lds) + wn * (TN * 1024);
    __syncthreads();
    if (cs_wave && wk == 1) {
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 v = {cs[j][4 * g], cs[j][4 * g + 1], cs[j][4 * g + 2], cs[j][4 * g + 3]};
          *reinterpret_cast<f32x4*>(parkc + ((j * 4 + g) * 64 + lane) * 4) = v;
        }
    }
    __syncthreads();
    if (cs_wave && wk == 0 && lane < 32) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = n0 + wn * (BN / WN) + j * 32 + lane;
        const float other = parkc[(j * 4 * 64 + lane) * 4];   // element 0 of piece 0: row 0 of the upper half's sums
        if (col < p.n) p.colsum[zi * p.colsum_si + col] += cs[j][0] + other;
      }
    }
  }

  // Split-K through a workspace: every slice stores its accumulators as they lie in the registers (1 KiB per store
  // instruction), then takes a ticket; the workgroup that draws the last one adds the slices in index order - its own
  // from registers - so that the result does not depend on which slice came last.
  if (p.ws_part != nullptr) {
    constexpr int TILE_ACC = WM * WN * WAVE_ACC;  // = BM * BN
    const int tile_id = bx;
    float* part = p.ws_part + (size_t)tile_id * p.splitk * TILE_ACC;
    float* mine = part + (size_t)ks_id * TILE_ACC + wq * WAVE_ACC;
    if (wk == 0) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f32x4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
            part_store4(mine + (((i * TN + j) * 4 + g) * 64 + lane) * 4, v);
          }
    }
    // the stores above go through to device-coherent memory; once they are acknowledged the ticket may be drawn
    __builtin_amdgcn_s_waitcnt(DS_VMCNT(0));
    __syncthreads();  // every wave is out of the k loop / the pair merge (the ticket word overlays the tile ring)
    unsigned* ticket = reinterpret_cast<unsigned*>(lds);
    if (tid == 0) *ticket = __hip_atomic_fetch_add(p.ws_count + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*ticket != (unsigned)(p.splitk - 1)) return;
    if (tid == 0) __hip_atomic_store(p.ws_count + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (wk == 0) {
      // every slice's copy is read back (this workgroup's own too: same bits as its registers), one 32x32 tile of
      // all slices per round trip; straight-line code, since the loads complete behind the compiler's back
      const int ns = p.splitk;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          f32x4 o[4][4];
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            const int sl = s < ns ? s : ns - 1;  // slots past the last slice re-read it and are not added
#pragma unroll
            for (int g = 0; g < 4; ++g)
              part_load4(part + (size_t)sl * TILE_ACC + (size_t)wq * WAVE_ACC + (((i * TN + j) * 4 + g) * 64 + lane) * 4, o[s][g]);
          }
          asm volatile("s_waitcnt vmcnt(0)"
                       : "+v"(o[0][0]), "+v"(o[0][1]), "+v"(o[0][2]), "+v"(o[0][3]), "+v"(o[1][0]), "+v"(o[1][1]), "+v"(o[1][2]),
                         "+v"(o[1][3]), "+v"(o[2][0]), "+v"(o[2][1]), "+v"(o[2][2]), "+v"(o[2][3]), "+v"(o[3][0]), "+v"(o[3][1]),
                         "+v"(o[3][2]), "+v"(o[3][3]));
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f32x4 t = o[0][g];
            if (ns > 1) t += o[1][g];
            if (ns > 2) t += o[2][g];
            if (ns > 3) t += o[3][g];
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][4 * g + e] = t[e];
          }
        }
    }
  }

  // With WK == 4 every wave holds a partial sum of the whole 64x64 tile: each parks the three 32x32 quadrants that are
  // not its own (as they lie in the registers; 4 x 12 KB = the tile ring), then adds to its own quadrant the three
  // copies of it, in the order of the waves that wrote them, and carries that quadrant through the epilogue as wave
  // (wave / 2, wave % 2) of a 2 x 2 grid.
  if constexpr (WK == 4) {
    static_assert(WK != 4 || 4 * 3 * 4096 <= STAGES * STAGE_BYTES, "quadrant merge fits the tile ring");
    // copy s (0..2) of quadrant q: 4 KB at lds + (q * 3 + s) * 4096, piece g of lane l at ((g * 64) + l) * 16
    auto park = [&](const f32x16& a, int q, int sl) {
      char* dst = lds + (q * 3 + sl) * 4096;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 v = {a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
        *reinterpret_cast<f32x4*>(dst + (g * 64 + lane) * 16) = v;
      }
    };
    auto gather = [&](f32x16& a, int q) {
#pragma unroll
      for (int sl = 0; sl < 3; ++sl)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 v = *reinterpret_cast<const f32x4*>(lds + (q * 3 + sl) * 4096 + (g * 64 + lane) * 16);
#pragma unroll
          for (int e = 0; e < 4; ++e) a[4 * g + e] += v[e];
        }
    };
    __syncthreads();  // every wave is out of the k loop
    // wave w is copy (w < q ? w : w - 1) of quadrant q != w
    if (wk == 0) { park(acc[0][1], 1, 0); park(acc[1][0], 2, 0); park(acc[1][1], 3, 0); }
    else if (wk == 1) { park(acc[0][0], 0, 0); park(acc[1][0], 2, 1); park(acc[1][1], 3, 1); }
    else if (wk == 2) { park(acc[0][0], 0, 1); park(acc[0][1], 1, 1); park(acc[1][1], 3, 2); }
    else { park(acc[0][0], 0, 2); park(acc[0][1], 1, 2); park(acc[1][0], 2, 2); }
    __syncthreads();
    if (wk == 1) acc[0][0] = acc[0][1];
    else if (wk == 2) acc[0][0] = acc[1][0];
    else if (wk == 3) acc[0][0] = acc[1][1];
    gather(acc[0][0], wk);
  }
  // the wave grid and the sub-tiles per wave as the epilogue sees them
  constexpr int EWM = WK == 4 ? 2 : WM, EWN = WK == 4 ? 2 : WN, ETM = WK == 4 ? 1 : TM, ETN = WK == 4 ? 1 : TN;
  const int ewm = WK == 4 ? (wk >> 1) : wm, ewn = WK == 4 ? (wk & 1) : wn;
  const bool carries = WK == 4 || wk == 0;

  // Epilogue through LDS, one 32-row MFMA block of every wave at a time: the waves that carry the sub-tiles park
  // alpha * acc + bias as fp32 rows, then every thread streams 8 consecutive columns of a row, so that residual /
  // auxiliary reads and C writes are 16-byte vectors covering whole rows of the tile.
  constexpr int LDW = BN + 4;
  constexpr int SLAB_ROWS = EWM * 32;
  constexpr int VPR = BN / 8;
  constexpr int VECS = SLAB_ROWS * VPR;
  static_assert(SLAB_ROWS * LDW * 4 <= STAGES * STAGE_BYTES, "staging slab fits the tile ring");
  float* sc = reinterpret_cast<float*>(lds);
  const int flags = p.flags;
#pragma unroll
  for (int i = 0; i < ETM; ++i) {
    __syncthreads();
    if (carries) {
#pragma unroll
      for (int j = 0; j < ETN; ++j) {
        const int cl = ewn * (BN / EWN) + j * 32 + (lane & 31);
        const int col = n0 + cl;
        const float bias = ((flags & DS_EPI_BIAS) && col < p.n) ? p.bias[col] : 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int rs = ewm * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
          sc[rs * LDW + cl] = acc[i][j][e] * p.alpha + bias;
        }
      }
    }
    __syncthreads();
#pragma unroll 2
    for (int v = tid; v < VECS; v += 64 * NW) {
      const int rs = v / VPR, cl = (v % VPR) * 8;
      const int row = m0 + (rs >> 5) * (BM / EWM) + i * 32 + (rs & 31), col = n0 + cl;
      if (row >= p.m || col >= p.n) continue;
      float x[8];
      const f32x4 lo = *reinterpret_cast<const f32x4*>(sc + rs * LDW + cl);
      const f32x4 hi = *reinterpret_cast<const f32x4*>(sc + rs * LDW + cl + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { x[e] = lo[e]; x[4 + e] = hi[e]; }
      gemm_epilogue_vec8<T>(p, c_off, (int64_t)row * p.ldc + col, x);
    }
  }
}

}  // namespace dsgemm
