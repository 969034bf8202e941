// C[M,N] = epilogue(A[M,K] · W[N,K]^T) for e4m3 operands on the 256x256 workgroup tile with the two waves of every SIMD
// working out of step ("ping-pong"). Call sites, operand layout and epilogue are those of gemm.hip.
//
// The tile, its eight waves (2 x 4, 128 x 64 outputs each), the direct global->LDS loads and the XCD-aware tile order are
// those of gemm_dma_kernel.hpp. What differs is the K loop. There all eight waves do the same thing at the same time:
// after the slab barrier they all read fragments (the matrix cores idle while LDS serves eight waves at once), then they
// all issue MFMAs (LDS idles), and the parts of a slab add up instead of overlapping. Here the waves of a workgroup form
// two groups with one wave on every SIMD each (waves 0-3 and 4-7), and a K step of 64 bytes per row is split into two
// phases separated by workgroup barriers:
//   R(j)  read the 12 fragments of K step j from LDS (and wait for this wave's direct-to-LDS loads of step j+1)
//   M(j)  issue the 8 MFMAs of K step j, with this wave's four loads of step j+3 placed between them
// The second group starts one phase late, so at any time one group is in an R phase and the other in an M phase: the
// matrix cores of a SIMD always have one wave issuing MFMAs while the other wave's LDS reads and load issue run under them.
// The ring holds four stages of 64-byte rows (4 x 32 KB); a stage is refilled three K steps ahead.
//
//   phase slot:   0      1      2      3      4      5    ...
//   waves 0-3:   R(0)   M(0)   R(1)   M(1)   R(2)   M(2)
//   waves 4-7:    -     R(0)   M(0)   R(1)   M(1)   R(2)  ...
//
// Stage (j+3)%4 held K step j-1, which the second group finished reading in slot 2j-1; the loads of step j+3 are issued
// in M(j), i.e. in slot 2j+1 or 2j+2, after the barrier that ended slot 2j-1 ... 2j. They have to be visible when the
// first group reads step j+3 in slot 2j+6: every wave waits for its own loads of step i+1 at the end of R(i) (slot 2i or
// 2i+1), and the barrier that follows publishes them; that leaves a load three phase slots to land.
// Every wave arrives at every barrier: a wave whose part of an edge tile lies outside C skips its fragment reads and MFMAs only.
// Measured on MI355X against the in-step kernel: 3-5 % slower on every shape of a 4096-position forward (1.41 against
// 1.49 PFLOP/s at N = K = 1024, 2.02 against 2.10 at K = 8192). Taking the waves out of step does not buy the overlap
// the in-step kernel lacks: the time goes to the loads themselves (see gemm_sp_kernel.hpp). The model's products stay on
// the in-step kernel; this one is kept as tile 6 of crl_gemm.
#pragma once
#include "gemm_dma_kernel.hpp"

namespace crl {

typedef DmaCfgT<64, 4> PpCfg;   // 64-byte rows, four stages

// Workgroup barrier without the memory waits of __syncthreads(): loads stay in flight across it. The "memory" clobber
// keeps the compiler from moving LDS accesses over it.
__device__ __forceinline__ void phase_barrier() { asm volatile("s_barrier" ::: "memory"); }
__device__ __forceinline__ void wait_lds_reads() { __builtin_amdgcn_s_waitcnt(0xC07F); }   // lgkmcnt(0) only

template <int OUT_DT, int RES_NORM = 0>
__global__ void __launch_bounds__(PpCfg::NT, 2) gemm_pp_kernel(const GemmArgs a, const uint8_t* zeros) {
  typedef PpCfg Cfg;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, NSTAGE = Cfg::NSTAGE, LOADS = Cfg::LOADS;
  constexpr int IN_DT = DT_FP8;
  static_assert(Cfg::ROWB == 64 && LOADS == 4 && NSTAGE == 4, "one e4m3 K step (64 bytes per row) per stage");
  extern __shared__ __align__(16) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % Cfg::WGM, wn = wave / Cfg::WGM;
  const int lr = lane & 31, g = lane >> 5;
  const bool lead = wave < 4;   // waves w and w+4 share a SIMD: one of each group per SIMD

  const int tiles_n = (a.N + BN - 1) / BN;
  const int nblk = gridDim.x;
  int pid = blockIdx.x;
  {
    const int per = nblk >> 3;
    if (pid < (per << 3)) pid = (pid & 7) * per + (pid >> 3);
  }
  // Tile order inside an XCD's range: groups of 8 x w tiles (M x N), w = 3 or 4, as in gemm_dma_kernel.hpp.
  int tile_m = pid / tiles_n, tile_n = pid - tile_m * tiles_n;
  {
    constexpr int GM = 8;
    const int tiles_m = (a.M + BM - 1) / BM;
    if (tiles_m % GM == 0) {
      const int ngrp = (tiles_n + 3) >> 2, wb = tiles_n / ngrp, extra = tiles_n - wb * ngrp;
      const int sr = pid / (GM * tiles_n), rem = pid - sr * (GM * tiles_n);
      const int big = GM * (wb + 1) * extra;
      int gi, r2, grp_w;
      if (rem < big) { grp_w = wb + 1; gi = rem / (GM * grp_w); r2 = rem - gi * GM * grp_w; }
      else { grp_w = wb; const int rem2 = rem - big; gi = rem2 / (GM * wb); r2 = rem2 - gi * GM * wb; gi += extra; }
      tile_m = sr * GM + r2 / grp_w;
      tile_n = gi * wb + (gi < extra ? gi : extra) + r2 % grp_w;
    }
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const long kbytes = (long)a.K;           // one byte per element
  const int nk = (int)((kbytes + Cfg::ROWB - 1) / Cfg::ROWB);
  const long kmax = kbytes - 16;

  if constexpr (RES_NORM != 0) {
    // Row statistics of this wave's 128 rows, landed outside the ring; the oldest load of the wave, so the first
    // wait below covers it.
    int m = m0 + wm * Cfg::WM + 2 * lane;
    m = m + 1 < a.M ? m : 0;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.res_stats + 2 * (long)m),
                                     (__attribute__((address_space(3))) void*)(smem + Cfg::STATS_OFF + wave * (2 * Cfg::WM * 4)), 16, 0, 0);
  }

  // Loader role: waves 0-3 fill the 256 weight rows of a stage, waves 4-7 the 256 activation rows, 64 rows each,
  // 16 rows per wave-instruction (four 16-byte chunks per row, swizzled on the global side).
  const bool loads_a = wave >= 4;
  const int rbase = (wave & 3) * 64;
  const uint8_t* gptr[LOADS];
  int kchunk[LOADS];
#pragma unroll
  for (int j = 0; j < LOADS; ++j) {
    const int r = rbase + Cfg::ROWS_PER_INSTR * j + lane / Cfg::CHUNKS;
    const int c = (lane % Cfg::CHUNKS) ^ dma_sw<Cfg::CHUNKS>(r);
    kchunk[j] = c << 4;
    if (loads_a) {
      int gm = m0 + r;
      gm = gm < a.M ? gm : a.M - 1;
      gptr[j] = reinterpret_cast<const uint8_t*>(a.A) + (long)gm * a.lda + kchunk[j];
    } else {
      int gn = n0 + r;
      gn = gn < a.N ? gn : a.N - 1;
      gptr[j] = reinterpret_cast<const uint8_t*>(a.W) + (long)gn * a.ldw + kchunk[j];
    }
  }
  const int lds_row0 = (loads_a ? BN : 0) + rbase;
  auto issue_one = [&](int kstep, int j) {
    uint8_t* st = smem + (kstep % NSTAGE) * Cfg::STAGE_BYTES + lds_row0 * Cfg::ROWB;
    const long kb = (long)kstep * Cfg::ROWB;
    const uint8_t* src = (kb + kchunk[j] <= kmax) ? gptr[j] + kb : zeros;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)(st + j * 1024), 16, 0, 0);
  };

  f32x16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  int wrow_off[TN], wrow_sw[TN], arow_off[TM], arow_sw[TM];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const int wr = wn * Cfg::WN + tn * 32 + lr;
    wrow_off[tn] = wr * Cfg::ROWB;
    wrow_sw[tn] = dma_sw<Cfg::CHUNKS>(wr);
  }
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int ar = wm * Cfg::WM + tm * 32 + lr;
    arow_off[tm] = (BN + ar) * Cfg::ROWB;
    arow_sw[tm] = dma_sw<Cfg::CHUNKS>(ar);
  }
  const bool wave_active = (m0 + wm * Cfg::WM < a.M) && (n0 + wn * Cfg::WN < a.N);

  // K steps 0..2 go out at once; step 0 has to be there before anybody reads.
#pragma unroll
  for (int s0 = 0; s0 < NSTAGE - 1; ++s0)
    if (s0 < nk) {
#pragma unroll
      for (int j = 0; j < LOADS; ++j) issue_one(s0, j);
    }
  if (nk >= 3) wait_vmcnt<2 * LOADS>();
  else if (nk == 2) wait_vmcnt<LOADS>();
  else wait_vmcnt<0>();
  phase_barrier();
  if (!lead) phase_barrier();   // slot 0: the first group reads step 0 alone

  for (int j = 0; j < nk; ++j) {
    // ---- R(j)
    const uint8_t* st = smem + (j % NSTAGE) * Cfg::STAGE_BYTES;
    Frag<IN_DT> wf[TN], xf[TM];
    if (wave_active) {
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const uint8_t* row = st + wrow_off[tn];
        wf[tn].lo = *reinterpret_cast<const i32x4_t*>(row + (((2 * g) ^ wrow_sw[tn]) << 4));
        wf[tn].hi = *reinterpret_cast<const i32x4_t*>(row + (((2 * g + 1) ^ wrow_sw[tn]) << 4));
      }
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        const uint8_t* row = st + arow_off[tm];
        xf[tm].lo = *reinterpret_cast<const i32x4_t*>(row + (((2 * g) ^ arow_sw[tm]) << 4));
        xf[tm].hi = *reinterpret_cast<const i32x4_t*>(row + (((2 * g + 1) ^ arow_sw[tm]) << 4));
      }
    }
    // This wave's loads of step j+1 must have landed before the barrier below publishes them; only the loads of
    // step j+2 (issued in M(j-1)) may stay in flight.
    if (j + 2 < nk) wait_vmcnt<LOADS>();
    else wait_vmcnt<0>();
    wait_lds_reads();
    __builtin_amdgcn_sched_barrier(0);
    phase_barrier();
    // ---- M(j)
    const bool more = j + NSTAGE - 1 < nk;
    if (wave_active) {
      __builtin_amdgcn_s_setprio(2);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          acc[tn][tm] = mfma_frag<IN_DT>(wf[tn], xf[tm], acc[tn][tm]);
          const int i = tn * TM + tm;
          if ((i & 1) == 1) {   // one load behind every second MFMA, held in place
            __builtin_amdgcn_sched_barrier(0);
            if (more) issue_one(j + NSTAGE - 1, i >> 1);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      __builtin_amdgcn_s_setprio(0);
    } else if (more) {
#pragma unroll
      for (int i = 0; i < LOADS; ++i) issue_one(j + NSTAGE - 1, i);
    }
    // Every phase ends in a barrier except the second group's last M phase (the first group's last barrier pairs
    // with the one after the second group's last R phase).
    if (lead || j + 1 < nk) phase_barrier();
  }

  // No wave reads the ring any more (the second group's last R phase ended before the first group's last barrier),
  // and every wave has waited for all of its loads: the ring is free for the epilogue patches.
  gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT, RES_NORM>(a, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                                     m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane,
                                                     reinterpret_cast<float*>(smem + Cfg::STATS_OFF) + wave * (2 * Cfg::WM));
}

template <int OUT_DT, int RES_NORM = 0>
static hipError_t launch_pp(const GemmArgs& a, hipStream_t st) {
  static std::atomic<bool> attr_set[16] = {};
  hipError_t e = hipSuccess;
  const uint8_t* zeros = device_zeros(&e);
  if (!zeros) return e;
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_pp_kernel<OUT_DT, RES_NORM>;
  if (!attr_set[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, PpCfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles = ((a.M + PpCfg::BM - 1) / PpCfg::BM) * ((a.N + PpCfg::BN - 1) / PpCfg::BN);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(PpCfg::NT), PpCfg::LDS_BYTES, st, a, zeros);
  return hipGetLastError();
}

}  // namespace crl
