// C[M,N] = epilogue(A[M,K] · W[N,K]^T) on the 256x256 workgroup tile: the GEMM of the large batches (every trunk linear
// of a 4096-position forward). The call sites, operand layout and epilogue are those described in gemm.hip. The kernel
// is a header because its instances are spread over two translation units (gemm_dma.hip, gemm_dma_resnorm.hip): a
// kernel added to a code object moves the others in it, and their speed depends measurably on where they land.
#pragma once
#include "gemm_tile.hpp"

#include <atomic>
#include <mutex>

namespace crl {

// ---- 256x256 tile fed by direct global->LDS loads ------------------------------------------
// The loads bypass the register file (global_load_lds_dwordx4: lane l of a wave-instruction
// writes LDS bytes [base + 16l, base + 16l + 16)), which frees the 32 staging registers and the
// LDS store instructions of the register-staged kernel. The kernel is written for a ring of
// NSTAGE stages of ROWB bytes per row; the instantiated form uses 128-byte rows and two stages
// (one barrier per 128 bytes of K): a 4-stage ring of 64-byte rows kept three stages in flight
// but paid twice the barriers and measured slower.
//  * A stage holds 256 weight rows then 256 activation rows; chunk c of row r sits at chunk
//    c ^ swizzle(r) (the same XOR pattern as above for 8 chunks per row).
//  * Wave w issues the loads for rows [64(w&3), +64) of the weight block (w < 4) or of the
//    activation block (w >= 4); the swizzle is applied on the global side (which chunk a lane
//    fetches). A K tail is fetched from a block of zeros.
template <int ROWB_, int NSTAGE_>
struct DmaCfgT {
  static constexpr int BM = 256, BN = 256, WGM = 2, WGN = 4, NW = 8, NT = 512;
  static constexpr int WM = 128, WN = 64, TM = 4, TN = 2;
  static constexpr int ROWB = ROWB_, NSTAGE = NSTAGE_;
  static constexpr int CHUNKS = ROWB / 16;            // 16-byte chunks per stage row
  static constexpr int ROWS_PER_INSTR = 64 / CHUNKS;  // rows one wave-instruction fills
  static constexpr int LOADS = 64 / ROWS_PER_INSTR;   // wave-instructions per wave and stage (64 rows each)
  static constexpr int STAGE_BYTES = (BM + BN) * ROWB;
  static constexpr int EPI_BYTES = NW * 32 * WN * 4;
  static constexpr int RING_BYTES = NSTAGE * STAGE_BYTES > EPI_BYTES ? NSTAGE * STAGE_BYTES : EPI_BYTES;
  static constexpr int STATS_OFF = RING_BYTES + 256;   // behind the landing strip of the L2 prefetch loads
  static constexpr int LDS_BYTES = STATS_OFF + NW * 2 * WM * 4;   // + row statistics of a residual normalised on the fly
};
typedef DmaCfgT<128, 2> DmaCfg2;     // 128-byte rows, 2 stages (one in flight), half as many barriers

__device__ __forceinline__ int dma_swizzle(int r) { return (((r >> 2) & 1) << 1) | (((r >> 1) ^ (r >> 3)) & 1); }
template <int CHUNKS>
__device__ __forceinline__ int dma_sw(int r) { return CHUNKS == 4 ? dma_swizzle(r) : lds_swizzle(r); }

// s_waitcnt with only vmcnt constrained (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

template <typename Cfg, int IN_DT, int OUT_DT, int RES_NORM = 0>
__global__ void __launch_bounds__(Cfg::NT, 2) gemm_dma_kernel(const GemmArgs a, const uint8_t* zeros, const int pf) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, NSTAGE = Cfg::NSTAGE, LOADS = Cfg::LOADS;
  constexpr int ESZ = (IN_DT == DT_FP8) ? 1 : 2;
  constexpr int KSTEPS = Cfg::ROWB / ((IN_DT == DT_FP8) ? 64 : 32);  // MFMA k-steps per stage
  extern __shared__ __align__(16) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % Cfg::WGM, wn = wave / Cfg::WGM;
  const int lr = lane & 31, g = lane >> 5;

  const int tiles_n = (a.N + BN - 1) / BN;
  const int nblk = gridDim.x;
  int pid = blockIdx.x;
  {
    const int per = nblk >> 3;
    if (pid < (per << 3)) pid = (pid & 7) * per + (pid >> 3);
  }
  // Inside an XCD's range the tiles are walked in groups of 8 x w (M x N), w = 4 where the tile columns divide by
  // four and 3 or 4 otherwise (13 columns: 4+3+3+3), so the 32 workgroups resident on the XCD share 8 activation
  // tiles and about 4 weight tiles (3 MB of operands at K = 1024 bytes, inside its 4 MB L2). Eight tile rows are
  // walked column group by column group before the next eight rows.
  int tile_m = pid / tiles_n, tile_n = pid - tile_m * tiles_n;
  int grp_w = 4, grp_q = tile_n & 3;   // width of this tile's column group and its place in it
  {
    constexpr int GM = 8;
    const int tiles_m = (a.M + BM - 1) / BM;
    // (16-bit operands keep the plain row-major order unless the columns divide by four: the three-wide groups and
    // the extra code measured 2 % slower for them, 1-2 % faster for e4m3.)
    if (tiles_m % GM == 0 && (IN_DT == DT_FP8 || tiles_n % 4 == 0)) {
      const int ngrp = (tiles_n + 3) >> 2, wb = tiles_n / ngrp, extra = tiles_n - wb * ngrp;
      const int sr = pid / (GM * tiles_n), rem = pid - sr * (GM * tiles_n);
      const int big = GM * (wb + 1) * extra;   // tiles of the `extra` groups that are one column wider
      int gi, r2;
      if (rem < big) { grp_w = wb + 1; gi = rem / (GM * grp_w); r2 = rem - gi * GM * grp_w; }
      else { grp_w = wb; const int rem2 = rem - big; gi = rem2 / (GM * wb); r2 = rem2 - gi * GM * wb; gi += extra; }
      grp_q = r2 % grp_w;
      tile_m = sr * GM + r2 / grp_w;
      tile_n = gi * wb + (gi < extra ? gi : extra) + grp_q;
    }
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const long kbytes = (long)a.K * ESZ;
  const int nslab = (int)((kbytes + Cfg::ROWB - 1) / Cfg::ROWB);
  const long kmax = kbytes - 16;

  if constexpr (RES_NORM != 0) {
    // Statistics of this wave's 128 rows (two rows = 16 bytes per lane), requested before anything else and landed
    // outside the ring: they are in LDS long before the epilogue asks for them.
    static_assert(Cfg::WM == 128, "one 16-byte load per lane covers the wave's rows");
    int m = m0 + wm * Cfg::WM + 2 * lane;
    m = m + 1 < a.M ? m : 0;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.res_stats + 2 * (long)m),
                                     (__attribute__((address_space(3))) void*)(smem + Cfg::STATS_OFF + wave * (2 * Cfg::WM * 4)), 16, 0, 0);
  }

  // Loader role of this wave.
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
      gptr[j] = reinterpret_cast<const uint8_t*>(a.A) + (long)gm * a.lda * ESZ + kchunk[j];
    } else {
      int gn = n0 + r;
      gn = gn < a.N ? gn : a.N - 1;
      gptr[j] = reinterpret_cast<const uint8_t*>(a.W) + (long)gn * a.ldw * ESZ + kchunk[j];
    }
  }
  const int lds_row0 = (loads_a ? BN : 0) + rbase;  // first stage row this wave fills
  auto issue_one = [&](int slab, int j) {
    uint8_t* st = smem + (slab % NSTAGE) * Cfg::STAGE_BYTES + lds_row0 * Cfg::ROWB;
    const long kb = (long)slab * Cfg::ROWB;
    const uint8_t* src = (kb + kchunk[j] <= kmax) ? gptr[j] + kb : zeros;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)(st + j * 1024), 16, 0, 0);
  };
  auto issue = [&](int slab) {
    uint8_t* st = smem + (slab % NSTAGE) * Cfg::STAGE_BYTES + lds_row0 * Cfg::ROWB;
    const long kb = (long)slab * Cfg::ROWB;
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
      const uint8_t* src = (kb + kchunk[j] <= kmax) ? gptr[j] + kb : zeros;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(st + j * 1024), 16, 0, 0);
    }
  };

  // L2 prefetch. The workgroups resident on an XCD walk K in step, so the 4-8 readers of an operand line ask for it
  // at the same moment and all of them wait out the one fetch from memory. Each reader therefore touches its share of
  // the lines of a slab `pf` slabs before any of them loads it: one dword per 128-byte line, landed in an LDS strip
  // nobody reads. Wave 0 takes 64 of the 256 activation rows (the quarter chosen by the tile's column), wave 1 32 of
  // the 256 weight rows (the eighth chosen by the tile's row; its upper lanes touch the second half-line).
  const uint8_t* pf_ptr = nullptr;
  int pf_n = 0, pf_step = 0;   // wave-instructions per slab and the byte distance between their rows
  if (IN_DT == DT_FP8 && pf > 0 && wave < 2) {
    if (wave == 0) {
      pf_n = (4 + grp_w - 1) / grp_w;
      int gm = m0 + ((grp_q * pf_n) & 3) * 64 + lane;
      gm = gm < a.M ? gm : a.M - 1;
      pf_ptr = reinterpret_cast<const uint8_t*>(a.A) + (long)gm * a.lda * ESZ;
      pf_step = (m0 + 256 <= a.M) ? 64 * a.lda * ESZ : 0;
    } else {
      pf_n = 1;
      int gn = n0 + (tile_m & 7) * 32 + (lane & 31);
      gn = gn < a.N ? gn : a.N - 1;
      pf_ptr = reinterpret_cast<const uint8_t*>(a.W) + (long)gn * a.ldw * ESZ + (lane >> 5) * 64;
    }
  }
  auto prefetch = [&](int slab) {
    if (pf_ptr && slab < nslab) {
      const long kb = (long)slab * Cfg::ROWB;
      const bool inside = kb + 64 + 4 <= kbytes;
      for (int i = 0; i < pf_n; ++i) {
        const uint8_t* src = inside ? pf_ptr + kb + (long)i * pf_step : zeros;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)(smem + Cfg::RING_BYTES), 4, 0, 0);
      }
    }
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

  auto read_frags = [&](Frag<IN_DT> (&wf)[TN], Frag<IN_DT> (&xf)[TM], const uint8_t* st, int ks) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const uint8_t* row = st + wrow_off[tn];
      if constexpr (IN_DT == DT_FP8) {
        wf[tn].lo = *reinterpret_cast<const i32x4_t*>(row + (((4 * ks + 2 * g) ^ wrow_sw[tn]) << 4));
        wf[tn].hi = *reinterpret_cast<const i32x4_t*>(row + (((4 * ks + 2 * g + 1) ^ wrow_sw[tn]) << 4));
      } else {
        wf[tn].lo = *reinterpret_cast<const i32x4_t*>(row + (((2 * ks + g) ^ wrow_sw[tn]) << 4));
      }
    }
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const uint8_t* row = st + arow_off[tm];
      if constexpr (IN_DT == DT_FP8) {
        xf[tm].lo = *reinterpret_cast<const i32x4_t*>(row + (((4 * ks + 2 * g) ^ arow_sw[tm]) << 4));
        xf[tm].hi = *reinterpret_cast<const i32x4_t*>(row + (((4 * ks + 2 * g + 1) ^ arow_sw[tm]) << 4));
      } else {
        xf[tm].lo = *reinterpret_cast<const i32x4_t*>(row + (((2 * ks + g) ^ arow_sw[tm]) << 4));
      }
    }
  };

  // A wave whose 128x64 part lies wholly outside C (the last tile column of N = 3104 holds 32 columns) still takes its
  // share of the loads and every barrier, but reads no fragments and issues no MFMAs.
  const bool wave_active = (m0 + wm * Cfg::WM < a.M) && (n0 + wn * Cfg::WN < a.N);

#pragma unroll
  for (int s0 = 0; s0 < NSTAGE - 1; ++s0)
    if (s0 < nslab) issue(s0);
  for (int s0 = NSTAGE - 1; s0 < NSTAGE - 1 + pf; ++s0) prefetch(s0);

  for (int slab = 0; slab < nslab; ++slab) {
    // Loads still allowed in flight behind this slab's: LOADS per later slab already issued.
    const int ahead = nslab - 1 - slab;
    if (NSTAGE >= 4 && ahead >= 2) wait_vmcnt<2 * LOADS>();
    else if (NSTAGE >= 3 && ahead == 1) wait_vmcnt<LOADS>();
    else wait_vmcnt<0>();
    __syncthreads();
    const bool more = slab + NSTAGE - 1 < nslab;
    prefetch(slab + NSTAGE - 1 + pf);
    const uint8_t* st = smem + (slab % NSTAGE) * Cfg::STAGE_BYTES;
    if (!wave_active) {   // no MFMAs to put the loads between
      if (more) issue(slab + NSTAGE - 1);
      continue;
    }
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      Frag<IN_DT> wf[TN], xf[TM];
      read_frags(wf, xf, st, ks);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
          acc[tn][tm] = mfma_frag<IN_DT>(wf[tn], xf[tm], acc[tn][tm]);
          // The loads of the slab that follows the ring go out one at a time, one behind each of this slab's first MFMAs,
          // held in place by scheduling barriers, instead of all in a row behind the barrier (a wave stalls at a load
          // until the memory pipeline takes it, and spread out those stalls fall under MFMAs that are already
          // executing) and early enough for the last of them to land under the slab's other MFMAs.
          const int j = ks * TN * TM + tn * TM + tm;
          if (j < LOADS) {
            __builtin_amdgcn_sched_barrier(0);
            if (more) issue_one(slab + NSTAGE - 1, j);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
    }
  }

  __syncthreads();  // every wave is done with the ring before it becomes epilogue scratch

  gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT, RES_NORM>(a, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                                     m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane,
                                                     reinterpret_cast<float*>(smem + Cfg::STATS_OFF) + wave * (2 * Cfg::WM));
}

template <typename DCfg, int IN_DT, int OUT_DT, int RES_NORM = 0>
static hipError_t launch_dma(const GemmArgs& a, hipStream_t st) {
  static std::atomic<bool> attr_set[16] = {};
  hipError_t e = hipSuccess;
  const uint8_t* zeros = device_zeros(&e);
  if (!zeros) return e;
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_dma_kernel<DCfg, IN_DT, OUT_DT, RES_NORM>;
  if (!attr_set[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, DCfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles = ((a.M + DCfg::BM - 1) / DCfg::BM) * ((a.N + DCfg::BN - 1) / DCfg::BN);
  // The L2 prefetch pays for e4m3 operands where the column groups are exactly four tiles wide and K is long enough to run ahead of
  // (measured: 3-4 % at N = 1024, K = 1024 and 1536 bytes; nothing or a small loss at 6 and 13 tile columns and at K = 256).
  const int tiles_n = (a.N + DCfg::BN - 1) / DCfg::BN;
  const long kbytes = (long)a.K * (IN_DT == DT_FP8 ? 1 : 2);
  const int pf = (IN_DT == DT_FP8 && tiles_n % 4 == 0 && kbytes >= 8 * DCfg::ROWB) ? 2 : 0;
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(DCfg::NT), DCfg::LDS_BYTES, st, a, zeros, pf);
  return hipGetLastError();
}

}  // namespace crl
