// C[M,N] = epilogue(A[M,K] · W[N,K]^T) for e4m3 operands on the 256x256 workgroup tile, four waves of 128x128 outputs
// each (one wave per SIMD), software-pipelined inside the wave. Call sites, operand layout and epilogue are those of gemm.hip.
//
// Against the eight-wave kernel of gemm_dma_kernel.hpp (128x64 per wave): a wave's 16 MFMAs of a K step reuse each of its
// eight operand fragments four times instead of 2-4, so the fragment reads of a K step fall from 96 KB to 64 KB per
// workgroup, and with a single wave per SIMD nothing hides a wave's own latencies but its own instruction stream. The K
// loop is therefore written as one straight block per K step of 64 bytes per row in which the wave issues, interleaved
// one for one by scheduling-group barriers,
//   * the 16 MFMAs of step j from fragment set j%2,
//   * the 16 LDS reads of step j+1 into the other fragment set,
//   * its 8 direct-to-LDS loads of step j+3,
// so the matrix pipe always has the next MFMA waiting while LDS and the memory pipe work under it.
// Measured on MI355X against the eight-wave kernel: equal at long K (2.11 against 2.08 PFLOP/s at K = 8192), slower at
// K = 1024 (1.33 against 1.52: four waves take twice as long over the epilogue, and the three K steps fetched past the
// end cost as much as three real ones). With its loads switched off the same loop runs at 2.85 PFLOP/s (with or without
// the barrier), with its MFMAs switched off the loads alone take 72 % of the full time (with or without the fragment
// reads, with three or four K steps in flight): neither side is the bound by itself, they overlap by a third.
// The model's products therefore stay on the eight-wave kernel; this one is kept as tile 8 of crl_gemm.
// The ring holds four stages of 64-byte rows (256 weight rows, then 256 activation rows, 16-byte chunks XOR-swizzled as
// in gemm_dma_kernel.hpp). One workgroup barrier per K step, at the top of the block:
//   before it, the wave waits for its own loads of step j+1 (issued two blocks earlier);
//   after it, step j+1 is readable by everybody, and stage (j+3)%4 is free: its last readers were the fragment reads of
//   step j-1, which every wave issued in block j-2 and consumed in block j-1.
#pragma once
#include "gemm_dma_kernel.hpp"

namespace crl {

struct SpCfg {
  static constexpr int BM = 256, BN = 256, WGM = 2, WGN = 2, NW = 4, NT = 256;
  static constexpr int WM = 128, WN = 128, TM = 4, TN = 4;
  static constexpr int ROWB = 64, NSTAGE = 4, CHUNKS = 4;
  static constexpr int ROWS_PER_INSTR = 16, LOADS = 8;          // a wave fills 128 of the 512 rows of a stage
  static constexpr int STAGE_BYTES = (BM + BN) * ROWB;          // 32 KB
  static constexpr int EPI_BYTES = NW * 32 * WN * 4;            // 64 KB
  static constexpr int RING_BYTES = NSTAGE * STAGE_BYTES;       // 128 KB
  static constexpr int STATS_OFF = RING_BYTES + 256;            // behind the landing strip of the L2 touches
  static constexpr int LDS_BYTES = STATS_OFF + NW * 2 * WM * 4;
  static_assert(EPI_BYTES <= RING_BYTES, "the epilogue patches reuse the ring");
};

__device__ __forceinline__ void sp_barrier() { asm volatile("s_barrier" ::: "memory"); }

template <int OUT_DT, int RES_NORM = 0>
__global__ void __launch_bounds__(SpCfg::NT) gemm_sp_kernel(const GemmArgs a, const uint8_t* zeros) {
  typedef SpCfg Cfg;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, NSTAGE = Cfg::NSTAGE, LOADS = Cfg::LOADS;
  constexpr int IN_DT = DT_FP8;
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
    // Row statistics of this wave's 128 rows, landed outside the ring: the wave's oldest load, covered by its first wait.
    int m = m0 + wm * Cfg::WM + 2 * lane;
    m = m + 1 < a.M ? m : 0;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.res_stats + 2 * (long)m),
                                     (__attribute__((address_space(3))) void*)(smem + Cfg::STATS_OFF + wave * (2 * Cfg::WM * 4)), 16, 0, 0);
  }

  // Loader role: waves 0-1 fill the weight rows [128w, +128) of a stage, waves 2-3 the activation rows [128(w-2), +128):
  // 16 rows per wave-instruction, four 16-byte chunks per row, the swizzle applied on the global side. Row 16*i + lane/4
  // of the wave's block has the same swizzle for every i (it depends on bits 1-3 of the row only).
  const bool loads_a = wave >= 2;
  const int rbase = (wave & 1) * 128;
  const int r0 = rbase + lane / Cfg::CHUNKS;
  const int kchunk = ((lane % Cfg::CHUNKS) ^ dma_sw<Cfg::CHUNKS>(r0)) << 4;
  const uint8_t* gptr[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int r = r0 + Cfg::ROWS_PER_INSTR * i;
    if (loads_a) {
      int gm = m0 + r;
      gm = gm < a.M ? gm : a.M - 1;
      gptr[i] = reinterpret_cast<const uint8_t*>(a.A) + (long)gm * a.lda + kchunk;
    } else {
      int gn = n0 + r;
      gn = gn < a.N ? gn : a.N - 1;
      gptr[i] = reinterpret_cast<const uint8_t*>(a.W) + (long)gn * a.ldw + kchunk;
    }
  }
  const int lds_row0 = (loads_a ? BN : 0) + rbase;
  auto issue_loads = [&](int kstep) {
    uint8_t* st = smem + (kstep % NSTAGE) * Cfg::STAGE_BYTES + lds_row0 * Cfg::ROWB;
    const long kb = (long)kstep * Cfg::ROWB;
    const bool inside = kb + kchunk <= kmax;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const uint8_t* src = inside ? gptr[i] + kb : zeros;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(st + i * 1024), 16, 0, 0);
    }
  };

  f32x16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  // The MFMAs below are inline assembly, so the compiler does not know that a matrix instruction must not read an
  // accumulation register in the cycles right after a v_accvgpr_write to it, and it is free to sink the zeroing down to
  // the first MFMA (seen: stale values in single registers of two tiles). This statement depends on every accumulator
  // and every MFMA depends on it: the zeroing is complete, and some cycles old, before the first MFMA issues.
  asm volatile("s_nop 7\n\ts_nop 7"
               : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]), "+a"(acc[1][1]), "+a"(acc[1][2]), "+a"(acc[1][3]),
                 "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[2][2]), "+a"(acc[2][3]), "+a"(acc[3][0]), "+a"(acc[3][1]), "+a"(acc[3][2]), "+a"(acc[3][3]));

  // Byte offsets of this lane's two 16-byte fragment halves inside a stage (fixed for the whole kernel).
  int woff[TN][2], xoff[TM][2];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const int wr = wn * Cfg::WN + tn * 32 + lr;
    const int sw = dma_sw<Cfg::CHUNKS>(wr);
    woff[tn][0] = wr * Cfg::ROWB + (((2 * g) ^ sw) << 4);
    woff[tn][1] = wr * Cfg::ROWB + (((2 * g + 1) ^ sw) << 4);
  }
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int ar = wm * Cfg::WM + tm * 32 + lr;
    const int sw = dma_sw<Cfg::CHUNKS>(ar);
    xoff[tm][0] = (BN + ar) * Cfg::ROWB + (((2 * g) ^ sw) << 4);
    xoff[tm][1] = (BN + ar) * Cfg::ROWB + (((2 * g + 1) ^ sw) << 4);
  }
  const bool wave_active = (m0 + wm * Cfg::WM < a.M) && (n0 + wn * Cfg::WN < a.N);

  // Fragments live in two sets of eight (four weight, four activation), 8 registers each: i32x8 = one MFMA operand.
  i32x8_t wf[2][TN], xf[2][TM];
  // Read number r (0..15) of a K step, in the order the MFMAs first need the fragments: w0, x0, x1, x2, x3, w1, w2, w3,
  // low then high half.
  auto read_one = [&](const uint8_t* st, auto setc, auto rc) {
    constexpr int set = decltype(setc)::value, r = decltype(rc)::value;
    constexpr int f = r >> 1, half = r & 1;
    constexpr bool is_w = f == 0 || f >= 5;
    constexpr int idx = f == 0 ? 0 : f <= 4 ? f - 1 : f - 4;
    const i32x4_t v = *reinterpret_cast<const i32x4_t*>(st + (is_w ? woff[idx][half] : xoff[idx][half]));
    i32x8_t& dst = is_w ? wf[set][idx] : xf[set][idx];
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[4 * half + e] = v[e];
  };
  auto read_frags = [&](int kstep, auto setc) {
    const uint8_t* st = smem + (kstep % NSTAGE) * Cfg::STAGE_BYTES;
    static_for<0, 16>([&](auto rc) { read_one(st, setc, rc); });
  };
  // The accumulators are pinned to the accumulation registers by the operand constraint: left to the register
  // allocator, 256 accumulator registers plus 128 fragment registers make it shuffle tiles between the two register
  // files inside the loop. The instruction is the e4m3 x e4m3 form (no format modifiers).
  auto mfma = [&](f32x16_t& c, const i32x8_t& w, const i32x8_t& x) {
    asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(w), "v"(x));
  };
  auto mfmas = [&](auto setc) {
    constexpr int set = decltype(setc)::value;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) mfma(acc[tn][tm], wf[set][tn], xf[set][tm]);
  };
  // One K step: the 16 MFMAs of step j (set CUR) in program order, and between them the fragment reads of step j+1
  // (other set; two behind each of the first four MFMAs, one behind each of the next eight, so the last read has four
  // MFMAs to land under) and the loads of step j+3 (one behind every second MFMA). Full scheduling barriers hold the order.
  auto block = [&](int j, auto curc, auto nextc, auto morec) {
    constexpr int CUR = decltype(curc)::value;
    constexpr bool NEXT = decltype(nextc)::value, MORE = decltype(morec)::value;
    using NSET = std::integral_constant<int, CUR ^ 1>;
    const uint8_t* st_next = smem + ((j + 1) % NSTAGE) * Cfg::STAGE_BYTES;
    uint8_t* st_load = smem + ((j + NSTAGE - 1) % NSTAGE) * Cfg::STAGE_BYTES + lds_row0 * Cfg::ROWB;
    const long kb = (long)(j + NSTAGE - 1) * Cfg::ROWB;
    const bool inside = kb + kchunk <= kmax;
    static_for<0, TN * TM>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      mfma(acc[i / TM][i % TM], wf[CUR][i / TM], xf[CUR][i % TM]);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (NEXT) {
        if constexpr (i < 4) {
          read_one(st_next, NSET{}, std::integral_constant<int, 2 * i>{});
          read_one(st_next, NSET{}, std::integral_constant<int, 2 * i + 1>{});
        } else if constexpr (i < 12) {
          read_one(st_next, NSET{}, std::integral_constant<int, i + 4>{});
        }
      }
      if constexpr (MORE && (i & 1) == 1) {
        constexpr int l = i >> 1;
        const uint8_t* src = inside ? gptr[l] + kb : zeros;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)(st_load + l * 1024), 16, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  using T = std::true_type;
  using F = std::false_type;

  // K steps 0..2 go out at once; step 0 has to be there before anybody reads. Steps past the end of K are fetched from
  // the block of zeros like a K tail: every block of the loop below is then the same straight code (reads of the next
  // step, loads three steps ahead), whatever nk is, and a step of zeros adds nothing to the accumulators. An odd nk is
  // rounded up for the same reason (the fragment sets alternate at compile time).
  const int nk2 = (nk + 1) & ~1;
#pragma unroll
  for (int s0 = 0; s0 < NSTAGE - 1; ++s0) issue_loads(s0);
  wait_vmcnt<2 * LOADS>();
  sp_barrier();

  if (wave_active) {
    read_frags(0, C0{});
    for (int j = 0; j < nk2; j += 2) {
      wait_vmcnt<LOADS>();      // this wave's loads of step j+1 have landed (those of step j+2 may be in flight)
      sp_barrier();
      block(j, C0{}, T{}, T{});
      wait_vmcnt<LOADS>();
      sp_barrier();
      block(j + 1, C1{}, T{}, T{});
    }
  } else {
    // A wave whose 128x128 part lies wholly outside C: its share of the loads and every barrier, nothing else.
    for (int j = 0; j < nk2; ++j) {
      wait_vmcnt<LOADS>();
      sp_barrier();
      issue_loads(j + NSTAGE - 1);
    }
  }
  wait_vmcnt<0>();   // the (zero) steps fetched past the end have landed too: the ring can be reused
  // The MFMAs above are opaque to the compiler's hazard handling: let the last of them (16 passes) retire before the
  // epilogue reads the accumulators.
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  sp_barrier();   // every wave is done with the ring before it becomes epilogue scratch

  gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT, RES_NORM>(a, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                                     m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane,
                                                     reinterpret_cast<float*>(smem + Cfg::STATS_OFF) + wave * (2 * Cfg::WM));
}

template <int OUT_DT, int RES_NORM = 0>
static hipError_t launch_sp(const GemmArgs& a, hipStream_t st) {
  static std::atomic<bool> attr_set[16] = {};
  hipError_t e = hipSuccess;
  const uint8_t* zeros = device_zeros(&e);
  if (!zeros) return e;
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_sp_kernel<OUT_DT, RES_NORM>;
  if (!attr_set[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, SpCfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles = ((a.M + SpCfg::BM - 1) / SpCfg::BM) * ((a.N + SpCfg::BN - 1) / SpCfg::BN);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(SpCfg::NT), SpCfg::LDS_BYTES, st, a, zeros);
  return hipGetLastError();
}

}  // namespace crl
