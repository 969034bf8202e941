// C[M,N] = epilogue(A[M,K] · W[N,K]^T) for e4m3 operands on the 256x256 workgroup tile: four waves of 128x128 outputs
// (one per SIMD), software-pipelined inside the wave, 16x16x128 MFMAs, fed in slabs of 128 bytes of K so that every
// direct-to-LDS wave-instruction fetches eight whole 128-byte lines. K must be whole slabs.
//
// Measured facts behind the design (MI355X, M=65536, N=3072, K=8192 unless noted):
//  * The same operand stream without any MFMA takes 704 us fetched as whole lines and 1007 us in 64-byte row pieces.
//  * One wave per SIMD has nobody else's instructions to hide its own behind: with per-read and per-load address
//    arithmetic in the loop (about 7 vector ALU instructions per MFMA) the same schedule ran 10 % slower than with
//    addresses that are lane registers + instruction immediates (fragments) and buffer descriptor + fixed lane offset +
//    scalar slab offset (loads). The loop below issues, per slab and wave, 64 MFMAs, 32 LDS reads, 16 loads, 4 vector
//    ALU instructions and scalar bookkeeping.
//  * Under the board's power limit the matrix pipe sustains 4.23 PFLOP/s with 16x16x128 MFMAs and 3.85 with 32x32x64
//    ones on random operand bits (2.10 against 1.90 GHz): the larger K per instruction halves the accumulator traffic.
//    A 16x16x128 MFMA adds its 128 products in one instruction, so sums differ in the last fp32 bits from kernels built
//    on 32x32x64 (64 products per instruction).
//
// Schedule. The ring holds two slabs; LDS is laid out weight rows of stage 0, of stage 1 (32 KB each), then activation
// rows of stage 0, of stage 1, so a stage is bit 15 of an address. Chunk c of row r sits at chunk c ^ (r & 7) ^ ((r >> 3) & 1):
// the 16 lanes that one LDS cycle serves (16 consecutive rows, same chunk) then hit 64 different banks. A wave
// holds the whole slab's fragments (8 weight, 8 activation, 16 rows x 128 bytes = 8 registers each, single-buffered)
// and 64 accumulator tiles acc[wi][xi] of 16x16. Slot u of a slab is one MFMA: slots 0..31 are wi = u / 4 with
// xi = u % 4, slots 32..63 the same wi with xi = 4 + u % 4. A fragment is refilled in place, for the next slab, two
// slots after its last use: X[0..3] in slots 30..33, W[wi] in slot 37 + 4 wi, X[4..7] in slots 62..65 (slots 64 and 65
// are slots 0 and 1 of the next slab). So the reads of slab s+1 run from slot 30 of slab s to slot 1 of slab s+1, and
// the stage of slab s is free from slot 2 of slab s on. Every wave loads 64 activation rows and 64 weight rows of slab
// s+2 per slab, one instruction every third slot from slot 5 to slot 50, and there are two workgroup barriers per slab:
//   P, before slot 4: the wave's reads of slab s have returned; after it the stage of slab s takes the loads of slab s+2;
//   Q, before slot 30: the wave's loads of slab s+1 have landed (the 9 loads issued since may be in flight).
// Every load has at least 43 slots (about 0.9 us) between its issue and the barrier that needs it. Past the end of K
// the loads go through a descriptor of zero length: they move nothing and keep the counts the waits rely on.
#pragma once
#include "gemm_dma_kernel.hpp"

namespace crl {

struct Sp2Cfg {
  static constexpr int BM = 256, BN = 256, WGM = 2, WGN = 2, NW = 4, NT = 256;
  static constexpr int WM = 128, WN = 128;
  static constexpr int ROWB = 128, NSTAGE = 2;
  static constexpr int STAGE_BYTES = (BM + BN) * ROWB;          // 64 KB
  static constexpr int EPI_BYTES = NW * 32 * WN * 4;            // 64 KB
  static constexpr int RING_BYTES = NSTAGE * STAGE_BYTES;       // 128 KB
  static constexpr int STATS_OFF = RING_BYTES + 256;
  static constexpr int LDS_BYTES = STATS_OFF + NW * 2 * WM * 4;
  static_assert(EPI_BYTES <= RING_BYTES, "the epilogue patches reuse the ring");
};

__device__ __forceinline__ void sp_barrier() { asm volatile("s_barrier" ::: "memory"); }

// Slot in which fragment f (0..7 = W[f], 8..15 = X[f - 8]) is refilled: for the next slab; slots 0 and 1: for the slab
// that has just begun.
constexpr int sp2_refill_slot(int f) { return (f < 8 ? 37 + 4 * f : f < 12 ? 30 + (f - 8) : 62 + (f - 12)) & 63; }
// Slot in which load j (0..7 activation rows, 8..15 weight rows) of slab s+2 is issued.
constexpr int sp2_load_slot(int j) { return 5 + 3 * j; }
constexpr int SP2_SLOT_P = 4, SP2_SLOT_Q = 30, SP2_LOADS_BEFORE_Q = 9;
static_assert(sp2_load_slot(SP2_LOADS_BEFORE_Q - 1) < SP2_SLOT_Q && sp2_load_slot(SP2_LOADS_BEFORE_Q) >= SP2_SLOT_Q, "count of loads ahead of barrier Q");

template <int OUT_DT, int RES_NORM = 0>
__global__ void __launch_bounds__(Sp2Cfg::NT) gemm_sp2_kernel(const GemmArgs a) {
  typedef Sp2Cfg Cfg;
  constexpr int BM = Cfg::BM, BN = Cfg::BN;
  extern __shared__ __align__(16) uint8_t smem[];

  // (the wave index as a scalar: everything derived from it, LDS destinations and global bases, stays in scalar registers)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

  const int nslab = a.K / Cfg::ROWB;        // the launcher sends only K % 128 == 0 here

  if constexpr (RES_NORM != 0) {
    // Row statistics of this wave's 128 rows, landed outside the ring: the wave's oldest load, covered by its first wait.
    int m = m0 + wm * Cfg::WM + 2 * lane;
    m = m + 1 < a.M ? m : 0;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.res_stats + 2 * (long)m),
                                     (__attribute__((address_space(3))) void*)(smem + Cfg::STATS_OFF + wave * (2 * Cfg::WM * 4)), 16, 0, 0);
  }

  // Loader role: wave w fills activation rows [64w, +64) and weight rows [64w, +64) of a stage, 8 rows per
  // wave-instruction, eight 16-byte chunks per row, the swizzle applied on the global side (lane 8r + c of instruction i
  // fetches chunk c ^ r ^ (i & 1) of its row). Buffer addressing: descriptor base = tile origin (scalar), lane offset (vector, fixed), slab
  // offset (scalar): no vector ALU work per load. The rows a tile touches end at most 256 * ld bytes behind its origin.
  uint32_t voff_w[8], voff_x[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = wave * 64 + 8 * i + (lane >> 3);
    const int kch = ((lane & 7) ^ (lane >> 3) ^ (i & 1)) << 4;
    const int rw = r < a.N - n0 ? r : a.N - n0 - 1, rx = r < a.M - m0 ? r : a.M - m0 - 1;
    voff_w[i] = (uint32_t)rw * (uint32_t)a.ldw + kch;
    voff_x[i] = (uint32_t)rx * (uint32_t)a.lda + kch;
  }
  auto make_rsrc = [&](const void* base, long rows, long ld) {
    const long span = (rows < 256 ? rows : 256) * ld;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)(span < 0x7fffffffL ? span : 0x7fffffffL), 0x00020000);
  };
  const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(reinterpret_cast<const uint8_t*>(a.W) + (long)n0 * a.ldw, a.N - n0, a.ldw);
  const __amdgpu_buffer_rsrc_t rsrc_x = make_rsrc(reinterpret_cast<const uint8_t*>(a.A) + (long)m0 * a.lda, a.M - m0, a.lda);
  const __amdgpu_buffer_rsrc_t rsrc_none = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(a.A), 0, 0, 0x00020000);
  const uint32_t lds_w0 = wave * 64 * Cfg::ROWB, lds_x0 = 65536u + wave * 64 * Cfg::ROWB;   // stage 0
  // Load j of a slab: 0..7 activation rows, 8..15 weight rows (in that order: the counted waits rely on it).
  auto load_one = [&](int slab, bool real, auto jc) {
    constexpr int j = decltype(jc)::value;
    constexpr int i = j & 7;
    const uint32_t dst0 = (j < 8 ? lds_x0 : lds_w0) ^ ((slab & 1) << 15);
    const __amdgpu_buffer_rsrc_t r = real ? (j < 8 ? rsrc_x : rsrc_w) : rsrc_none;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)(smem + dst0 + i * 1024), 16,
                                             (int)(j < 8 ? voff_x[i] : voff_w[i]), slab * Cfg::ROWB, 0, 0);
  };
  auto issue_loads = [&](int slab, bool real) { static_for<0, 16>([&](auto jc) { load_one(slab, real, jc); }); };

  f32x4_t acc[8][8];   // [wi][xi]
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
  // The MFMAs below are inline assembly, so the compiler does not know that a matrix instruction must not read an
  // accumulation register in the cycles right after a v_accvgpr_write to it, and it is free to sink the zeroing down to
  // the first MFMA. These statements depend on every accumulator and every MFMA depends on them: the zeroing is
  // complete, and some cycles old, before the first MFMA issues.
#pragma unroll
  for (int i = 0; i < 8; ++i)
    asm volatile("s_nop 3" : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]), "+a"(acc[i][4]), "+a"(acc[i][5]), "+a"(acc[i][6]), "+a"(acc[i][7]));

  // Fragment addresses: lane l holds K bytes [32 (l / 16), +32) of row l % 16 of a 16-row fragment, i.e. chunks
  // (2 (l / 16) + half) ^ swizzle(row) of its row, and the swizzle depends on l % 16 only. Two lane addresses per operand
  // (one per half) plus the immediate 2048 i for fragment i cover every read of a stage.
  const int l15 = lane & 15, qk = lane >> 4;
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)smem);   // LDS address of the ring
  uint32_t wb[2], xb[2];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    wb[half] = lds0 + (wn * Cfg::WN + l15) * Cfg::ROWB + (((2 * qk + half) ^ (l15 & 7) ^ (l15 >> 3)) << 4);
    xb[half] = lds0 + 65536 + (wm * Cfg::WM + l15) * Cfg::ROWB + (((2 * qk + half) ^ (l15 & 7) ^ (l15 >> 3)) << 4);
  }
  auto flip_stage = [&]() {
#pragma unroll
    for (int half = 0; half < 2; ++half) { wb[half] ^= 32768u; xb[half] ^= 32768u; }
  };
  const bool wave_active = (m0 + wm * Cfg::WM < a.M) && (n0 + wn * Cfg::WN < a.N);

  i32x8_t wf[8], xf[8];
  // Fragment f: 0..7 = W[f], 8..15 = X[f - 8]; both 16-byte halves, from the stage the address registers point at.
  auto read_frag = [&](auto fc) {
    constexpr int f = decltype(fc)::value;
    constexpr bool is_w = f < 8;
    constexpr int idx = f & 7;
    const i32x4_t lo = *reinterpret_cast<const __attribute__((address_space(3))) i32x4_t*>((is_w ? wb[0] : xb[0]) + idx * 16 * Cfg::ROWB);
    const i32x4_t hi = *reinterpret_cast<const __attribute__((address_space(3))) i32x4_t*>((is_w ? wb[1] : xb[1]) + idx * 16 * Cfg::ROWB);
    i32x8_t& dst = is_w ? wf[idx] : xf[idx];
    dst = i32x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  // The accumulators are pinned to the accumulation registers by the operand constraint of the inline-assembly MFMAs. The
  // instruction is the e4m3 x e4m3 form (no format modifiers).
  auto mfma = [&](f32x4_t& c, const i32x8_t& w, const i32x8_t& x) {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(w), "v"(x));
  };
  // Slot u of slab s; full scheduling barriers hold the order. `real`: slab s+2 exists.
  auto slot = [&](int s, bool real, auto uc) {
    constexpr int u = decltype(uc)::value;
    constexpr int wi = (u & 31) >> 2, xi = (u & 3) + 4 * (u >> 5);
    if constexpr (u == 2) flip_stage();   // the address registers now point at the stage of slab s+1
    if constexpr (u == SP2_SLOT_P) {
      __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): this wave's reads of slab s have returned
      sp_barrier();
    }
    if constexpr (u == SP2_SLOT_Q) {
      wait_vmcnt<SP2_LOADS_BEFORE_Q>();     // this wave's loads of slab s+1 have landed
      sp_barrier();
    }
    mfma(acc[wi][xi], wf[wi], xf[xi]);
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, 16>([&](auto fc) {
      if constexpr (sp2_refill_slot(decltype(fc)::value) == u) read_frag(fc);
    });
    static_for<0, 16>([&](auto jc) {
      if constexpr (sp2_load_slot(decltype(jc)::value) == u) load_one(s + 2, real, jc);
    });
    __builtin_amdgcn_sched_barrier(0);
  };

  issue_loads(0, true);
  issue_loads(1, nslab > 1);
  wait_vmcnt<16>();
  sp_barrier();

  if (wave_active) {
    // Slab 0: every fragment but the three that slots 0 and 1 fetch, then its slots 0-3. The loop body runs from slot
    // 4 of a slab to slot 3 of the next, so that the wait the compiler puts at a loop header (every LDS read returned)
    // coincides with the one barrier P needs anyway.
    static_for<0, 16>([&](auto fc) {
      if constexpr (sp2_refill_slot(decltype(fc)::value) > 1) read_frag(fc);
    });
    static_for<0, 4>([&](auto uc) { slot(0, false, uc); });
    for (int s = 0; s < nslab; ++s) {
      const bool real = s + 2 < nslab;
      static_for<4, 64>([&](auto uc) { slot(s, real, uc); });
      if (s + 1 < nslab) static_for<0, 4>([&](auto uc) { slot(s + 1, false, uc); });
    }
  } else {
    // A wave whose 128x128 part lies wholly outside C: its share of the loads and both barriers of every slab.
    for (int s = 0; s < nslab; ++s) {
      const bool real = s + 2 < nslab;
      sp_barrier();
      static_for<0, SP2_LOADS_BEFORE_Q>([&](auto jc) { load_one(s + 2, real, jc); });
      wait_vmcnt<SP2_LOADS_BEFORE_Q>();
      sp_barrier();
      static_for<SP2_LOADS_BEFORE_Q, 16>([&](auto jc) { load_one(s + 2, real, jc); });
    }
  }
  wait_vmcnt<0>();
  // The MFMAs above are opaque to the compiler's hazard handling: let the last of them retire before the epilogue reads
  // the accumulators.
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  sp_barrier();   // every wave is done with the ring before it becomes epilogue scratch

  gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT, RES_NORM>(a, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                                     m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane,
                                                     reinterpret_cast<float*>(smem + Cfg::STATS_OFF) + wave * (2 * Cfg::WM));
}

template <int OUT_DT, int RES_NORM = 0>
static hipError_t launch_sp2(const GemmArgs& a, hipStream_t st) {
  static std::atomic<bool> attr_set[16] = {};
  hipError_t e = hipSuccess;
  // Whole slabs of K only, and lane offsets inside a tile's 256 rows that fit 32 bits.
  if (a.K % Sp2Cfg::ROWB != 0 || a.K <= 0 || (long)a.lda * 256 >= (1L << 31) || (long)a.ldw * 256 >= (1L << 31)) return hipErrorInvalidValue;
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_sp2_kernel<OUT_DT, RES_NORM>;
  if (!attr_set[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Sp2Cfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles = ((a.M + Sp2Cfg::BM - 1) / Sp2Cfg::BM) * ((a.N + Sp2Cfg::BN - 1) / Sp2Cfg::BN);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(Sp2Cfg::NT), Sp2Cfg::LDS_BYTES, st, a);
  return hipGetLastError();
}

}  // namespace crl
