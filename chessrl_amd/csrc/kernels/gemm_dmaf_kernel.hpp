// C[M,N] = epilogue(A[M,K] · W[N,K]^T), e4m3 or 16-bit operands, K a whole number of 128-byte slabs: the eight-wave in-step
// 256x256 kernel of gemm_dma_kernel.hpp with its address arithmetic taken out of the main loop. There a wave issues,
// per slab of 16 MFMAs, 24 LDS reads and 8 loads, another 85 vector ALU instructions: a 64-bit add, a compare and two
// selects per load (slab offset, K tail from a block of zeros), an add per fragment read. Here
//  * LDS is laid out weight rows of stage 0, of stage 1 (32 KB each), then activation rows of stage 0, of stage 1, so a
//    stage is bit 15 of an address: a fragment address is one of four lane registers per operand plus an instruction
//    immediate, and all eight registers change stage with one XOR each per slab;
//  * loads use buffer addressing: descriptor base = tile origin (scalar), a fixed lane offset, the slab offset in a
//    scalar register; past the end of K they go through a descriptor of zero length (they move nothing and keep the
//    instruction stream free of branches).
// Same tile walk, same K order and same epilogue as gemm_dma_kernel.hpp: the outputs are bit-equal.
#pragma once
#include "gemm_dma_kernel.hpp"

namespace crl {

struct DmafCfg {
  static constexpr int BM = 256, BN = 256, WGM = 2, WGN = 4, NW = 8, NT = 512;
  static constexpr int WM = 128, WN = 64, TM = 4, TN = 2;
  static constexpr int ROWB = 128, LOADS = 8;
  static constexpr int RING_BYTES = 2 * (BM + BN) * ROWB;   // 128 KB
  static constexpr int EPI_BYTES = NW * 32 * WN * 4;        // 64 KB: the two weight stages
  static constexpr int STATS_OFF = RING_BYTES + 256;        // behind the landing strip of the L2 touches
  static constexpr int COLS_OFF = STATS_OFF + NW * 2 * WM * 4;   // per-column epilogue constants: [wave][bias, gain, offset][WN]
  static constexpr int LDS_BYTES = COLS_OFF + NW * 3 * WN * 4;
  // XTRA instances: up to 32 weight rows beyond the last tile column, two stages of 4 KB on an 8 KB boundary (a stage is
  // bit 12 of an address there).
  static constexpr int XTRA_OFF = (LDS_BYTES + 8191) / 8192 * 8192;
  static constexpr int LDS_BYTES_XTRA = XTRA_OFF + 8192;
  static_assert(LDS_BYTES_XTRA <= 160 * 1024, "LDS of a CU");
};

// The tile walk's constants, worked out once on the host: the walk divides a workgroup index by six launch constants,
// and as generic integer divisions those were most of the ~410 instructions a workgroup issued before its first load.
// q = n / d for n, d < 65536 is the high half of n * ceil(2^32 / d) (d = 1: n itself).
struct DmafWalk {
  int tiles_n, grouped, wb, extra, big;
  uint32_t m_tn, m_8tn, m_8w1, m_8w0, m_w1, m_w0;   // magics of tiles_n, 8 tiles_n, 8 (wb+1), 8 wb, wb+1, wb
};
inline uint32_t dmaf_magic(uint32_t d) { return d <= 1 ? 0u : (uint32_t)(((1ull << 32) + d - 1) / d); }
__device__ __forceinline__ int dmaf_div(int n, uint32_t magic) { return magic ? (int)__umulhi((uint32_t)n, magic) : n; }
inline DmafWalk dmaf_walk(int M, int N, bool fp8) {
  DmafWalk w{};
  const int tiles_n = (N + 255) / 256, tiles_m = (M + 255) / 256;
  w.tiles_n = tiles_n;
  // (16-bit operands keep the plain row-major order unless the columns divide by four, as in gemm_dma_kernel.hpp)
  w.grouped = tiles_m % 8 == 0 && (fp8 || tiles_n % 4 == 0);
  const int ngrp = (tiles_n + 3) >> 2;
  w.wb = tiles_n / ngrp;
  w.extra = tiles_n - w.wb * ngrp;
  w.big = 8 * (w.wb + 1) * w.extra;
  w.m_tn = dmaf_magic(tiles_n); w.m_8tn = dmaf_magic(8 * tiles_n);
  w.m_8w1 = dmaf_magic(8 * (w.wb + 1)); w.m_8w0 = dmaf_magic(8 * w.wb);
  w.m_w1 = dmaf_magic(w.wb + 1); w.m_w0 = dmaf_magic(w.wb);
  return w;
}

// LEAN: the epilogue without its edge and type guards (gemm_epilogue's LEAN; dmaf_lean_ok says when).
// XTRA: the tile columns cover the first nsplit columns only (nsplit a multiple of 256), and the workgroups of the last
// tile column also compute the up to 32 columns behind them (the second output of a column split): every wave one more
// 32x32 MFMA tile per K step, rows [32 wn, +32) of its 128, on weight rows that four more loads per slab bring in. Same
// operands in the same K order as a tile column of their own would use (bit-equal), without that column's second pass
// over the activations.
template <int IN_DT, int OUT_DT, int RES_NORM = 0, int LEAN = 0, int XTRA = 0>
__global__ void __launch_bounds__(DmafCfg::NT, 2) gemm_dmaf_kernel(const GemmArgs a, const int pf, const DmafWalk wk) {
  typedef DmafCfg Cfg;
  constexpr int ESZ = IN_DT == DT_FP8 ? 1 : 2;                      // bytes per operand element
  constexpr int KSTEPS = Cfg::ROWB / (IN_DT == DT_FP8 ? 64 : 32);   // MFMA K steps per slab
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, LOADS = Cfg::LOADS;
  extern __shared__ __align__(16) uint8_t smem[];

  // (the wave index as a scalar: everything derived from it, LDS destinations and descriptors, stays in scalar registers)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % Cfg::WGM, wn = wave / Cfg::WGM;
  const int lr = lane & 31, g = lane >> 5;

  const int tiles_n = wk.tiles_n;
  const int nblk = gridDim.x;
  // Tiles are walked from the last row of tiles to the first. The kernels around a product (norms, attention) walk their
  // rows upwards, so this product starts on the rows its producer wrote last and ends on the rows its consumer reads first,
  // which are the ones the memory-side cache still holds (measured on a 4096-position pass: -0.4 ms over its 60 launches).
  int pid = nblk - 1 - (int)blockIdx.x;
  {
    const int per = nblk >> 3;
    if (pid < (per << 3)) pid = (pid & 7) * per + (pid >> 3);
  }
  // Tile order inside an XCD's range: groups of 8 x w tiles (M x N), w = 3 or 4, as in gemm_dma_kernel.hpp.
  int tile_m = dmaf_div(pid, wk.m_tn), tile_n = pid - tile_m * tiles_n;
  int grp_w = 4, grp_q = tile_n & 3;
  if (wk.grouped) {
    constexpr int GM = 8;
    const int wb = wk.wb, extra = wk.extra, big = wk.big;
    const int sr = dmaf_div(pid, wk.m_8tn), rem = pid - sr * (GM * tiles_n);
    int gi, r2, rq;
    if (rem < big) { grp_w = wb + 1; gi = dmaf_div(rem, wk.m_8w1); r2 = rem - gi * GM * grp_w; rq = dmaf_div(r2, wk.m_w1); }
    else { grp_w = wb; const int rem2 = rem - big; gi = dmaf_div(rem2, wk.m_8w0); r2 = rem2 - gi * GM * wb; rq = dmaf_div(r2, wk.m_w0); gi += extra; }
    grp_q = r2 - rq * grp_w;
    tile_m = sr * GM + rq;
    tile_n = gi * wb + (gi < extra ? gi : extra) + grp_q;
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int nslab = a.K * ESZ / Cfg::ROWB;  // the launcher sends only whole slabs of K here

  // Loader role: waves 0-3 fill weight rows [64w, +64) of a stage, waves 4-7 activation rows [64(w-4), +64): 8 rows per
  // wave-instruction, eight 16-byte chunks per row, the swizzle applied on the global side (row 8 i + lane / 8 of the
  // wave's 64 has swizzle (lane / 8) ^ i).
  const bool loads_a = wave >= 4;
  const int rbase = (wave & 3) * 64;
  const int ld = (loads_a ? a.lda : a.ldw) * ESZ;   // row stride in bytes
  const int rows_left = loads_a ? a.M - m0 : a.N - n0;
  uint32_t voff[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    int r = rbase + 8 * i + (lane >> 3);
    r = r < rows_left ? r : rows_left - 1;
    voff[i] = (uint32_t)r * (uint32_t)ld + (((lane & 7) ^ (lane >> 3) ^ i) << 4);
  }
  auto make_rsrc = [&](const void* base, long rows, long ldb) {
    const long span = (rows < 256 ? rows : 256) * ldb;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)(span < 0x7fffffffL ? span : 0x7fffffffL), 0x00020000);
  };
  const __amdgpu_buffer_rsrc_t rsrc_w = make_rsrc(reinterpret_cast<const uint8_t*>(a.W) + (long)n0 * a.ldw * ESZ, a.N - n0, (long)a.ldw * ESZ);
  const __amdgpu_buffer_rsrc_t rsrc_x = make_rsrc(reinterpret_cast<const uint8_t*>(a.A) + (long)m0 * a.lda * ESZ, a.M - m0, (long)a.lda * ESZ);
  const __amdgpu_buffer_rsrc_t rsrc_none = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(a.A), 0, 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_mine = loads_a ? rsrc_x : rsrc_w;
  const uint32_t lds_load0 = (loads_a ? 65536u : 0u) + rbase * Cfg::ROWB;   // stage 0
  auto issue_one = [&](int slab, const __amdgpu_buffer_rsrc_t& r, auto ic) {
    constexpr int i = decltype(ic)::value;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)(smem + (lds_load0 ^ ((slab & 1) << 15)) + i * 1024), 16,
                                             (int)voff[i], slab * Cfg::ROWB, 0, 0);
  };
  // XTRA: waves 0-3 bring in eight of the extra weight rows each.
  const bool extra = XTRA != 0 && tile_n == tiles_n - 1;
  const int n_x = n0 + BN;   // first extra column
  uint32_t voff_x = 0;
  __amdgpu_buffer_rsrc_t rsrc_xw = rsrc_none;
  if constexpr (XTRA != 0) {
    if (extra && !loads_a) {
      const int rows_x = a.N - n_x < 32 ? a.N - n_x : 32;
      int r = 8 * wave + (lane >> 3);
      r = r < rows_x ? r : rows_x - 1;
      voff_x = (uint32_t)r * (uint32_t)ld + (((lane & 7) ^ (lane >> 3) ^ wave) << 4);
      rsrc_xw = make_rsrc(reinterpret_cast<const uint8_t*>(a.W) + (long)n_x * a.ldw * ESZ, rows_x, (long)a.ldw * ESZ);
    }
  }
  auto issue_extra = [&](int slab, bool live) {
    if constexpr (XTRA != 0) {
      if (extra && !loads_a)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(live ? rsrc_xw : rsrc_none,
                                                 (__attribute__((address_space(3))) void*)(smem + Cfg::XTRA_OFF + ((slab & 1) << 12) + wave * 1024), 16,
                                                 (int)voff_x, slab * Cfg::ROWB, 0, 0);
    }
  };
  // The first slab is requested as early as its addresses exist; everything else the prologue sets up follows.
  static_for<0, LOADS>([&](auto ic) { issue_one(0, rsrc_mine, ic); });
  issue_extra(0, true);
  __builtin_amdgcn_sched_barrier(0);

  // The per-column constants of the epilogue (bias; gain and offset of a residual normalised on the fly) for this wave's
  // 64 columns, one column per lane, landed outside the ring: requested first, in LDS long before the epilogue asks.
  // Columns past N repeat the last one; nothing of theirs is stored.
  {
    int n = n0 + wn * Cfg::WN + lane;
    n = n < a.N ? n : a.N - 1;
    uint8_t* cols = smem + Cfg::COLS_OFF + wave * (3 * Cfg::WN * 4);
    if (a.bias)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.bias + n), (__attribute__((address_space(3))) void*)cols, 4, 0, 0);
    if constexpr (RES_NORM != 0) {
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.res_gamma + n),
                                       (__attribute__((address_space(3))) void*)(cols + Cfg::WN * 4), 4, 0, 0);
      if (a.res_beta)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.res_beta + n),
                                         (__attribute__((address_space(3))) void*)(cols + 2 * Cfg::WN * 4), 4, 0, 0);
    }
  }
  if constexpr (RES_NORM != 0) {
    // Statistics of this wave's 128 rows (two rows = 16 bytes per lane), requested before anything else and landed
    // outside the ring.
    int m = m0 + wm * Cfg::WM + 2 * lane;
    m = m + 1 < a.M ? m : 0;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.res_stats + 2 * (long)m),
                                     (__attribute__((address_space(3))) void*)(smem + Cfg::STATS_OFF + wave * (2 * Cfg::WM * 4)), 16, 0, 0);
  }


  // L2 touches, as in gemm_dma_kernel.hpp: wave 0 touches its share of the activation lines of a slab `pf` slabs before
  // anybody loads it, wave 1 its share of the weight lines; one dword per 128-byte line into an LDS strip nobody reads.
  uint32_t pf_off = 0;
  int pf_n = 0, pf_step = 0;
  if (pf > 0 && wave < 2) {
    if (wave == 0) {
      pf_n = grp_w >= 4 ? 1 : grp_w >= 2 ? 2 : 4;   // ceil(4 / grp_w)
      int r = ((grp_q * pf_n) & 3) * 64 + lane;
      r = r < a.M - m0 ? r : a.M - m0 - 1;
      pf_off = (uint32_t)r * (uint32_t)(a.lda * ESZ);
      pf_step = (m0 + 256 <= a.M) ? 64 * a.lda * ESZ : 0;
    } else {
      pf_n = 1;
      int r = (tile_m & 7) * 32 + (lane & 31);
      r = r < a.N - n0 ? r : a.N - n0 - 1;
      pf_off = (uint32_t)r * (uint32_t)(a.ldw * ESZ) + (lane >> 5) * 64;
    }
  }
  const __amdgpu_buffer_rsrc_t rsrc_pf = wave == 0 ? rsrc_x : rsrc_w;
  auto prefetch = [&](int slab) {
    if (pf_n > 0 && slab < nslab) {
      for (int i = 0; i < pf_n; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_pf, (__attribute__((address_space(3))) void*)(smem + Cfg::RING_BYTES), 4,
                                                 (int)pf_off, slab * Cfg::ROWB + i * pf_step, 0, 0);
    }
  };

  f32x16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Fragment addresses. A lane's 16-byte piece of row 32 t + lr of a wave's block sits at chunk c ^ swizzle(row) with
  // c = 4 ks + half + 2g for e4m3 (two pieces per K step of 64 bytes) and c = 2 ks + g for 16-bit operands (one piece
  // per K step of 32 bytes), and swizzle(row) = swizzle(lr) ^ 4 (t & 1). With L = (2g or g) ^ swizzle(lr) the chunk is
  // Kc ^ L for a compile-time Kc that takes four values (0, 1, 4, 5 or 0, 2, 4, 6): four lane addresses per operand
  // plus the immediate 4096 t cover every read of a stage.
  const int L0 = (IN_DT == DT_FP8 ? 2 * g : g) ^ lds_swizzle(lr);
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)smem);
  uint32_t wb[4], xb[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int kc = IN_DT == DT_FP8 ? ((k & 1) | ((k >> 1) << 2)) : 2 * k;
    wb[k] = lds0 + (wn * Cfg::WN + lr) * Cfg::ROWB + ((kc ^ L0) << 4);
    xb[k] = lds0 + 65536 + (wm * Cfg::WM + lr) * Cfg::ROWB + ((kc ^ L0) << 4);
  }
  auto read_piece = [&](bool is_w, int t, int ks, int half) -> i32x4_t {
    const int kc = (IN_DT == DT_FP8 ? 4 * ks + half : 2 * ks) ^ (4 * (t & 1));
    const int k = IN_DT == DT_FP8 ? ((kc & 1) | ((kc >> 2) << 1)) : kc >> 1;
    return *reinterpret_cast<const __attribute__((address_space(3))) i32x4_t*>((is_w ? wb[k] : xb[k]) + t * 32 * Cfg::ROWB);
  };

  // XTRA: fragment addresses of the extra weight rows (row lr of 32) and of this wave's rows [32 wn, +32) of its activation block.
  uint32_t eb[4] = {0, 0, 0, 0};
  f32x16_t accx;
#pragma unroll
  for (int r = 0; r < 16; ++r) accx[r] = 0.f;
  const uint32_t xrow_off = (uint32_t)wn * 32 * Cfg::ROWB;
  if constexpr (XTRA != 0) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int kc = (k & 1) | ((k >> 1) << 2);
      eb[k] = lds0 + Cfg::XTRA_OFF + lr * Cfg::ROWB + ((kc ^ L0) << 4);
    }
  }

  // A wave whose 128x64 part lies wholly outside C still takes its share of the loads and every barrier.
  const bool wave_active = (m0 + wm * Cfg::WM < a.M) && (n0 + wn * Cfg::WN < a.N);


  for (int s0 = 1; s0 < 1 + pf; ++s0) prefetch(s0);

  for (int slab = 0; slab < nslab; ++slab) {
    wait_vmcnt<0>();
    __syncthreads();
    const __amdgpu_buffer_rsrc_t rnext = slab + 1 < nslab ? rsrc_mine : rsrc_none;
    prefetch(slab + 1 + pf);
    if (!wave_active) {
      static_for<0, LOADS>([&](auto ic) { issue_one(slab + 1, rnext, ic); });
      issue_extra(slab + 1, slab + 1 < nslab);
      continue;
    }
    static_for<0, KSTEPS>([&](auto ksc) {
      constexpr int ks = decltype(ksc)::value;
      Frag<IN_DT> wf[TN], xf[TM];
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        wf[tn].lo = read_piece(true, tn, ks, 0);
        if constexpr (IN_DT == DT_FP8) wf[tn].hi = read_piece(true, tn, ks, 1);
      }
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) {
        xf[tm].lo = read_piece(false, tm, ks, 0);
        if constexpr (IN_DT == DT_FP8) xf[tm].hi = read_piece(false, tm, ks, 1);
      }
      static_for<0, TN * TM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        constexpr int tn = i / TM, tm = i % TM;
        acc[tn][tm] = mfma_frag<IN_DT>(wf[tn], xf[tm], acc[tn][tm]);
        // The next slab's loads go out one at a time, one behind each of the slab's first eight MFMAs, held in place by
        // scheduling barriers: the last of them then has the rest of the slab's MFMAs in which to land before the wave
        // waits for it. Measured on the products of a large pass, e4m3: spread over all sixteen MFMAs (one behind every
        // second) +3.8 %, starting one MFMA earlier or two later, or two loads behind each of four MFMAs, +1 %; 16-bit
        // operands (32 MFMAs per slab): all eight at the head of the slab +2.6 %, behind every second of the first sixteen +2.6 %.
        if constexpr (ks == 0) {
          __builtin_amdgcn_sched_barrier(0);
          issue_one(slab + 1, rnext, std::integral_constant<int, i>{});
          if constexpr (i == TN * TM - 1) issue_extra(slab + 1, slab + 1 < nslab);
          __builtin_amdgcn_sched_barrier(0);
        }
      });
      if constexpr (XTRA != 0 && IN_DT == DT_FP8) {
        if (extra) {
          constexpr int k0 = (4 * ks) & 1 | (((4 * ks) >> 2) << 1), k1 = ((4 * ks + 1) & 1) | (((4 * ks + 1) >> 2) << 1);
          Frag<IN_DT> wfx, xfx;
          wfx.lo = *reinterpret_cast<const __attribute__((address_space(3))) i32x4_t*>(eb[k0]);
          wfx.hi = *reinterpret_cast<const __attribute__((address_space(3))) i32x4_t*>(eb[k1]);
          // (rows 32 t + lr of a block carry the swizzle of lr with bit 2 flipped for odd t: the other pair of lane addresses)
          const uint32_t xa0 = ((wn & 1) ? xb[k0 ^ 2] : xb[k0]) + xrow_off, xa1 = ((wn & 1) ? xb[k1 ^ 2] : xb[k1]) + xrow_off;
          xfx.lo = *reinterpret_cast<const __attribute__((address_space(3))) i32x4_t*>(xa0);
          xfx.hi = *reinterpret_cast<const __attribute__((address_space(3))) i32x4_t*>(xa1);
          accx = mfma_frag<IN_DT>(wfx, xfx, accx);
        }
      }
    });
    if constexpr (XTRA != 0) {
#pragma unroll
      for (int k = 0; k < 4; ++k) eb[k] ^= 4096u;
    }
    // The address registers follow the ring to the other stage.
#pragma unroll
    for (int k = 0; k < 4; ++k) { wb[k] ^= 32768u; xb[k] ^= 32768u; }
  }

  wait_vmcnt<0>();
  __syncthreads();  // every wave is done with the ring (and the empty loads past the end have retired) before it becomes epilogue scratch

  gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT, RES_NORM, LEAN>(a, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                                     m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane,
                                                     reinterpret_cast<float*>(smem + Cfg::STATS_OFF) + wave * (2 * Cfg::WM),
                                                     reinterpret_cast<const float*>(smem + Cfg::COLS_OFF) + wave * (3 * Cfg::WN));
  if constexpr (XTRA != 0) {
    if (extra) {
      // The extra columns' 32x32 tile of this wave, through the same patch (its bias comes from global memory).
      f32x16_t ax[1][1];
      ax[0][0] = accx;
      wave_lds_fence();
      gemm_epilogue<32, 32, OUT_DT, 0, LEAN>(a, ax, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                             m0 + wm * Cfg::WM + wn * 32, n_x, lane);
    }
  }
}

// 0: the general epilogue; 1: without edge, alignment and type guards; 2: with the call's shape fixed at compile time as well
// (see gemm_epilogue), which is what the products of a large forward pass are.
inline int dmaf_lean_level(const GemmArgs& a, int out_dt, bool res_norm);
inline bool dmaf_lean_ok(const GemmArgs& a) {
  return a.M % DmafCfg::BM == 0 && a.vec_ok && a.N % 8 == 0 && a.nsplit % 8 == 0 && !a.amax && a.res_rows == 0 && !a.ln_out &&
         (!a.res || a.res_dtype == DT_BF16);
}

inline int dmaf_lean_level(const GemmArgs& a, int out_dt, bool res_norm) {
  if (!dmaf_lean_ok(a)) return 0;
  if (!a.stream_out) return 1;
  if (res_norm) return a.act == ACT_NONE ? 2 : 1;
  if (a.res || a.alpha != 1.f) return 1;
  return a.act == (out_dt == DT_FP8 ? ACT_MISH : ACT_NONE) ? 2 : 1;
}

// Whether the XTRA instance serves this call: a column split at a multiple of 256 with at most 32 columns behind it.
inline bool dmaf_xtra_ok(const GemmArgs& a) {
  return a.C2 != nullptr && a.nsplit >= 256 && a.nsplit % 256 == 0 && a.N > a.nsplit && a.N - a.nsplit <= 32;
}

template <int IN_DT, int OUT_DT, int RES_NORM = 0, int LEAN = 0, int XTRA = 0>
static hipError_t launch_dmaf(const GemmArgs& a, hipStream_t st) {
  static std::atomic<bool> attr_set[16] = {};
  hipError_t e = hipSuccess;
  // Whole slabs of K only, and lane offsets inside a tile's 256 rows that fit 31 bits.
  constexpr int ESZ = IN_DT == DT_FP8 ? 1 : 2;
  if ((a.K * ESZ) % DmafCfg::ROWB != 0 || a.K <= 0 || (long)a.lda * ESZ * 256 >= (1L << 31) || (long)a.ldw * ESZ * 256 >= (1L << 31)) return hipErrorInvalidValue;
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_dmaf_kernel<IN_DT, OUT_DT, RES_NORM, LEAN, XTRA>;
  constexpr int LDS = XTRA ? DmafCfg::LDS_BYTES_XTRA : DmafCfg::LDS_BYTES;
  if (!attr_set[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int Nt = XTRA ? a.nsplit : a.N;   // columns the tile columns cover
  const int tiles_n = (Nt + DmafCfg::BN - 1) / DmafCfg::BN;
  const int tiles = ((a.M + DmafCfg::BM - 1) / DmafCfg::BM) * tiles_n;
  // (the L2 touches pay for e4m3 operands only: the 16-bit instances lose 2-6 % with them)
  const int pf = (IN_DT == DT_FP8 && tiles_n % 4 == 0 && (long)a.K >= 8 * DmafCfg::ROWB) ? 2 : 0;
  if (tiles >= 65536) return hipErrorInvalidValue;   // (the walk's divisions are exact below that; the caller has another kernel)
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(DmafCfg::NT), LDS, st, a, pf, dmaf_walk(a.M, Nt, IN_DT == DT_FP8));
  return hipGetLastError();
}

}  // namespace crl
