// C[M,N] = epilogue(A[M,K] · W[N,K]^T) on a 128x128, 64x64 or 32x32 workgroup tile fed by direct-to-LDS loads through a
// ring of stages, K a whole number of 128-byte slabs: the kernel for products of at most 256 tiles (the products of a
// batch of 1 to 64 positions), where every CU holds one workgroup and nothing but the kernel's own pipeline hides memory
// latency. The register-staged kernels of gemm.hip keep one slab in flight (128x128: 1.3 us per slab for 0.27 us of MFMA
// work); here all stages but one are in flight (three of four on the 128x128 tile, fifteen of sixteen on the 32x32
// tile), waited for with counted waits, and the addressing is that of gemm_dmaf_kernel.hpp: fragment addresses are lane
// registers plus instruction immediates, loads go through buffer descriptors with the slab offset in a scalar register,
// and past the end of K through a descriptor of zero length so that every slab issues the same instructions and the
// counts hold. Same K order and epilogue as the other tiled kernels: bit-equal results.
#pragma once
#include "gemm_dmaf_kernel.hpp"

namespace crl {

// BT = 128: eight waves of 64x32 on a 128x128 tile (8 MFMAs per 12 fragment reads and slab), four stages of 32 KB. Four
// waves of 64x64 (16 MFMAs per 16 reads) issue fewer instructions but have half as many loads and MFMA streams in
// flight: measured 4 to 5 % slower on bf16 and 6 to 10 % on e4m3 (M=4096, N=1024, K=1024: 17.0 -> 16.3 us bf16, 10.4 -> 9.3 us e4m3).
// BT = 64: four waves of 32x32 on a 64x64 tile, eight stages of 16 KB, for products of at most a few hundred such tiles
// (a forward pass over a few positions), where the time is the latency of walking K and the seven slabs in flight hide it.
// BT = 32: one wave computes a 32x32 tile and fills the weight rows, a second wave only fills the activation rows; sixteen
// stages of 8 KB, so the whole of K = 1024 16-bit elements is in flight at once: one position's products, spread over
// four times as many CUs as on 64x64 tiles.
// Either way a wave fills 32 of a stage's rows with four load instructions.
template <int BT>
struct DmamCfgT {
  static_assert(BT == 128 || BT == 64 || BT == 32, "three tile sizes");
  static constexpr int BM = BT, BN = BT, WGM = BT >= 64 ? 2 : 1, WGN = BT >= 64 ? BT / 32 : 1;
  static constexpr int NCOMP = WGM * WGN;                       // waves that compute
  static constexpr int NW = BT >= 64 ? NCOMP : 2, NT = 64 * NW; // waves that load: all of them
  static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
  static constexpr int ROWB = 128, NSTAGE = 512 / BT;
  static constexpr int ROWS_PER_WAVE = 2 * BM / NW;             // 32
  static constexpr int LOADS = ROWS_PER_WAVE / 8;               // 4
  static constexpr int PART_BYTES = NSTAGE * BN * ROWB;         // 64 KB: the weight rows of all stages, then the activation rows
  static constexpr int RING_BYTES = 2 * PART_BYTES;             // 128 KB
  static constexpr int EPI_BYTES = NCOMP * 32 * WN * 4;         // 32 KB (16 KB, 4 KB)
  static constexpr int STATS_OFF = RING_BYTES + 256;
  static constexpr int COLS_OFF = STATS_OFF + NW * 2 * WM * 4;  // per-column epilogue constants: [wave][bias, gain, offset][64]
  static constexpr int COLS_STRIDE = 3 * 64;                    // floats per wave (a wave's bias load lands 64 of them)
  static constexpr int LDS_BYTES = COLS_OFF + NW * COLS_STRIDE * 4;
  static_assert(WN == 32 && LOADS == 4 && (NSTAGE - 2) * LOADS + 1 < 64, "wave shape; the counted waits fit the counter");
  static_assert(EPI_BYTES <= RING_BYTES && LDS_BYTES <= 160 * 1024, "LDS of a CU");
};
typedef DmamCfgT<128> DmamCfg;

// A bare barrier: the waits it needs are written out in front of it (a __syncthreads waits for every outstanding memory
// operation, i.e. for the slabs that are meant to stay in flight).
__device__ __forceinline__ void dmam_barrier() { asm volatile("s_barrier" ::: "memory"); }

// One 16-byte-per-lane load to LDS through a buffer descriptor. A function of its own on purpose: written inside a kernel
// template where an argument depends on a template parameter, this builtin makes the host pass drop the kernel's stub
// without a diagnostic (the library then fails to load over the unresolved name; the build checks for that).
__device__ __forceinline__ void dmam_load16(__amdgpu_buffer_rsrc_t r, uint8_t* dst, int voff, int soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)dst, 16, voff, soff, 0, 0);
}

// LEAN: the epilogue without its edge and type guards (gemm_epilogue's LEAN = 1; the launcher says when).
template <typename Cfg, int IN_DT, int OUT_DT, int LEAN>
__global__ void __launch_bounds__(Cfg::NT) gemm_dmam_kernel(const GemmArgs a, const DmafWalk wk) {
  constexpr int ESZ = IN_DT == DT_FP8 ? 1 : 2;                      // bytes per operand element
  constexpr int KSTEPS = Cfg::ROWB / (IN_DT == DT_FP8 ? 64 : 32);   // MFMA K steps per slab
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, LOADS = Cfg::LOADS, NSTAGE = Cfg::NSTAGE;
  constexpr int STAGE = BN * Cfg::ROWB;   // bytes of one operand's rows in one stage
  extern __shared__ __align__(16) uint8_t smem[];

  // (the wave index as a scalar: everything derived from it, LDS destinations and descriptors, stays in scalar registers)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % Cfg::WGM, wn = wave / Cfg::WGM;
  const int lr = lane & 31, g = lane >> 5;

  // Workgroup b runs on XCD b & 7, which owns a contiguous range of the row-major tile order.
  int pid = blockIdx.x;
  {
    const int per = gridDim.x >> 3;
    if (pid < (per << 3)) pid = (pid & 7) * per + (pid >> 3);
  }
  const int tile_m = dmaf_div(pid, wk.m_tn), tile_n = pid - tile_m * wk.tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int nslab = a.K * ESZ / Cfg::ROWB;  // the launcher sends only whole slabs of K here

  // Loader role: the first half of the waves fills the weight rows of a stage, the second half the activation rows,
  // ROWS_PER_WAVE consecutive rows each: 8 rows per wave-instruction, eight 16-byte chunks per row, the swizzle applied
  // on the global side (row r = rbase + 8 i + lane / 8 has swizzle lds_swizzle(r) = (lane / 8) ^ ((rbase / 8 + i) & 7)).
  const bool loads_a = wave >= Cfg::NW / 2;
  const int rbase = (wave & (Cfg::NW / 2 - 1)) * Cfg::ROWS_PER_WAVE;
  const int ld = (loads_a ? a.lda : a.ldw) * ESZ;   // row stride in bytes
  const int rows_left = loads_a ? a.M - m0 : a.N - n0;
  uint32_t voff[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    int r = rbase + 8 * i + (lane >> 3);
    r = r < rows_left ? r : rows_left - 1;
    voff[i] = (uint32_t)r * (uint32_t)ld + (((lane & 7) ^ (lane >> 3) ^ ((rbase / 8 + i) & 7)) << 4);
  }
  const long span = (long)(rows_left < BM ? rows_left : BM) * ld;
  const uint8_t* origin = loads_a ? reinterpret_cast<const uint8_t*>(a.A) + (long)m0 * a.lda * ESZ
                                  : reinterpret_cast<const uint8_t*>(a.W) + (long)n0 * a.ldw * ESZ;
  const __amdgpu_buffer_rsrc_t rsrc_mine = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(origin), 0, (int)(span < 0x7fffffffL ? span : 0x7fffffffL), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_none = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(a.A), 0, 0, 0x00020000);
  const uint32_t lds_load0 = (loads_a ? Cfg::PART_BYTES : 0) + rbase * Cfg::ROWB;   // stage 0
  auto issue_slab = [&](int slab) {
    const __amdgpu_buffer_rsrc_t r = slab < nslab ? rsrc_mine : rsrc_none;
    uint8_t* dst = smem + lds_load0 + (slab & (NSTAGE - 1)) * STAGE;
    static_for<0, LOADS>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      dmam_load16(r, dst + i * 1024, (int)voff[i], slab * Cfg::ROWB);
    });
  };
  // All slabs but one of the ring go out as early as their addresses exist.
#pragma unroll
  for (int s0 = 0; s0 < NSTAGE - 1; ++s0) issue_slab(s0);
  __builtin_amdgcn_sched_barrier(0);

  // The per-column constants of the epilogue for this wave's 32 columns (and the 32 behind them, which nothing reads), one column per lane, landed outside the ring. Columns past N repeat the last one; nothing of theirs is stored.
  if (a.bias) {
    int n = n0 + wn * Cfg::WN + lane;
    n = n < a.N ? n : a.N - 1;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a.bias + n),
                                     (__attribute__((address_space(3))) void*)(smem + Cfg::COLS_OFF + wave * (Cfg::COLS_STRIDE * 4)), 4, 0, 0);
  }
  const int extra_loads = a.bias ? 1 : 0;   // (issued behind the first slabs: the first wait allows for it)

  f32x16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Fragment addresses, as in gemm_dmaf_kernel.hpp: chunk Kc ^ L with L = (2g or g) ^ swizzle(lr) per lane and a
  // compile-time Kc that takes four values; four lane addresses per operand plus the immediate 4096 t.
  // (a 32-column wave may start at row 32 of the weight rows, whose swizzle differs from row 0's)
  const int LW = (IN_DT == DT_FP8 ? 2 * g : g) ^ lds_swizzle(wn * Cfg::WN + lr);
  const int LX = (IN_DT == DT_FP8 ? 2 * g : g) ^ lds_swizzle(wm * Cfg::WM + lr);
  const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)smem);
  uint32_t wb0[4], xb0[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int kc = IN_DT == DT_FP8 ? ((k & 1) | ((k >> 1) << 2)) : 2 * k;
    wb0[k] = lds0 + (wn * Cfg::WN + lr) * Cfg::ROWB + ((kc ^ LW) << 4);
    xb0[k] = lds0 + Cfg::PART_BYTES + (wm * Cfg::WM + lr) * Cfg::ROWB + ((kc ^ LX) << 4);
  }

  const bool wave_active = wave < Cfg::NCOMP && (m0 + wm * Cfg::WM < a.M) && (n0 + wn * Cfg::WN < a.N);

  for (int slab = 0; slab < nslab; ++slab) {
    // This wave's loads of the slab have landed; the NSTAGE - 2 slabs requested after it (and, the first time round, the
    // column constants) may stay in flight.
    if (slab == 0 && extra_loads) wait_vmcnt<(NSTAGE - 2) * LOADS + 1>();
    else wait_vmcnt<(NSTAGE - 2) * LOADS>();
    dmam_barrier();
    // Stage (slab - 1) % NSTAGE held slab - 1: every wave has finished with it before it reached this barrier.
    issue_slab(slab + NSTAGE - 1);
    if (!wave_active) continue;
    const uint32_t soff = (slab & (NSTAGE - 1)) * STAGE;
    auto read_piece = [&](bool is_w, int t, int ks, int half) -> i32x4_t {
      const int kc = (IN_DT == DT_FP8 ? 4 * ks + half : 2 * ks) ^ (4 * (t & 1));
      const int k = IN_DT == DT_FP8 ? ((kc & 1) | ((kc >> 2) << 1)) : kc >> 1;
      return *reinterpret_cast<const __attribute__((address_space(3))) i32x4_t*>((is_w ? wb0[k] : xb0[k]) + soff + t * 32 * Cfg::ROWB);
    };
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
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) acc[tn][tm] = mfma_frag<IN_DT>(wf[tn], xf[tm], acc[tn][tm]);
    });
  }

  wait_vmcnt<0>();
  dmam_barrier();  // every wave is done with the ring, and the empty loads past the end of K have retired
  if (wave >= Cfg::NCOMP) return;   // (a wave that only loads)

  gemm_epilogue<Cfg::WM, Cfg::WN, OUT_DT, 0, LEAN>(a, acc, reinterpret_cast<float*>(smem) + wave * (32 * Cfg::WN),
                                              m0 + wm * Cfg::WM, n0 + wn * Cfg::WN, lane, nullptr,
                                              reinterpret_cast<const float*>(smem + Cfg::COLS_OFF) + wave * Cfg::COLS_STRIDE);
}

template <int IN_DT, int OUT_DT, int LEAN = 0, typename Cfg = DmamCfg>
static hipError_t launch_dmam(const GemmArgs& a, hipStream_t st) {
  static std::atomic<bool> attr_set[16] = {};
  hipError_t e = hipSuccess;
  constexpr int ESZ = IN_DT == DT_FP8 ? 1 : 2;
  if ((a.K * ESZ) % DmamCfg::ROWB != 0 || a.K <= 0 || a.res_stats || (long)a.lda * ESZ * 128 >= (1L << 31) || (long)a.ldw * ESZ * 128 >= (1L << 31))
    return hipErrorInvalidValue;
  int dev = 0;
  (void)hipGetDevice(&dev);
  auto kern = gemm_dmam_kernel<Cfg, IN_DT, OUT_DT, LEAN>;
  if (!attr_set[dev]) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const int tiles_n = (a.N + Cfg::BN - 1) / Cfg::BN;
  const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * tiles_n;
  if (tiles >= 65536) return hipErrorInvalidValue;
  DmafWalk wk{};
  wk.tiles_n = tiles_n;
  wk.m_tn = dmaf_magic(tiles_n);
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(Cfg::NT), Cfg::LDS_BYTES, st, a, wk);
  return hipGetLastError();
}

}  // namespace crl
